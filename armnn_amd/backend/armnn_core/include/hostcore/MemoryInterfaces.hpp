// Minimal host core: the memory side of the backend API, declared together because the pieces only make sense as a set --
// the per-network memory manager a backend hands out, the factory that creates its tensor handles, and the registry
// the optimizer and the loaded network look both up in.  Each class keeps the name, members and semantics Arm NN gives
// it (include/armnn/backends/IMemoryManager.hpp:12-22, include/armnn/backends/ITensorHandleFactory.hpp:46-102,
// src/backends/backendsCommon/TensorHandleFactoryRegistry.hpp:23-67); the Arm NN-named headers forward here.
#pragma once
#include <armnn/backends/ITensorHandle.hpp>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace armnn
{
// ---- lifetime-aware device memory of one loaded network: Acquire() before the first inference, Release() after ----
class IMemoryManager
{
protected:
    IMemoryManager() {}
public:
    virtual void Acquire() = 0;
    virtual void Release() = 0;
    virtual ~IMemoryManager() {}
};

// ---- creation of tensor handles, and what the optimizer may ask about them -----------------------------------------
class IConnectableLayer;
enum class CapabilityClass { PaddingRequired = 1, FallbackImportDisabled = 2, CapabilityClassMax = 254 };
struct Capability
{
    Capability(CapabilityClass c, bool v) : m_CapabilityClass(c), m_Value(v) {}
    CapabilityClass m_CapabilityClass;
    bool m_Value;
};

class ITensorHandleFactory
{
public:
    using FactoryId = std::string;
    static const FactoryId LegacyFactoryId;
    static const FactoryId DeferredFactoryId;
    virtual ~ITensorHandleFactory() {}
    virtual std::unique_ptr<ITensorHandle> CreateSubTensorHandle(ITensorHandle& parent, TensorShape const& subTensorShape,
                                                                 unsigned int const* subTensorOrigin) const = 0;
    virtual std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& tensorInfo) const = 0;
    virtual std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& tensorInfo, DataLayout dataLayout) const = 0;
    virtual std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& tensorInfo, const bool IsMemoryManaged) const
    {
        IgnoreUnused(IsMemoryManaged);
        return CreateTensorHandle(tensorInfo);
    }
    virtual std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& tensorInfo, DataLayout dataLayout,
                                                              const bool IsMemoryManaged) const
    {
        IgnoreUnused(IsMemoryManaged);
        return CreateTensorHandle(tensorInfo, dataLayout);
    }
    virtual const FactoryId& GetId() const = 0;
    virtual bool SupportsInPlaceComputation() const { return false; }
    virtual bool SupportsSubTensors() const = 0;
    virtual bool SupportsMapUnmap() const { return true; }
    virtual MemorySourceFlags GetExportFlags() const { return 0; }
    virtual MemorySourceFlags GetImportFlags() const { return 0; }
    virtual std::vector<Capability> GetCapabilities(const IConnectableLayer*, const IConnectableLayer*, CapabilityClass)
    {
        return std::vector<Capability>();
    }
};
enum class EdgeStrategy { Undefined, DirectCompatibility, ExportToTarget, CopyToTarget };

// ---- owner of every registered factory and memory manager --------------------------------------------------------
class TensorHandleFactoryRegistry
{
public:
    TensorHandleFactoryRegistry() = default;
    TensorHandleFactoryRegistry(const TensorHandleFactoryRegistry&) = delete;
    TensorHandleFactoryRegistry(TensorHandleFactoryRegistry&&) = delete;
    void RegisterFactory(std::unique_ptr<ITensorHandleFactory> allocator);
    void RegisterMemoryManager(std::shared_ptr<IMemoryManager> memoryManger);
    ITensorHandleFactory* GetFactory(ITensorHandleFactory::FactoryId id) const;
    void RegisterCopyAndImportFactoryPair(ITensorHandleFactory::FactoryId copyFactoryId, ITensorHandleFactory::FactoryId importFactoryId);
    ITensorHandleFactory::FactoryId GetMatchingImportFactoryId(ITensorHandleFactory::FactoryId copyFactoryId);
    void AquireMemory();
    void ReleaseMemory();
    std::vector<std::shared_ptr<IMemoryManager>>& GetMemoryManagers() { return m_MemoryManagers; }
private:
    std::vector<std::unique_ptr<ITensorHandleFactory>> m_Factories;
    std::vector<std::shared_ptr<IMemoryManager>> m_MemoryManagers;
    std::map<ITensorHandleFactory::FactoryId, ITensorHandleFactory::FactoryId> m_FactoryMappings;
};
} // namespace armnn
