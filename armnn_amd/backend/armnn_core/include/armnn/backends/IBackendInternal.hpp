// Minimal host core: include/armnn/backends/IBackendInternal.hpp:75-208.
#pragma once
#include "IBackendContext.hpp"
#include "ICustomAllocator.hpp"
#include "ILayerSupport.hpp"
#include "IMemoryManager.hpp"
#include "ITensorHandleFactory.hpp"
#include "OptimizationViews.hpp"
#include "SubgraphView.hpp"
#include "WorkloadFactory.hpp"
#include "../BackendOptions.hpp"
#include "../IRuntime.hpp"
#include "../Types.hpp"
#include <memory>
#include <vector>

namespace armnn
{
class TensorHandleFactoryRegistry;

struct BackendVersion
{
    uint32_t m_Major;
    uint32_t m_Minor;
    constexpr BackendVersion() : m_Major(0), m_Minor(0) {}
    constexpr BackendVersion(uint32_t major, uint32_t minor) : m_Major(major), m_Minor(minor) {}
    bool operator==(const BackendVersion& other) const { return m_Major == other.m_Major && m_Minor == other.m_Minor; }
    bool operator<=(const BackendVersion& other) const
    {
        return m_Major < other.m_Major || (m_Major == other.m_Major && m_Minor <= other.m_Minor);
    }
};

class IBackendInternal : public IBackend
{
protected:
    IBackendInternal() = default;
public:
    ~IBackendInternal() override = default;
    using IWorkloadFactoryPtr = std::unique_ptr<IWorkloadFactory>;
    using IBackendContextPtr = std::unique_ptr<IBackendContext>;
    using ILayerSupportSharedPtr = std::shared_ptr<ILayerSupport>;
    using IBackendSpecificModelContextPtr = std::shared_ptr<IBackendModelContext>;
    using IMemoryManagerUniquePtr = std::unique_ptr<IMemoryManager>;
    using IMemoryManagerSharedPtr = std::shared_ptr<IMemoryManager>;

    virtual IMemoryManagerUniquePtr CreateMemoryManager() const { return IMemoryManagerUniquePtr(); }
    virtual IWorkloadFactoryPtr CreateWorkloadFactory(const IMemoryManagerSharedPtr& memoryManager = nullptr) const = 0;
    virtual IWorkloadFactoryPtr CreateWorkloadFactory(TensorHandleFactoryRegistry& tensorHandleFactoryRegistry) const
    {
        IgnoreUnused(tensorHandleFactoryRegistry);
        return IWorkloadFactoryPtr{};
    }
    // A backend that is handed model options of its own must override the overloads that take them: the defaults answer
    // with nothing then (IBackendInternal.cpp:24-58, 88-102).
    virtual IWorkloadFactoryPtr CreateWorkloadFactory(const IMemoryManagerSharedPtr& memoryManager, const ModelOptions& modelOptions) const
    {
        if (NamesThisBackend(modelOptions)) return IWorkloadFactoryPtr{};
        return CreateWorkloadFactory(memoryManager);
    }
    virtual IWorkloadFactoryPtr CreateWorkloadFactory(TensorHandleFactoryRegistry& tensorHandleFactoryRegistry,
                                                      const ModelOptions& modelOptions) const
    {
        if (NamesThisBackend(modelOptions)) return IWorkloadFactoryPtr{};
        return CreateWorkloadFactory(tensorHandleFactoryRegistry);
    }
    virtual IWorkloadFactoryPtr CreateWorkloadFactory(TensorHandleFactoryRegistry& tensorHandleFactoryRegistry,
                                                      const ModelOptions& modelOptions, MemorySourceFlags inputFlags,
                                                      MemorySourceFlags outputFlags) const
    {
        IgnoreUnused(inputFlags, outputFlags);
        return CreateWorkloadFactory(tensorHandleFactoryRegistry, modelOptions);
    }
    /// may throw BackendUnavailableException: the runtime then leaves the backend out of its device spec
    virtual IBackendContextPtr CreateBackendContext(const IRuntime::CreationOptions&) const { return IBackendContextPtr{}; }
    virtual IBackendSpecificModelContextPtr CreateBackendSpecificModelContext(const ModelOptions&) const
    {
        return IBackendSpecificModelContextPtr{};
    }
    virtual ILayerSupportSharedPtr GetLayerSupport() const = 0;
    virtual ILayerSupportSharedPtr GetLayerSupport(const ModelOptions& modelOptions) const
    {
        if (NamesThisBackend(modelOptions)) return ILayerSupportSharedPtr{};
        return GetLayerSupport();
    }
    virtual OptimizationViews OptimizeSubgraphView(const SubgraphView& subgraph) const;
    virtual OptimizationViews OptimizeSubgraphView(const SubgraphView& subgraph, const ModelOptions& modelOptions) const
    {
        IgnoreUnused(modelOptions);
        return OptimizeSubgraphView(subgraph);
    }
    bool SupportsTensorAllocatorAPI() const { return !GetHandleFactoryPreferences().empty(); }
    virtual std::vector<ITensorHandleFactory::FactoryId> GetHandleFactoryPreferences() const
    {
        return std::vector<ITensorHandleFactory::FactoryId>();
    }
    virtual void RegisterTensorHandleFactories(TensorHandleFactoryRegistry& /*registry*/) {}
    virtual void RegisterTensorHandleFactories(TensorHandleFactoryRegistry& registry, MemorySourceFlags inputFlags,
                                               MemorySourceFlags outputFlags)
    {
        IgnoreUnused(inputFlags, outputFlags);
        RegisterTensorHandleFactories(registry);
    }
    static constexpr BackendVersion GetApiVersion() { return BackendVersion(1, 0); }
    virtual BackendCapabilities GetCapabilities() const { return BackendCapabilities("IBackendInternal NullCapabilities"); }
    /// the backend takes its memory from the caller's allocator from now on; false (with a reason) when it cannot
    virtual bool UseCustomMemoryAllocator(std::shared_ptr<ICustomAllocator> allocator, armnn::Optional<std::string&> errMsg)
    {
        IgnoreUnused(allocator);
        if (errMsg) errMsg.value() = "The backend " + GetId().Get() + " doesn't support using a custom allocator.";
        return false;
    }
    /// the allocator a caller-side memory plan uses for this backend's tensors when the caller named none
    virtual std::unique_ptr<ICustomAllocator> GetDefaultAllocator() const
    {
        throw armnn::Exception("GetDefaultAllocator: Function has not been implemented in backend.");
    }
    virtual unsigned int GetNumberOfCacheFiles() const { return 0; }
private:
    bool NamesThisBackend(const ModelOptions& modelOptions) const
    {
        for (const BackendOptions& group : modelOptions)
            if (group.GetBackendId() == GetId()) return true;
        return false;
    }
};
using IBackendInternalUniquePtr = std::unique_ptr<IBackendInternal>;
} // namespace armnn
