// Minimal host core: include/armnn/backends/ITensorHandleFactory.hpp:46-102.
#pragma once
#include "ITensorHandle.hpp"
#include <string>
#include <vector>

namespace armnn
{
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
} // namespace armnn
