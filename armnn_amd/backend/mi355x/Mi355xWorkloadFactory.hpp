// IWorkloadFactory of the Mi355x backend (RefWorkloadFactory, src/backends/reference/RefWorkloadFactory.cpp:148-673, is
// the CpuRef counterpart): turns a queue descriptor into the device workload, or null for layer kinds the backend
// does not implement.
#pragma once
#include "Mi355xMemoryManager.hpp"

#include <armnn/backends/WorkloadFactory.hpp>

namespace armnn
{
class Mi355xWorkloadFactory : public IWorkloadFactory
{
public:
    explicit Mi355xWorkloadFactory(const std::shared_ptr<Mi355xMemoryManager>& memoryManager);
    Mi355xWorkloadFactory();

    const BackendId& GetBackendId() const override;
    static bool IsLayerSupported(const IConnectableLayer& layer, Optional<DataType> dataType, std::string& outReasonIfUnsupported);
    bool SupportsSubTensors() const override { return false; }
    std::unique_ptr<ITensorHandle> CreateSubTensorHandle(ITensorHandle&, TensorShape const&, unsigned int const*) const override { return nullptr; }
    std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& tensorInfo, const bool IsMemoryManaged = true) const override;
    std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& tensorInfo, DataLayout dataLayout, const bool IsMemoryManaged = true) const override;
    std::unique_ptr<IWorkload> CreateWorkload(LayerType type, const QueueDescriptor& descriptor, const WorkloadInfo& info) const override;
private:
    mutable std::shared_ptr<Mi355xMemoryManager> m_MemoryManager;
};
} // namespace armnn
