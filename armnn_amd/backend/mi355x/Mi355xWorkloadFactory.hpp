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
    /// The Convolution2d workload THIS factory created last, while it has created no other workload that writes device
    /// tensors since: the one an Addition created next may take over (Mi355xAdditionWorkload::TakeOver).  A loaded network
    /// has a factory of its own and creates its workloads in execution order, so pairs never cross networks, whatever else
    /// the process loads meanwhile.  Shared with the convolution workload, which withdraws itself when it is destroyed.
    struct Candidate;
    std::shared_ptr<Candidate> m_Candidate;
};
} // namespace armnn
