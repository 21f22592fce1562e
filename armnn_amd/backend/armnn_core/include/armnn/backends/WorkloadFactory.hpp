// Minimal host core: include/armnn/backends/WorkloadFactory.hpp:22-82.
#pragma once
#include "ITensorHandle.hpp"
#include "IWorkload.hpp"
#include "WorkloadData.hpp"
#include "WorkloadInfo.hpp"
#include "../BackendOptions.hpp"
#include "../INetwork.hpp"
#include "../Optional.hpp"
#include <memory>

namespace armnn
{
class IWorkloadFactory
{
public:
    virtual ~IWorkloadFactory() {}
    virtual void AfterWorkloadsCreated() {}
    virtual const BackendId& GetBackendId() const = 0;
    /// asks the backend's ILayerSupport with the tensor infos the layer would run with
    /// (src/backends/backendsCommon/WorkloadFactory.cpp:70-94 and the per-layer info lists of :258-291)
    static bool IsLayerSupported(const BackendId& backendId, const IConnectableLayer& layer, Optional<DataType> dataType,
                                 std::string& outReasonIfUnsupported, const ModelOptions& modelOptions = {});
    virtual bool SupportsSubTensors() const = 0;
    virtual std::unique_ptr<ITensorHandle> CreateSubTensorHandle(ITensorHandle& parent, TensorShape const& subTensorShape,
                                                                 unsigned int const* subTensorOrigin) const = 0;
    virtual std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& tensorInfo, const bool IsMemoryManaged = true) const = 0;
    virtual std::unique_ptr<ITensorHandle> CreateTensorHandle(const TensorInfo& tensorInfo, DataLayout dataLayout,
                                                              const bool IsMemoryManaged = true) const = 0;
    virtual std::unique_ptr<IWorkload> CreateWorkload(LayerType type, const QueueDescriptor& descriptor,
                                                      const WorkloadInfo& info) const = 0;
};
} // namespace armnn
