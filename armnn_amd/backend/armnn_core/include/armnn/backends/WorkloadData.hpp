// Minimal host core: queue descriptors (include/armnn/backends/WorkloadData.hpp) for the layer kinds this core holds.
// Validate() enforces the rules of src/backends/backendsCommon/WorkloadData.cpp for the quantized conv / depthwise /
// fully-connected path (:180-205 bias quantization, :353-393 per-axis rules, :1036-1098, :1253-1328, :1392-1494).
#pragma once
#include "ITensorHandle.hpp"
#include "WorkloadInfo.hpp"
#include "../Descriptors.hpp"
#include <string>
#include <vector>

namespace armnn
{
class ConstTensorHandle;

struct QueueDescriptor
{
    std::vector<ITensorHandle*> m_Inputs;
    std::vector<ITensorHandle*> m_Outputs;
    void* m_AdditionalInfoObject;
    virtual ~QueueDescriptor() = default;
    void ValidateInputsOutputs(const std::string& descName, unsigned int numExpectedIn, unsigned int numExpectedOut) const;
    template <typename T>
    const T* GetAdditionalInformation() const { return static_cast<T*>(m_AdditionalInfoObject); }
    bool m_AllowExpandedDims = false;
protected:
    QueueDescriptor() : m_AdditionalInfoObject(nullptr) {}
    QueueDescriptor(QueueDescriptor const&) = default;
    QueueDescriptor& operator=(QueueDescriptor const&) = default;
};

template <typename LayerDescriptor>
struct QueueDescriptorWithParameters : public QueueDescriptor
{
    LayerDescriptor m_Parameters;
    virtual ~QueueDescriptorWithParameters() = default;
protected:
    QueueDescriptorWithParameters() = default;
    QueueDescriptorWithParameters(QueueDescriptorWithParameters const&) = default;
    QueueDescriptorWithParameters& operator=(QueueDescriptorWithParameters const&) = default;
};

struct MemCopyQueueDescriptor : QueueDescriptor { void Validate(const WorkloadInfo& workloadInfo) const; };
using InputQueueDescriptor = MemCopyQueueDescriptor;
using OutputQueueDescriptor = MemCopyQueueDescriptor;

struct ConstantQueueDescriptor : QueueDescriptor
{
    ConstantQueueDescriptor() : m_LayerOutput(nullptr) {}
    const ConstTensorHandle* m_LayerOutput;
    void Validate(const WorkloadInfo& workloadInfo) const;
};
struct ActivationQueueDescriptor : QueueDescriptorWithParameters<ActivationDescriptor> { void Validate(const WorkloadInfo&) const; };
struct Convolution2dQueueDescriptor : QueueDescriptorWithParameters<Convolution2dDescriptor> { void Validate(const WorkloadInfo&) const; };
struct DepthwiseConvolution2dQueueDescriptor : QueueDescriptorWithParameters<DepthwiseConvolution2dDescriptor> { void Validate(const WorkloadInfo&) const; };
struct FullyConnectedQueueDescriptor : QueueDescriptorWithParameters<FullyConnectedDescriptor> { void Validate(const WorkloadInfo&) const; };
struct Pooling2dQueueDescriptor : QueueDescriptorWithParameters<Pooling2dDescriptor> { void Validate(const WorkloadInfo&) const; };
struct MeanQueueDescriptor : QueueDescriptorWithParameters<MeanDescriptor> { void Validate(const WorkloadInfo&) const; };
struct PadQueueDescriptor : QueueDescriptorWithParameters<PadDescriptor> { void Validate(const WorkloadInfo&) const; };
struct SoftmaxQueueDescriptor : QueueDescriptorWithParameters<SoftmaxDescriptor> { void Validate(const WorkloadInfo&) const; };
struct ElementwiseBinaryQueueDescriptor : QueueDescriptorWithParameters<ElementwiseBinaryDescriptor> { void Validate(const WorkloadInfo&) const; };
struct ReshapeQueueDescriptor : QueueDescriptorWithParameters<ReshapeDescriptor> { void Validate(const WorkloadInfo&) const; };
} // namespace armnn
