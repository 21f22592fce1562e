// Workloads of the Mi355x backend.  Each one is the device counterpart of a CpuRef workload and does its GPU work through
// the C ABI only.  Convolution2d / DepthwiseConvolution2d / FullyConnected build their device plan (weights re-laid-out
// for the kernel, per-channel requantization constants) on the first Execute(), when the constant inputs have been
// produced -- the point at which RefConvolution2dWorkload::PostAllocationConfigure builds its decoders
// (src/backends/reference/workloads/RefConvolution2dWorkload.cpp:24-36).
#pragma once
#include "Mi355xDevice.hpp"

#include <armnn/backends/Workload.hpp>
#include <armnn/backends/WorkloadData.hpp>

#include <mutex>
#include <vector>

namespace armnn
{
/// the fused activation a layer carries as its "additional info" object, translated for the C ABI
struct Mi355xFusedActivation
{
    int32_t function = MI355X_ACT_NONE;
    float a = 0.0f, b = 0.0f;
    /// the descriptor was Mi355xFeedsOnlyAnAddition()
    bool feedsOnlyAnAddition = false;
    static Mi355xFusedActivation From(const ActivationDescriptor* descriptor);
};

/// The additional-info object of a Convolution2d whose output goes to one Addition of this backend and nowhere else:
/// Linear with slope 1 and offset 0, the identity, so a reader that applies it changes nothing.
ActivationDescriptor Mi355xFeedsOnlyAnAddition();

/// The additional-info object this backend's optimizer attaches to a DepthwiseConvolution2d whose output goes to one 1x1
/// Convolution2d of this backend and nowhere else: the fused activation (first member, so a reader that takes the object
/// for an ActivationDescriptor, as every workload does, reads exactly that) plus the mark.  Objects of this type are kept
/// in a registry while they live, so a workload can tell them from a plain ActivationDescriptor without touching memory
/// behind one.
struct Mi355xLayerNote
{
    ActivationDescriptor activation;
    bool onlyConsumerIsAPointwiseConvolution = false;
    /// on an unpadded 1x1 stride-1 Convolution2d: its output goes to one Pooling2d over the whole image and nowhere else
    bool onlyConsumerIsAGlobalPooling = false;

    /// a note as a layer's additional-info object; `activation` null: the identity (Mi355xFeedsOnlyAnAddition's descriptor)
    static std::shared_ptr<void> Make(const ActivationDescriptor* activation, bool onlyConsumerIsAPointwiseConvolution,
                                      bool onlyConsumerIsAGlobalPooling = false);
    /// the note behind a queue descriptor's additional-info pointer, or null if that is something else
    static const Mi355xLayerNote* From(const void* additionalInfo);
};

/// Every workload here reads its tensor handles when it executes, so the runtime may swap a handle for one that adopted
/// caller memory (pre-imported inputs and outputs; RefBaseWorkload, src/backends/reference/workloads/RefBaseWorkload.hpp:13-35).
template <typename QueueDescriptor>
class Mi355xBaseWorkload : public BaseWorkload<QueueDescriptor>
{
public:
    using BaseWorkload<QueueDescriptor>::BaseWorkload;
    bool SupportsTensorHandleReplacement() const override { return true; }
    void ReplaceInputTensorHandle(ITensorHandle* tensorHandle, unsigned int slot) override { this->m_Data.m_Inputs[slot] = tensorHandle; }
    void ReplaceOutputTensorHandle(ITensorHandle* tensorHandle, unsigned int slot) override { this->m_Data.m_Outputs[slot] = tensorHandle; }
};

/// counterpart of RefConvolution2dWorkload (RefConvolution2dWorkload.cpp:38-58)
class Mi355xConvolution2dWorkload : public Mi355xBaseWorkload<Convolution2dQueueDescriptor>
{
public:
    Mi355xConvolution2dWorkload(const Convolution2dQueueDescriptor& descriptor, const WorkloadInfo& info);
    ~Mi355xConvolution2dWorkload() override;
    void Execute() const override;
    /// kernel the plan resolved to; empty before the first Execute()
    std::string GetKernelDescription() const;
    /// the layer was marked Mi355xFeedsOnlyAnAddition()
    bool FeedsOnlyAnAddition() const { return m_FeedsOnlyAnAddition; }
    const ITensorHandle* GetOutputHandle() const { return m_Data.m_Outputs[0]; }
    /// From now on Execute() does nothing: the Addition that consumes this convolution calls ExecuteWithAddition() in its
    /// own Execute().
    void LeaveExecutionToTheAddition() { m_RunsInsideTheAddition = true; }
    bool RunsInsideTheAddition() const { return m_RunsInsideTheAddition; }
    /// `depthwise` was created just before this workload.  If it is marked as feeding one pointwise convolution only, writes
    /// the tensor this workload reads, and this is an unpadded 1x1 stride-1 convolution that no Addition runs, the two become a
    /// pair: the depthwise workload's Execute() does nothing from now on and this workload's Execute() runs both -- as one
    /// launch per lane where the device library recommends it for the two plans (mi355x_conv2d_fusion_pays) and the pair's
    /// output does not share memory with the pair's input, else one after the other.
    bool TakeOver(class Mi355xDepthwiseConvolution2dWorkload* depthwise);
    /// the depthwise workload of the pair is going away
    void ForgetDepthwise() { m_Depthwise = nullptr; }
    /// pairs formed / executions as one launch / executions as two launches since the process started (tests, benchmarks)
    static unsigned long long DepthwisePairsFormed();
    static unsigned long long DepthwisePairsRunFused();
    static unsigned long long DepthwisePairsRunApart();
    /// the layer was marked: its output goes to one Pooling2d over the whole image and nowhere else
    bool OnlyConsumerIsAGlobalPooling() const { return m_OnlyConsumerIsAGlobalPooling; }
    /// From now on Execute() does nothing: the Pooling2d that consumes this convolution calls ExecuteWithPooling() in its
    /// own Execute().
    void LeaveExecutionToThePooling() { m_RunsInsideThePooling = true; }
    /// This convolution and the pooling `pool` of its output as one launch per lane, writing `pooled` only -- where the device
    /// library takes and recommends the pair (mi355x_conv2d_pool_fusable, mi355x_conv2d_pool_fusion_pays), the input is
    /// 16-byte aligned and `pooled` shares no memory with it: returns true.  Otherwise executes this convolution as
    /// Execute() would have and returns false: the pooling is left to the caller.
    bool ExecuteWithPooling(const mi355x_pool2d_desc& pool, ITensorHandle* pooled, const TensorInfo& pooledInfo) const;
    /// convolution and Addition as one launch per lane: sum = activation(convolution(input) + other)
    void ExecuteWithAddition(const ITensorHandle* other, const TensorInfo& otherInfo, ITensorHandle* sum, const TensorInfo& sumInfo,
                             const Mi355xFusedActivation& activation) const;
private:
    void BuildPlan() const;
    void Run(void* y) const;
    void ExecuteOwn() const;
    WorkloadInfo m_Info;
    bool m_FeedsOnlyAnAddition = false;
    bool m_RunsInsideTheAddition = false;
    bool m_OnlyConsumerIsAGlobalPooling = false;
    bool m_RunsInsideThePooling = false;
    mutable int m_FusePool = -1;          // -1 not decided yet, 0 convolution and pooling run as two launches, 1 as one
    class Mi355xDepthwiseConvolution2dWorkload* m_Depthwise = nullptr;
    mutable int m_FusePair = -1;          // -1 not decided yet, 0 the pair runs as two launches, 1 as one
    mutable mi355x_conv2d_t m_Plan = nullptr;
    mutable std::once_flag m_Once;
};

/// counterpart of RefDepthwiseConvolution2dWorkload (RefDepthwiseConvolution2dWorkload.cpp:38-62)
class Mi355xDepthwiseConvolution2dWorkload : public Mi355xBaseWorkload<DepthwiseConvolution2dQueueDescriptor>
{
public:
    Mi355xDepthwiseConvolution2dWorkload(const DepthwiseConvolution2dQueueDescriptor& descriptor, const WorkloadInfo& info);
    ~Mi355xDepthwiseConvolution2dWorkload() override;
    void Execute() const override;
    /// the layer was marked: its output goes to one 1x1 Convolution2d of this backend and nowhere else
    bool OnlyConsumerIsAPointwiseConvolution() const { return m_OnlyConsumerIsAPointwise; }
    const ITensorHandle* GetOutputHandle() const { return m_Data.m_Outputs[0]; }
    const ITensorHandle* GetInputHandle() const { return m_Data.m_Inputs[0]; }
    const TensorInfo& GetInputInfo() const { return m_Info.m_InputTensorInfos[0]; }
    /// From now on Execute() does nothing: `pointwise`, the convolution that consumes this layer, runs it (see its TakeOver()).
    void LeaveExecutionTo(Mi355xConvolution2dWorkload* pointwise) { m_Pointwise = pointwise; }
    /// the convolution of the pair is going away: this workload runs itself again
    void ForgetPointwise() { m_Pointwise = nullptr; }
    /// the layer itself, whoever executes it
    void Run() const;
    /// the device plan (built on first use)
    mi355x_conv2d_t Plan() const;
private:
    void BuildPlan() const;
    WorkloadInfo m_Info;
    bool m_OnlyConsumerIsAPointwise = false;
    Mi355xConvolution2dWorkload* m_Pointwise = nullptr;
    mutable mi355x_conv2d_t m_Plan = nullptr;
    mutable std::once_flag m_Once;
};

/// counterpart of RefFullyConnectedWorkload (RefFullyConnectedWorkload.cpp:39-67)
class Mi355xFullyConnectedWorkload : public Mi355xBaseWorkload<FullyConnectedQueueDescriptor>
{
public:
    Mi355xFullyConnectedWorkload(const FullyConnectedQueueDescriptor& descriptor, const WorkloadInfo& info);
    ~Mi355xFullyConnectedWorkload() override;
    void Execute() const override;
private:
    void BuildPlan() const;
    WorkloadInfo m_Info;
    mutable mi355x_fc_t m_Plan = nullptr;
    mutable std::once_flag m_Once;
};

/// counterpart of RefActivationWorkload (RefActivationWorkload.cpp:23-36)
class Mi355xActivationWorkload : public Mi355xBaseWorkload<ActivationQueueDescriptor>
{
public:
    Mi355xActivationWorkload(const ActivationQueueDescriptor& descriptor, const WorkloadInfo& info);
    void Execute() const override;
private:
    WorkloadInfo m_Info;
};

/// counterpart of RefPooling2dWorkload (RefPooling2dWorkload.cpp:17-40)
class Mi355xPooling2dWorkload : public Mi355xBaseWorkload<Pooling2dQueueDescriptor>
{
public:
    Mi355xPooling2dWorkload(const Pooling2dQueueDescriptor& descriptor, const WorkloadInfo& info);
    void Execute() const override;
    /// `convolution` is the workload created directly before this one.  If it is marked as feeding one pooling over the whole
    /// image only and writes the tensor this workload reads, it leaves its execution to this workload, whose Execute() then
    /// runs both (Mi355xConvolution2dWorkload::ExecuteWithPooling).  Returns whether the pair was formed.  The convolution
    /// must outlive every Execute() of this workload (both belong to one loaded network).
    bool TakeOver(Mi355xConvolution2dWorkload* convolution);
    bool RunsAConvolution() const { return m_Convolution != nullptr; }
    /// pairs formed / executions as one launch / executions as two launches since the process started (tests, benchmarks)
    static unsigned long long PairsFormed();
    static unsigned long long PairsRunFused();
    static unsigned long long PairsRunApart();
private:
    mi355x_pool2d_desc Describe() const;
    WorkloadInfo m_Info;
    const Mi355xConvolution2dWorkload* m_Convolution = nullptr;
};

/// counterpart of RefMeanWorkload (RefMeanWorkload.cpp:26-42) for the mean over height and width of an NHWC tensor: the
/// float sum over the window in row order divided by the element count is what an average Pooling2d over the whole
/// feature map computes, and that kernel is what runs
class Mi355xMeanWorkload : public Mi355xBaseWorkload<MeanQueueDescriptor>
{
public:
    Mi355xMeanWorkload(const MeanQueueDescriptor& descriptor, const WorkloadInfo& info);
    void Execute() const override;
private:
    WorkloadInfo m_Info;
};

/// counterpart of RefPadWorkload (RefPadWorkload.cpp:18-40)
class Mi355xPadWorkload : public Mi355xBaseWorkload<PadQueueDescriptor>
{
public:
    Mi355xPadWorkload(const PadQueueDescriptor& descriptor, const WorkloadInfo& info);
    void Execute() const override;
private:
    WorkloadInfo m_Info;
};

/// counterpart of RefSoftmaxWorkload (RefSoftmaxWorkload.cpp:21-43)
class Mi355xSoftmaxWorkload : public Mi355xBaseWorkload<SoftmaxQueueDescriptor>
{
public:
    Mi355xSoftmaxWorkload(const SoftmaxQueueDescriptor& descriptor, const WorkloadInfo& info);
    void Execute() const override;
private:
    WorkloadInfo m_Info;
};

/// counterpart of RefElementwiseBinaryWorkload for BinaryOperation::Add (RefElementwiseBinaryWorkload.cpp:27-107)
class Mi355xAdditionWorkload : public Mi355xBaseWorkload<ElementwiseBinaryQueueDescriptor>
{
public:
    Mi355xAdditionWorkload(const ElementwiseBinaryQueueDescriptor& descriptor, const WorkloadInfo& info);
    void Execute() const override;
    /// `convolution` is the workload created directly before this one.  If it produces one of this Addition's inputs and
    /// nothing else reads that tensor, it leaves its execution to this workload, which then runs both as one launch.
    /// Nothing ran between the two, so every tensor the convolution reads is still intact when this workload executes;
    /// only this Addition's own output may have taken the place of the convolution's input, which Execute() checks.
    /// Returns whether the pair was formed.  The convolution must outlive every Execute() of this workload (both belong
    /// to one loaded network).
    bool TakeOver(Mi355xConvolution2dWorkload* convolution);
    bool RunsAConvolution() const { return m_Convolution != nullptr; }
    /// how many pairs this process has formed so far, and how many executions of a pair ran as two launches because the
    /// sum had been placed over the convolution's input (for tests and benchmarks)
    static unsigned long long PairsFormed();
    static unsigned long long PairsRunApart();
private:
    WorkloadInfo m_Info;
    const Mi355xConvolution2dWorkload* m_Convolution = nullptr;
    unsigned int m_OtherInput = 0;
};

/// counterpart of RefReshapeWorkload (RefReshapeWorkload.cpp:14-31): a device-to-device copy
class Mi355xReshapeWorkload : public Mi355xBaseWorkload<ReshapeQueueDescriptor>
{
public:
    Mi355xReshapeWorkload(const ReshapeQueueDescriptor& descriptor, const WorkloadInfo& info);
    void Execute() const override;
private:
    WorkloadInfo m_Info;
};

/// counterpart of RefConstantWorkload (RefConstantWorkload.cpp:22-47): uploads the layer's data once
class Mi355xConstantWorkload : public Mi355xBaseWorkload<ConstantQueueDescriptor>
{
public:
    Mi355xConstantWorkload(const ConstantQueueDescriptor& descriptor, const WorkloadInfo& info);
    void Execute() const override;
private:
    mutable bool m_RanOnce = false;
};
} // namespace armnn
