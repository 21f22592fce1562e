#include "Mi355xWorkloads.hpp"
#include "Mi355xBackendId.hpp"
#include "Mi355xTensorHandle.hpp"
#include "Mi355xTimer.hpp"

#include <Profiling.hpp>

#include <armnn/backends/TensorHandle.hpp>
#include <armnn/utility/PolymorphicDowncast.hpp>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <set>
#include <cstring>

namespace armnn
{
namespace
{
// Device address of a workload operand.  Every operand of a workload this backend creates was made by this backend's
// tensor handle factory; anything else reaches it through a MemCopy layer.
const Mi355xTensorHandle& Dev(const ITensorHandle* h)
{
    const auto* d = dynamic_cast<const Mi355xTensorHandle*>(h);
    if (!d) throw InvalidArgumentException("Mi355x workload: operand is not a device tensor handle");
    return *d;
}
const void* In(const ITensorHandle* h) { return Dev(h).GetDevicePointerForRead(); }
void* Out(ITensorHandle* h)
{
    const Mi355xTensorHandle& d = Dev(h);
    d.MarkDeviceWritten();
    return d.GetDevicePointer();
}

std::atomic<unsigned long long> g_PairsFormed{0}, g_PairsRunApart{0};

// One slice of a batch and the stream it runs on.
struct Lane
{
    mi355x_stream_t stream;
    unsigned int index, count;
    /// this lane's part of a dense tensor whose outermost dimension is the batch
    const void* Of(const void* base, const TensorInfo& info) const { return static_cast<const unsigned char*>(base) + info.GetNumBytes() / count * index; }
    void* Of(void* base, const TensorInfo& info) const { return static_cast<unsigned char*>(base) + info.GetNumBytes() / count * index; }
};

// Calls `launch` once per lane when `batch` splits into lanes, else once for the whole batch on the joined stream.
// Operand addresses are taken before this (reading an adopted input may queue its transfer, lane by lane).
template <typename Launch>
void ForEachLane(unsigned int batch, Launch&& launch)
{
    const unsigned int lanes = mi355x::LanesFor(batch);
    if (lanes == 1)
    {
        launch(Lane{mi355x::Stream(), 0u, 1u});
        return;
    }
    mi355x::Fork();
    for (unsigned int k = 0; k < lanes; ++k) launch(Lane{mi355x::LaneStream(k), k, lanes});
}

// batch of a tensor that has one: the outermost of at least two dimensions
unsigned int BatchOf(const TensorInfo& info) { return info.GetNumDimensions() >= 2 ? info.GetShape()[0] : 1u; }

// the kernel a plan resolved to, for the profiler's details record
std::string Describe(mi355x_conv2d_t plan)
{
    int32_t algo = 0;
    char buf[256] = {0};
    return mi355x_conv2d_algo(plan, &algo, buf, sizeof(buf)) == 0 ? std::string(buf) : std::string();
}
std::string Describe(mi355x_fc_t plan)
{
    int32_t algo = 0;
    char buf[256] = {0};
    return mi355x_fc_algo(plan, &algo, buf, sizeof(buf)) == 0 ? std::string(buf) : std::string();
}

// Host copy of a constant operand plus its quantization in C-ABI form.  The copy is taken through Map(), so it
// works for any handle type a constant may arrive in.
struct HostConstant
{
    std::vector<unsigned char> data;
    std::vector<float> scales;
    mi355x_const_quant quant{};

    HostConstant(const ITensorHandle* handle, const TensorInfo& info)
    {
        data.resize(info.GetNumBytes());
        const void* p = handle->Map(true);
        if (!p) throw NullPointerException("Mi355x workload: constant operand has no data");
        std::memcpy(data.data(), p, data.size());
        handle->Unmap();
        scales = info.GetQuantizationScales();
        if (scales.empty()) scales.push_back(1.0f);
        quant.dtype = mi355x::ToDType(info.GetDataType());
        quant.offset = info.GetQuantizationOffset();
        quant.n_scales = static_cast<uint32_t>(scales.size());
        quant.scales = scales.data();
    }
};
} // namespace

Mi355xFusedActivation Mi355xFusedActivation::From(const ActivationDescriptor* d)
{
    Mi355xFusedActivation f;
    if (!d) return f;
    switch (d->m_Function)
    {
        case ActivationFunction::ReLu: f.function = MI355X_ACT_RELU; break;
        case ActivationFunction::BoundedReLu: f.function = MI355X_ACT_BOUNDED_RELU; f.a = d->m_A; f.b = d->m_B; break;
        case ActivationFunction::Linear:
            if (d->m_A == 1.0f && d->m_B == 0.0f) { f.feedsOnlyAnAddition = true; break; }
            throw InvalidArgumentException("Mi355x: only ReLu / BoundedReLu can be fused into a layer");
        default: throw InvalidArgumentException("Mi355x: only ReLu / BoundedReLu can be fused into a layer");
    }
    return f;
}

ActivationDescriptor Mi355xFeedsOnlyAnAddition()
{
    ActivationDescriptor d;
    d.m_Function = ActivationFunction::Linear;
    d.m_A = 1.0f;
    d.m_B = 0.0f;
    return d;
}

// ---- the note on a depthwise layer ---------------------------------------------------------------------------------------
namespace
{
std::mutex g_NotesMutex;
std::set<const void*> g_Notes;
std::atomic<unsigned long long> g_DepthwisePairsFormed{0}, g_DepthwisePairsRunFused{0}, g_DepthwisePairsRunApart{0};
std::atomic<unsigned long long> g_PoolingPairsFormed{0}, g_PoolingPairsRunFused{0}, g_PoolingPairsRunApart{0};
}

std::shared_ptr<void> Mi355xLayerNote::Make(const ActivationDescriptor* activation, bool onlyConsumerIsAPointwiseConvolution,
                                            bool onlyConsumerIsAGlobalPooling)
{
    auto* note = new Mi355xLayerNote;
    note->activation = activation ? *activation : Mi355xFeedsOnlyAnAddition();
    note->onlyConsumerIsAPointwiseConvolution = onlyConsumerIsAPointwiseConvolution;
    note->onlyConsumerIsAGlobalPooling = onlyConsumerIsAGlobalPooling;
    {
        std::lock_guard<std::mutex> lock(g_NotesMutex);
        g_Notes.insert(note);
    }
    return std::shared_ptr<void>(note, [](void* p) {
        {
            std::lock_guard<std::mutex> lock(g_NotesMutex);
            g_Notes.erase(p);
        }
        delete static_cast<Mi355xLayerNote*>(p);
    });
}

const Mi355xLayerNote* Mi355xLayerNote::From(const void* additionalInfo)
{
    if (!additionalInfo) return nullptr;
    std::lock_guard<std::mutex> lock(g_NotesMutex);
    return g_Notes.count(additionalInfo) ? static_cast<const Mi355xLayerNote*>(additionalInfo) : nullptr;
}

// ---- Convolution2d ---------------------------------------------------------------------------------------------------
Mi355xConvolution2dWorkload::Mi355xConvolution2dWorkload(const Convolution2dQueueDescriptor& descriptor, const WorkloadInfo& info)
    : Mi355xBaseWorkload<Convolution2dQueueDescriptor>(descriptor, info), m_Info(info)
{
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Mi355xConvolution2dWorkload_Construct", descriptor.m_Parameters, info, this->GetGuid());
    if (m_Data.m_Parameters.m_DataLayout != DataLayout::NHWC) throw InvalidArgumentException("Mi355xConvolution2dWorkload: NHWC only");
    m_FeedsOnlyAnAddition = Mi355xFusedActivation::From(m_Data.GetAdditionalInformation<ActivationDescriptor>()).feedsOnlyAnAddition;   // validates early
    if (const Mi355xLayerNote* note = Mi355xLayerNote::From(m_Data.m_AdditionalInfoObject))
        if (note->onlyConsumerIsAGlobalPooling)
        {
            // a note without an activation carries the identity, which is also how a plain descriptor marks "feeds an Addition"
            m_OnlyConsumerIsAGlobalPooling = true;
            m_FeedsOnlyAnAddition = false;
        }
}

Mi355xConvolution2dWorkload::~Mi355xConvolution2dWorkload()
{
    if (m_Depthwise) m_Depthwise->ForgetPointwise();
    if (m_Plan) mi355x_conv2d_destroy(m_Plan);
}

unsigned long long Mi355xConvolution2dWorkload::DepthwisePairsFormed() { return g_DepthwisePairsFormed.load(); }
unsigned long long Mi355xConvolution2dWorkload::DepthwisePairsRunFused() { return g_DepthwisePairsRunFused.load(); }
unsigned long long Mi355xConvolution2dWorkload::DepthwisePairsRunApart() { return g_DepthwisePairsRunApart.load(); }

bool Mi355xConvolution2dWorkload::TakeOver(Mi355xDepthwiseConvolution2dWorkload* depthwise)
{
    if (!depthwise || m_Depthwise || m_FeedsOnlyAnAddition || !depthwise->OnlyConsumerIsAPointwiseConvolution()) return false;
    if (depthwise->GetOutputHandle() == nullptr || depthwise->GetOutputHandle() != m_Data.m_Inputs[0]) return false;
    const Convolution2dDescriptor& p = m_Data.m_Parameters;
    const TensorShape& w = m_Info.m_InputTensorInfos[1].GetShape();
    if (w[1] != 1 || w[2] != 1 || p.m_StrideX != 1 || p.m_StrideY != 1 || p.m_PadLeft || p.m_PadRight || p.m_PadTop || p.m_PadBottom) return false;
    m_Depthwise = depthwise;
    depthwise->LeaveExecutionTo(this);
    g_DepthwisePairsFormed.fetch_add(1);
    return true;
}

void Mi355xConvolution2dWorkload::BuildPlan() const
{
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const TensorInfo& w = m_Info.m_InputTensorInfos[1];
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const Convolution2dDescriptor& p = m_Data.m_Parameters;
    const Mi355xFusedActivation act = Mi355xFusedActivation::From(m_Data.GetAdditionalInformation<ActivationDescriptor>());

    mi355x_conv2d_desc d{};
    d.in_h = in.GetShape()[1]; d.in_w = in.GetShape()[2]; d.in_c = in.GetShape()[3];
    d.out_h = out.GetShape()[1]; d.out_w = out.GetShape()[2]; d.out_c = out.GetShape()[3];
    d.kernel_h = w.GetShape()[1]; d.kernel_w = w.GetShape()[2];
    d.pad_top = p.m_PadTop; d.pad_left = p.m_PadLeft;
    d.stride_x = p.m_StrideX; d.stride_y = p.m_StrideY;
    d.dilation_x = p.m_DilationX; d.dilation_y = p.m_DilationY;
    d.depthwise = 0;
    d.bias_enabled = p.m_BiasEnabled ? 1u : 0u;
    d.input = mi355x::ToQuant(in);
    d.output = mi355x::ToQuant(out);
    d.activation = act.function; d.activation_a = act.a; d.activation_b = act.b;
    d.algo = MI355X_ALGO_AUTO;

    HostConstant weights(m_Data.m_Inputs[1], w);
    std::unique_ptr<HostConstant> bias;
    if (p.m_BiasEnabled) bias = std::make_unique<HostConstant>(m_Data.m_Inputs[2], m_Info.m_InputTensorInfos[2]);
    mi355x::EnsureDevice();
    mi355x::Check(mi355x_conv2d_create(&d, weights.data.data(), &weights.quant,
                                       bias ? reinterpret_cast<const int32_t*>(bias->data.data()) : nullptr,
                                       bias ? &bias->quant : nullptr, &m_Plan),
                  "mi355x_conv2d_create");
    // the batch runs as this many slices side by side (Execute() asks the same question for every launch)
    mi355x::Check(mi355x_conv2d_set_concurrency(m_Plan, mi355x::LanesFor(in.GetShape()[0])), "mi355x_conv2d_set_concurrency");
    WorkloadInfo details = m_Info;
    details.m_ConvolutionMethod = Optional<std::string>(Describe(m_Plan));
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Mi355xConvolution2dWorkload_Plan", m_Data.m_Parameters, details, this->GetGuid());
}

void Mi355xConvolution2dWorkload::Execute() const
{
    if (m_RunsInsideTheAddition || m_RunsInsideThePooling) return;
    ARMNN_SCOPED_PROFILING_EVENT_MI355X_NAME_GUID("Mi355xConvolution2dWorkload_Execute");
    ExecuteOwn();
}

bool Mi355xConvolution2dWorkload::ExecuteWithPooling(const mi355x_pool2d_desc& pool, ITensorHandle* pooled, const TensorInfo& pooledInfo) const
{
    // (no profiling event of its own: the pooling workload's event covers the pair, as an Addition's covers its convolution)
    std::call_once(m_Once, [this] { BuildPlan(); });
    if (!m_Plan) throw RuntimeException("Mi355xConvolution2dWorkload: no device plan (its creation failed earlier)");
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const uint32_t batch = in.GetShape()[0];
    if (m_FusePool < 0)
        m_FusePool = mi355x_conv2d_pool_fusable(m_Plan, &pool) == 0 &&
                     mi355x_conv2d_pool_fusion_pays(m_Plan, &pool, batch / mi355x::LanesFor(batch)) == 1 ? 1 : 0;
    const unsigned char* x = static_cast<const unsigned char*>(In(m_Data.m_Inputs[0]));
    unsigned char* y = static_cast<unsigned char*>(Out(pooled));
    // as with the other pairs: the pooled tensor may have been placed where the convolution's input lies
    const bool overlap = x < y + pooledInfo.GetNumBytes() && y < x + in.GetNumBytes();
    const bool aligned = (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    if (m_FusePool != 1 || overlap || !aligned)
    {
        g_PoolingPairsRunApart.fetch_add(1);
        ExecuteOwn();
        return false;
    }
    // the depthwise layer in front of this convolution, if it left its execution to this workload, runs first as it is:
    // the pair (depthwise, this convolution) as one launch would write the tensor the pooling then had to read again
    if (m_Depthwise) m_Depthwise->Run();
    g_PoolingPairsRunFused.fetch_add(1);
    ForEachLane(batch, [&](const Lane& l) {
        mi355x::Check(mi355x_conv2d_run_pooled(m_Plan, &pool, batch / l.count, l.Of(static_cast<const void*>(x), in),
                                               l.Of(static_cast<void*>(y), pooledInfo), l.stream), "mi355x_conv2d_run_pooled");
    });
    return true;
}

void Mi355xConvolution2dWorkload::ExecuteOwn() const
{
    if (m_Depthwise)
    {
        // the pair: the depthwise layer in front of this convolution has left its execution to this workload
        std::call_once(m_Once, [this] { BuildPlan(); });
        if (!m_Plan) throw RuntimeException("Mi355xConvolution2dWorkload: no device plan (its creation failed earlier)");
        const mi355x_conv2d_t first = m_Depthwise->Plan();
        const TensorInfo& in = m_Depthwise->GetInputInfo();
        const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
        const uint32_t batch = in.GetShape()[0];
        if (m_FusePair < 0)
            m_FusePair = mi355x_conv2d_fusable(first, m_Plan) == 0 &&
                         mi355x_conv2d_fusion_pays(first, m_Plan, batch / mi355x::LanesFor(batch)) == 1 ? 1 : 0;
        const unsigned char* x = static_cast<const unsigned char*>(In(m_Depthwise->GetInputHandle()));
        unsigned char* y = static_cast<unsigned char*>(Out(m_Data.m_Outputs[0]));
        // The pair's output began its life after the pair's input ended its own, so a memory manager that shares addresses may
        // have put the one where the other is; one launch that reads and writes the same range would race.  The fused
        // kernels also want 16-byte aligned tensors.
        const bool overlap = x < y + out.GetNumBytes() && y < x + in.GetNumBytes();
        const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
        if (m_FusePair == 1 && !overlap && aligned)
        {
            g_DepthwisePairsRunFused.fetch_add(1);
            ForEachLane(batch, [&](const Lane& l) {
                mi355x::Check(mi355x_conv2d_run_fused(first, m_Plan, batch / l.count, l.Of(static_cast<const void*>(x), in),
                                                      l.Of(static_cast<void*>(y), out), l.stream), "mi355x_conv2d_run_fused");
            });
            return;
        }
        g_DepthwisePairsRunApart.fetch_add(1);
        m_Depthwise->Run();
    }
    Run(Out(m_Data.m_Outputs[0]));
}

void Mi355xConvolution2dWorkload::Run(void* y) const
{
    std::call_once(m_Once, [this] { BuildPlan(); });
    if (!m_Plan) throw RuntimeException("Mi355xConvolution2dWorkload: no device plan (its creation failed earlier)");
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const uint32_t batch = in.GetShape()[0];
    const void* x = In(m_Data.m_Inputs[0]);
    ForEachLane(batch, [&](const Lane& l) {
        mi355x::Check(mi355x_conv2d_run(m_Plan, batch / l.count, l.Of(x, in), l.Of(y, out), l.stream), "mi355x_conv2d_run");
    });
}

void Mi355xConvolution2dWorkload::ExecuteWithAddition(const ITensorHandle* other, const TensorInfo& otherInfo, ITensorHandle* sum,
                                                      const TensorInfo& sumInfo, const Mi355xFusedActivation& activation) const
{
    std::call_once(m_Once, [this] { BuildPlan(); });
    if (!m_Plan) throw RuntimeException("Mi355xConvolution2dWorkload: no device plan (its creation failed earlier)");
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const uint32_t batch = in.GetShape()[0];
    const mi355x_quant qOther = mi355x::ToQuant(otherInfo);
    const mi355x_quant qSum = mi355x::ToQuant(sumInfo);
    const mi355x_quant qOwn = mi355x::ToQuant(out);
    const unsigned char* x = static_cast<const unsigned char*>(In(m_Data.m_Inputs[0]));
    const void* r = In(other);
    unsigned char* y = static_cast<unsigned char*>(Out(sum));
    // The sum's tensor began its life after the convolution's input ended its own, so a memory manager that shares
    // addresses may have put the one where the other is.  One launch that reads and writes the same range would race:
    // then the convolution writes its own output first (that tensor lives until the Addition has run).
    const bool overlap = x < y + sumInfo.GetNumBytes() && y < x + in.GetNumBytes();
    if (overlap)
    {
        g_PairsRunApart.fetch_add(1);
        void* own = Out(m_Data.m_Outputs[0]);
        ForEachLane(batch, [&](const Lane& l) {
            mi355x::Check(mi355x_conv2d_run(m_Plan, batch / l.count, l.Of(static_cast<const void*>(x), in), l.Of(own, out), l.stream), "mi355x_conv2d_run");
            mi355x::Check(mi355x_add_run(out.GetNumElements() / l.count, &qOwn, &qOther, &qSum, activation.function, activation.a, activation.b,
                                         l.Of(static_cast<const void*>(own), out), l.Of(r, otherInfo), l.Of(static_cast<void*>(y), sumInfo), l.stream),
                          "mi355x_add_run");
        });
        return;
    }
    ForEachLane(batch, [&](const Lane& l) {
        mi355x::Check(mi355x_conv2d_run_add(m_Plan, batch / l.count, l.Of(static_cast<const void*>(x), in), l.Of(r, otherInfo), &qOther, &qSum,
                                            activation.function, activation.a, activation.b, l.Of(static_cast<void*>(y), sumInfo), l.stream),
                      "mi355x_conv2d_run_add");
    });
}

std::string Mi355xConvolution2dWorkload::GetKernelDescription() const
{
    if (!m_Plan) return std::string();
    int32_t algo = 0;
    char buf[256] = {0};
    mi355x_conv2d_algo(m_Plan, &algo, buf, sizeof(buf));
    return buf;
}

// ---- DepthwiseConvolution2d ------------------------------------------------------------------------------------------
Mi355xDepthwiseConvolution2dWorkload::Mi355xDepthwiseConvolution2dWorkload(const DepthwiseConvolution2dQueueDescriptor& descriptor, const WorkloadInfo& info)
    : Mi355xBaseWorkload<DepthwiseConvolution2dQueueDescriptor>(descriptor, info), m_Info(info)
{
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Mi355xDepthwiseConvolution2dWorkload_Construct", descriptor.m_Parameters, info, this->GetGuid());
    if (m_Data.m_Parameters.m_DataLayout != DataLayout::NHWC) throw InvalidArgumentException("Mi355xDepthwiseConvolution2dWorkload: NHWC only");
    Mi355xFusedActivation::From(m_Data.GetAdditionalInformation<ActivationDescriptor>());
    if (const Mi355xLayerNote* note = Mi355xLayerNote::From(m_Data.m_AdditionalInfoObject)) m_OnlyConsumerIsAPointwise = note->onlyConsumerIsAPointwiseConvolution;
}

Mi355xDepthwiseConvolution2dWorkload::~Mi355xDepthwiseConvolution2dWorkload()
{
    if (m_Pointwise) m_Pointwise->ForgetDepthwise();
    if (m_Plan) mi355x_conv2d_destroy(m_Plan);
}

mi355x_conv2d_t Mi355xDepthwiseConvolution2dWorkload::Plan() const
{
    std::call_once(m_Once, [this] { BuildPlan(); });
    if (!m_Plan) throw RuntimeException("Mi355xDepthwiseConvolution2dWorkload: no device plan (its creation failed earlier)");
    return m_Plan;
}

void Mi355xDepthwiseConvolution2dWorkload::BuildPlan() const
{
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const TensorInfo& w = m_Info.m_InputTensorInfos[1];   // [1, H, W, O]
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const DepthwiseConvolution2dDescriptor& p = m_Data.m_Parameters;
    const Mi355xFusedActivation act = Mi355xFusedActivation::From(m_Data.GetAdditionalInformation<ActivationDescriptor>());

    mi355x_conv2d_desc d{};
    d.in_h = in.GetShape()[1]; d.in_w = in.GetShape()[2]; d.in_c = in.GetShape()[3];
    d.out_h = out.GetShape()[1]; d.out_w = out.GetShape()[2]; d.out_c = out.GetShape()[3];
    d.kernel_h = w.GetShape()[1]; d.kernel_w = w.GetShape()[2];
    d.pad_top = p.m_PadTop; d.pad_left = p.m_PadLeft;
    d.stride_x = p.m_StrideX; d.stride_y = p.m_StrideY;
    d.dilation_x = p.m_DilationX; d.dilation_y = p.m_DilationY;
    d.depthwise = 1;
    d.bias_enabled = p.m_BiasEnabled ? 1u : 0u;
    d.input = mi355x::ToQuant(in);
    d.output = mi355x::ToQuant(out);
    d.activation = act.function; d.activation_a = act.a; d.activation_b = act.b;
    d.algo = MI355X_ALGO_AUTO;

    HostConstant weights(m_Data.m_Inputs[1], w);
    std::unique_ptr<HostConstant> bias;
    if (p.m_BiasEnabled) bias = std::make_unique<HostConstant>(m_Data.m_Inputs[2], m_Info.m_InputTensorInfos[2]);
    mi355x::EnsureDevice();
    mi355x::Check(mi355x_conv2d_create(&d, weights.data.data(), &weights.quant,
                                       bias ? reinterpret_cast<const int32_t*>(bias->data.data()) : nullptr,
                                       bias ? &bias->quant : nullptr, &m_Plan),
                  "mi355x_conv2d_create(depthwise)");
    WorkloadInfo details = m_Info;
    details.m_ConvolutionMethod = Optional<std::string>(Describe(m_Plan));
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Mi355xDepthwiseConvolution2dWorkload_Plan", m_Data.m_Parameters, details, this->GetGuid());
}

void Mi355xDepthwiseConvolution2dWorkload::Execute() const
{
    if (m_Pointwise) return;              // the pointwise convolution behind this layer runs the pair
    ARMNN_SCOPED_PROFILING_EVENT_MI355X_NAME_GUID("Mi355xDepthwiseConvolution2dWorkload_Execute");
    Run();
}

void Mi355xDepthwiseConvolution2dWorkload::Run() const
{
    Plan();
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const uint32_t batch = in.GetShape()[0];
    const void* x = In(m_Data.m_Inputs[0]);
    void* y = Out(m_Data.m_Outputs[0]);
    ForEachLane(batch, [&](const Lane& l) {
        mi355x::Check(mi355x_conv2d_run(m_Plan, batch / l.count, l.Of(x, in), l.Of(y, out), l.stream), "mi355x_conv2d_run(depthwise)");
    });
}

// ---- FullyConnected --------------------------------------------------------------------------------------------------
Mi355xFullyConnectedWorkload::Mi355xFullyConnectedWorkload(const FullyConnectedQueueDescriptor& descriptor, const WorkloadInfo& info)
    : Mi355xBaseWorkload<FullyConnectedQueueDescriptor>(descriptor, info), m_Info(info)
{
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Mi355xFullyConnectedWorkload_Construct", descriptor.m_Parameters, info, this->GetGuid());
    Mi355xFusedActivation::From(m_Data.GetAdditionalInformation<ActivationDescriptor>());
}

Mi355xFullyConnectedWorkload::~Mi355xFullyConnectedWorkload()
{
    if (m_Plan) mi355x_fc_destroy(m_Plan);
}

void Mi355xFullyConnectedWorkload::BuildPlan() const
{
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const TensorInfo& w = m_Info.m_InputTensorInfos[1];
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const FullyConnectedDescriptor& p = m_Data.m_Parameters;
    const Mi355xFusedActivation act = Mi355xFusedActivation::From(m_Data.GetAdditionalInformation<ActivationDescriptor>());

    mi355x_fc_desc d{};
    d.k = in.GetNumElements() / in.GetShape()[0];       // GetNumActivations, RefFullyConnectedWorkload.cpp:16-24
    d.out_features = out.GetShape()[1];
    d.transpose_weights = p.m_TransposeWeightMatrix ? 1u : 0u;
    d.bias_enabled = p.m_BiasEnabled ? 1u : 0u;
    d.input = mi355x::ToQuant(in);
    d.output = mi355x::ToQuant(out);
    d.activation = act.function; d.activation_a = act.a; d.activation_b = act.b;
    d.algo = MI355X_ALGO_AUTO;

    HostConstant weights(m_Data.m_Inputs[1], w);
    std::unique_ptr<HostConstant> bias;
    if (p.m_BiasEnabled) bias = std::make_unique<HostConstant>(m_Data.m_Inputs[2], m_Info.m_InputTensorInfos[2]);
    mi355x::EnsureDevice();
    mi355x::Check(mi355x_fc_create(&d, weights.data.data(), &weights.quant,
                                   bias ? reinterpret_cast<const int32_t*>(bias->data.data()) : nullptr,
                                   bias ? &bias->quant : nullptr, &m_Plan),
                  "mi355x_fc_create");
    WorkloadInfo details = m_Info;
    details.m_ConvolutionMethod = Optional<std::string>(Describe(m_Plan));
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Mi355xFullyConnectedWorkload_Plan", m_Data.m_Parameters, details, this->GetGuid());
}

void Mi355xFullyConnectedWorkload::Execute() const
{
    ARMNN_SCOPED_PROFILING_EVENT_MI355X_NAME_GUID("Mi355xFullyConnectedWorkload_Execute");
    std::call_once(m_Once, [this] { BuildPlan(); });
    if (!m_Plan) throw RuntimeException("Mi355xFullyConnectedWorkload: no device plan (its creation failed earlier)");
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const uint32_t batch = in.GetShape()[0];
    const void* x = In(m_Data.m_Inputs[0]);
    void* y = Out(m_Data.m_Outputs[0]);
    ForEachLane(batch, [&](const Lane& l) {
        mi355x::Check(mi355x_fc_run(m_Plan, batch / l.count, l.Of(x, in), l.Of(y, out), l.stream), "mi355x_fc_run");
    });
}

// ---- Activation ------------------------------------------------------------------------------------------------------
Mi355xActivationWorkload::Mi355xActivationWorkload(const ActivationQueueDescriptor& descriptor, const WorkloadInfo& info)
    : Mi355xBaseWorkload<ActivationQueueDescriptor>(descriptor, info), m_Info(info)
{
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Mi355xActivationWorkload_Construct", descriptor.m_Parameters, info, this->GetGuid());
    Mi355xFusedActivation::From(&m_Data.m_Parameters);
}

void Mi355xActivationWorkload::Execute() const
{
    ARMNN_SCOPED_PROFILING_EVENT_MI355X_NAME_GUID("Mi355xActivationWorkload_Execute");
    const Mi355xFusedActivation act = Mi355xFusedActivation::From(&m_Data.m_Parameters);
    const mi355x_quant qi = mi355x::ToQuant(m_Info.m_InputTensorInfos[0]);
    const mi355x_quant qo = mi355x::ToQuant(m_Info.m_OutputTensorInfos[0]);
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const void* x = In(m_Data.m_Inputs[0]);
    void* y = Out(m_Data.m_Outputs[0]);
    ForEachLane(BatchOf(in), [&](const Lane& l) {
        mi355x::Check(mi355x_activation_run(in.GetNumElements() / l.count, &qi, &qo, act.function, act.a, act.b, l.Of(x, in), l.Of(y, out), l.stream),
                      "mi355x_activation_run");
    });
}

// ---- Pooling2d -------------------------------------------------------------------------------------------------------
Mi355xPooling2dWorkload::Mi355xPooling2dWorkload(const Pooling2dQueueDescriptor& descriptor, const WorkloadInfo& info)
    : Mi355xBaseWorkload<Pooling2dQueueDescriptor>(descriptor, info), m_Info(info)
{
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Mi355xPooling2dWorkload_Construct", descriptor.m_Parameters, info, this->GetGuid());
    if (m_Data.m_Parameters.m_DataLayout != DataLayout::NHWC) throw InvalidArgumentException("Mi355xPooling2dWorkload: NHWC only");
}

unsigned long long Mi355xPooling2dWorkload::PairsFormed() { return g_PoolingPairsFormed.load(); }
unsigned long long Mi355xPooling2dWorkload::PairsRunFused() { return g_PoolingPairsRunFused.load(); }
unsigned long long Mi355xPooling2dWorkload::PairsRunApart() { return g_PoolingPairsRunApart.load(); }

bool Mi355xPooling2dWorkload::TakeOver(Mi355xConvolution2dWorkload* convolution)
{
    if (!convolution || m_Convolution || !convolution->OnlyConsumerIsAGlobalPooling()) return false;
    if (!convolution->GetOutputHandle() || convolution->GetOutputHandle() != m_Data.m_Inputs[0]) return false;
    m_Convolution = convolution;
    convolution->LeaveExecutionToThePooling();
    g_PoolingPairsFormed.fetch_add(1);
    return true;
}

mi355x_pool2d_desc Mi355xPooling2dWorkload::Describe() const
{
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const Pooling2dDescriptor& p = m_Data.m_Parameters;
    mi355x_pool2d_desc d{};
    d.in_h = in.GetShape()[1]; d.in_w = in.GetShape()[2]; d.channels = in.GetShape()[3];
    d.out_h = out.GetShape()[1]; d.out_w = out.GetShape()[2];
    d.pool_w = p.m_PoolWidth; d.pool_h = p.m_PoolHeight; d.stride_x = p.m_StrideX; d.stride_y = p.m_StrideY;
    d.pad_left = p.m_PadLeft; d.pad_right = p.m_PadRight; d.pad_top = p.m_PadTop; d.pad_bottom = p.m_PadBottom;
    d.pool_type = p.m_PoolType == PoolingAlgorithm::Max ? 0 : 1;
    d.padding_method = p.m_PaddingMethod == PaddingMethod::IgnoreValue ? 0 : 1;
    d.input = mi355x::ToQuant(in);
    d.output = mi355x::ToQuant(out);
    return d;
}

void Mi355xPooling2dWorkload::Execute() const
{
    ARMNN_SCOPED_PROFILING_EVENT_MI355X_NAME_GUID("Mi355xPooling2dWorkload_Execute");
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const mi355x_pool2d_desc d = Describe();
    // the convolution in front has left its execution to this workload: both as one launch, or the convolution first
    if (m_Convolution && m_Convolution->ExecuteWithPooling(d, m_Data.m_Outputs[0], out)) return;
    const void* x = In(m_Data.m_Inputs[0]);
    void* y = Out(m_Data.m_Outputs[0]);
    ForEachLane(in.GetShape()[0], [&](const Lane& l) {
        mi355x::Check(mi355x_pool2d_run(&d, in.GetShape()[0] / l.count, l.Of(x, in), l.Of(y, out), l.stream), "mi355x_pool2d_run");
    });
}

// ---- Mean ------------------------------------------------------------------------------------------------------------
Mi355xMeanWorkload::Mi355xMeanWorkload(const MeanQueueDescriptor& descriptor, const WorkloadInfo& info)
    : Mi355xBaseWorkload<MeanQueueDescriptor>(descriptor, info), m_Info(info)
{
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Mi355xMeanWorkload_Construct", descriptor.m_Parameters, info, this->GetGuid());
    std::vector<unsigned int> axes = m_Data.m_Parameters.m_Axis;
    std::sort(axes.begin(), axes.end());
    if (m_Info.m_InputTensorInfos[0].GetNumDimensions() != 4 || axes != std::vector<unsigned int>{1, 2})
        throw InvalidArgumentException("Mi355xMeanWorkload: the mean over height and width of a 4-D NHWC tensor only");
}

void Mi355xMeanWorkload::Execute() const
{
    ARMNN_SCOPED_PROFILING_EVENT_MI355X_NAME_GUID("Mi355xMeanWorkload_Execute");
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    mi355x_pool2d_desc d{};
    d.in_h = in.GetShape()[1]; d.in_w = in.GetShape()[2]; d.channels = in.GetShape()[3];
    d.out_h = 1; d.out_w = 1;
    d.pool_w = d.in_w; d.pool_h = d.in_h; d.stride_x = 1; d.stride_y = 1;
    d.pool_type = 1;
    d.padding_method = 1;
    d.input = mi355x::ToQuant(in);
    d.output = mi355x::ToQuant(out);
    const void* x = In(m_Data.m_Inputs[0]);
    void* y = Out(m_Data.m_Outputs[0]);
    ForEachLane(in.GetShape()[0], [&](const Lane& l) {
        mi355x::Check(mi355x_pool2d_run(&d, in.GetShape()[0] / l.count, l.Of(x, in), l.Of(y, out), l.stream), "mi355x_pool2d_run (mean)");
    });
}

// ---- Pad -------------------------------------------------------------------------------------------------------------
Mi355xPadWorkload::Mi355xPadWorkload(const PadQueueDescriptor& descriptor, const WorkloadInfo& info)
    : Mi355xBaseWorkload<PadQueueDescriptor>(descriptor, info), m_Info(info)
{
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Mi355xPadWorkload_Construct", descriptor.m_Parameters, info, this->GetGuid());
    if (m_Data.m_Parameters.m_PaddingMode != PaddingMode::Constant) throw InvalidArgumentException("Mi355xPadWorkload: constant padding only");
    if (m_Info.m_InputTensorInfos[0].GetNumDimensions() > 4) throw InvalidArgumentException("Mi355xPadWorkload: at most 4 dimensions");
}

void Mi355xPadWorkload::Execute() const
{
    ARMNN_SCOPED_PROFILING_EVENT_MI355X_NAME_GUID("Mi355xPadWorkload_Execute");
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const PadDescriptor& p = m_Data.m_Parameters;
    mi355x_pad_desc d{};
    d.rank = in.GetNumDimensions();
    for (unsigned int k = 0; k < d.rank; ++k)
    {
        d.in_shape[k] = in.GetShape()[k];
        d.pad_before[k] = p.m_PadList[k].first;
        d.pad_after[k] = p.m_PadList[k].second;
    }
    d.pad_value = p.m_PadValue;
    d.input = mi355x::ToQuant(in);
    d.output = mi355x::ToQuant(m_Info.m_OutputTensorInfos[0]);
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const void* x = In(m_Data.m_Inputs[0]);
    void* y = Out(m_Data.m_Outputs[0]);
    // the batch splits only if nothing is added in front of or behind it
    const bool batchPadded = p.m_PadList[0].first != 0 || p.m_PadList[0].second != 0;
    ForEachLane(batchPadded ? 1u : BatchOf(in), [&](const Lane& l) {
        mi355x_pad_desc slice = d;
        slice.in_shape[0] = d.in_shape[0] / l.count;
        mi355x::Check(mi355x_pad_run(&slice, l.Of(x, in), l.Of(y, out), l.stream), "mi355x_pad_run");
    });
}

// ---- Softmax ---------------------------------------------------------------------------------------------------------
Mi355xSoftmaxWorkload::Mi355xSoftmaxWorkload(const SoftmaxQueueDescriptor& descriptor, const WorkloadInfo& info)
    : Mi355xBaseWorkload<SoftmaxQueueDescriptor>(descriptor, info), m_Info(info)
{
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Mi355xSoftmaxWorkload_Construct", descriptor.m_Parameters, info, this->GetGuid());
}

void Mi355xSoftmaxWorkload::Execute() const
{
    ARMNN_SCOPED_PROFILING_EVENT_MI355X_NAME_GUID("Mi355xSoftmaxWorkload_Execute");
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const unsigned int rank = in.GetNumDimensions();
    const uint32_t cols = in.GetShape()[rank - 1];
    const uint32_t rows = cols ? in.GetNumElements() / cols : 0;
    const mi355x_quant qi = mi355x::ToQuant(in);
    const mi355x_quant qo = mi355x::ToQuant(m_Info.m_OutputTensorInfos[0]);
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const void* x = In(m_Data.m_Inputs[0]);
    void* y = Out(m_Data.m_Outputs[0]);
    ForEachLane(BatchOf(in), [&](const Lane& l) {
        mi355x::Check(mi355x_softmax_run(rows / l.count, cols, m_Data.m_Parameters.m_Beta, &qi, &qo, l.Of(x, in), l.Of(y, out), l.stream), "mi355x_softmax_run");
    });
}

// ---- Add -------------------------------------------------------------------------------------------------------------
Mi355xAdditionWorkload::Mi355xAdditionWorkload(const ElementwiseBinaryQueueDescriptor& descriptor, const WorkloadInfo& info)
    : Mi355xBaseWorkload<ElementwiseBinaryQueueDescriptor>(descriptor, info), m_Info(info)
{
    ARMNN_REPORT_PROFILING_WORKLOAD_DESC("Mi355xAdditionWorkload_Construct", descriptor.m_Parameters, info, this->GetGuid());
    if (m_Data.m_Parameters.m_Operation != BinaryOperation::Add) throw InvalidArgumentException("Mi355xAdditionWorkload: Add only");
    Mi355xFusedActivation::From(m_Data.GetAdditionalInformation<ActivationDescriptor>());
}

unsigned long long Mi355xAdditionWorkload::PairsFormed() { return g_PairsFormed.load(); }
unsigned long long Mi355xAdditionWorkload::PairsRunApart() { return g_PairsRunApart.load(); }

bool Mi355xAdditionWorkload::TakeOver(Mi355xConvolution2dWorkload* convolution)
{
    if (!convolution || m_Convolution || !convolution->FeedsOnlyAnAddition() || convolution->RunsInsideTheAddition()) return false;
    const ITensorHandle* produced = convolution->GetOutputHandle();
    if (!produced || m_Data.m_Inputs[0] == m_Data.m_Inputs[1]) return false;
    unsigned int own;
    if (m_Data.m_Inputs[0] == produced) own = 0;
    else if (m_Data.m_Inputs[1] == produced) own = 1;
    else return false;
    // no broadcast: both inputs have the shape of the sum
    if (m_Info.m_InputTensorInfos[0].GetShape() != m_Info.m_OutputTensorInfos[0].GetShape() ||
        m_Info.m_InputTensorInfos[1].GetShape() != m_Info.m_OutputTensorInfos[0].GetShape())
        return false;
    m_OtherInput = 1 - own;
    m_Convolution = convolution;
    convolution->LeaveExecutionToTheAddition();
    g_PairsFormed.fetch_add(1);
    return true;
}

void Mi355xAdditionWorkload::Execute() const
{
    ARMNN_SCOPED_PROFILING_EVENT_MI355X_NAME_GUID("Mi355xAdditionWorkload_Execute");
    const Mi355xFusedActivation act = Mi355xFusedActivation::From(m_Data.GetAdditionalInformation<ActivationDescriptor>());
    if (m_Convolution)
    {
        m_Convolution->ExecuteWithAddition(m_Data.m_Inputs[m_OtherInput], m_Info.m_InputTensorInfos[m_OtherInput], m_Data.m_Outputs[0],
                                           m_Info.m_OutputTensorInfos[0], act);
        return;
    }
    const mi355x_quant q0 = mi355x::ToQuant(m_Info.m_InputTensorInfos[0]);
    const mi355x_quant q1 = mi355x::ToQuant(m_Info.m_InputTensorInfos[1]);
    const mi355x_quant qo = mi355x::ToQuant(m_Info.m_OutputTensorInfos[0]);
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const void* x0 = In(m_Data.m_Inputs[0]);
    const void* x1 = In(m_Data.m_Inputs[1]);
    void* y = Out(m_Data.m_Outputs[0]);
    ForEachLane(BatchOf(out), [&](const Lane& l) {
        mi355x::Check(mi355x_add_run(out.GetNumElements() / l.count, &q0, &q1, &qo, act.function, act.a, act.b, l.Of(x0, m_Info.m_InputTensorInfos[0]),
                                     l.Of(x1, m_Info.m_InputTensorInfos[1]), l.Of(y, out), l.stream),
                      "mi355x_add_run");
    });
}

// ---- Reshape ---------------------------------------------------------------------------------------------------------
Mi355xReshapeWorkload::Mi355xReshapeWorkload(const ReshapeQueueDescriptor& descriptor, const WorkloadInfo& info)
    : Mi355xBaseWorkload<ReshapeQueueDescriptor>(descriptor, info), m_Info(info)
{
}

void Mi355xReshapeWorkload::Execute() const
{
    ARMNN_SCOPED_PROFILING_EVENT_MI355X_NAME_GUID("Mi355xReshapeWorkload_Execute");
    const size_t bytes = m_Info.m_InputTensorInfos[0].GetNumBytes();
    if (!bytes) return;
    const TensorInfo& in = m_Info.m_InputTensorInfos[0];
    const TensorInfo& out = m_Info.m_OutputTensorInfos[0];
    const void* x = In(m_Data.m_Inputs[0]);
    void* y = Out(m_Data.m_Outputs[0]);
    // a reshape that keeps the batch outermost moves each image's bytes within its own slice
    const bool keepsBatch = BatchOf(in) == BatchOf(out);
    ForEachLane(keepsBatch ? BatchOf(in) : 1u, [&](const Lane& l) {
        mi355x::Check(mi355x_memcpy_d2d(l.Of(y, out), l.Of(x, in), bytes / l.count, l.stream), "mi355x_memcpy_d2d");
    });
}

// ---- Constant --------------------------------------------------------------------------------------------------------
Mi355xConstantWorkload::Mi355xConstantWorkload(const ConstantQueueDescriptor& descriptor, const WorkloadInfo& info)
    : Mi355xBaseWorkload<ConstantQueueDescriptor>(descriptor, info)
{
}

void Mi355xConstantWorkload::Execute() const
{
    // The runtime keeps constant workloads in the queue it runs for every inference (LoadedNetwork.cpp:366-394 and the
    // loop of LoadedNetwork::Execute); the data goes to the device the first time only, as with
    // ClConstantWorkload (src/backends/cl/workloads/ClConstantWorkload.cpp:53-120).
    if (m_RanOnce) return;
    ARMNN_SCOPED_PROFILING_EVENT_MI355X_NAME_GUID("Mi355xConstantWorkload_Execute");
    const void* src = m_Data.m_LayerOutput->Map(true);
    if (!src) throw NullPointerException("Mi355xConstantWorkload: layer has no data");
    m_Data.m_Outputs[0]->CopyInFrom(src);
    m_Data.m_LayerOutput->Unmap();
    m_RanOnce = true;
}
} // namespace armnn
