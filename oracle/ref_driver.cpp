//
// Thin extern "C" driver over the REAL Arm NN CpuRef hot-path functions -- TEST INFRASTRUCTURE ONLY.
//
// This file is compiled together with a handful of the reference's own source files, taken where they
// lie in the reference tree (see oracle/Makefile, target _ref), into oracle/_ref/libarmnn_cpuref_hotpath.so.
// It does for each call what the reference workloads do in Execute(): build TensorInfos, make
// decoders/encoders with MakeDecoder/MakeEncoder, and call Convolve / FullyConnected / Activation /
// Pooling2d / Softmax / ElementwiseBinaryFunction / Pad (RefConvolution2dWorkload.cpp:38-58,
// RefDepthwiseConvolution2dWorkload.cpp:38-62, RefFullyConnectedWorkload.cpp:39-67,
// RefActivationWorkload.cpp:23-36, RefPooling2dWorkload.cpp, RefSoftmaxWorkload.cpp,
// RefElementwiseBinaryWorkload.cpp:27-107, RefPadWorkload.cpp:18-40).  It is used to validate the C restatement
// (cpuref_oracle.c), to generate golden fixtures, and as the timed CPU baseline.
//
#include "cpuref_oracle.h"

#include "ConvImpl.hpp"
#include "FullyConnected.hpp"
#include "Activation.hpp"
#include "Pooling2d.hpp"
#include "Softmax.hpp"
#include "ElementwiseFunction.hpp"
#include "Pad.hpp"
#include "Reduce.hpp"
#include "Decoders.hpp"
#include "Encoders.hpp"

#include <armnn/Descriptors.hpp>
#include <armnn/Tensor.hpp>
#include <armnn/TypesUtils.hpp>
#include <armnn/backends/ITensorHandle.hpp>

#include <cstring>
#include <functional>
#include <string>

using namespace armnn;

namespace
{
thread_local std::string g_err;

DataType ToDataType(int32_t code)
{
    switch (code)
    {
        case ORC_QASYMM_S8: return DataType::QAsymmS8;
        case ORC_QASYMM_U8: return DataType::QAsymmU8;
        case ORC_QSYMM_S8:  return DataType::QSymmS8;
        case ORC_SIGNED32:  return DataType::Signed32;
        case ORC_FLOAT32:   return DataType::Float32;
        default: throw InvalidArgumentException("unknown dtype code");
    }
}

TensorInfo ToInfo(const orc_tensor* t)
{
    TensorShape shape(t->ndim, t->shape);
    TensorInfo info(shape, ToDataType(t->dtype));
    if (t->n_scales > 0)
    {
        info.SetQuantizationScales(std::vector<float>(t->scales, t->scales + t->n_scales));
    }
    if (t->quant_dim >= 0)
    {
        info.SetQuantizationDim(Optional<unsigned int>(static_cast<unsigned int>(t->quant_dim)));
    }
    info.SetQuantizationOffset(t->offset);
    return info;
}

// the caller's memory behind the tensor-handle interface Pad() reads and writes through
class BorrowedHandle : public ITensorHandle
{
public:
    BorrowedHandle(void* memory, const TensorShape& shape) : m_Memory(memory), m_Shape(shape) {}
    void Manage() override {}
    void Allocate() override {}
    ITensorHandle* GetParent() const override { return nullptr; }
    const void* Map(bool) const override { return m_Memory; }
    void Unmap() const override {}
    TensorShape GetStrides() const override { return m_Shape; }
    TensorShape GetShape() const override { return m_Shape; }
    void CopyOutTo(void*) const override {}
    void CopyInFrom(const void*) override {}
private:
    void* m_Memory;
    TensorShape m_Shape;
};

template <typename F>
int Guard(F&& f)
{
    try { f(); return 0; }
    catch (const std::exception& e) { g_err = e.what(); return -1; }
    catch (...) { g_err = "unknown exception"; return -1; }
}
} // namespace

extern "C" {

const char* ref_last_error(void) { return g_err.c_str(); }

float   ref_dequantize_s8(int8_t v, float s, int32_t o)  { return armnn::Dequantize<int8_t>(v, s, o); }
float   ref_dequantize_u8(uint8_t v, float s, int32_t o) { return armnn::Dequantize<uint8_t>(v, s, o); }
float   ref_dequantize_s32(int32_t v, float s, int32_t o){ return armnn::Dequantize<int32_t>(v, s, o); }
int8_t  ref_quantize_s8(float v, float s, int32_t o)     { return armnn::Quantize<int8_t>(v, s, o); }
uint8_t ref_quantize_u8(float v, float s, int32_t o)     { return armnn::Quantize<uint8_t>(v, s, o); }

int ref_decode_tensor(const orc_tensor* t, int is_depthwise, float* out)
{
    return Guard([&] {
        TensorInfo info = ToInfo(t);
        auto dec = MakeDecoder<float>(info, t->data);
        std::vector<float> v = dec->DecodeTensor(info.GetShape(), is_depthwise != 0);
        std::memcpy(out, v.data(), v.size() * sizeof(float));
    });
}

int ref_conv2d(const orc_tensor* in, const orc_tensor* weights, const orc_tensor* bias,
               const orc_tensor* out, const orc_conv_params* p, int /*fast*/)
{
    return Guard([&] {
        TensorInfo ii = ToInfo(in), wi = ToInfo(weights), oi = ToInfo(out);
        auto inDec  = MakeDecoder<float>(ii, in->data);
        auto outEnc = MakeEncoder<float>(oi, out->data);
        auto wDec   = MakeDecoder<float>(wi, weights->data);
        std::unique_ptr<Decoder<float>> bDec;
        if (p->bias_enabled)
        {
            if (!bias) throw InvalidArgumentException("bias enabled without bias tensor");
            bDec = MakeDecoder<float>(ToInfo(bias), bias->data);
        }
        Convolve(ii.GetShape(), *inDec, oi.GetShape(), *outEnc, wi.GetShape(), *wDec,
                 p->bias_enabled != 0, bDec.get(),
                 p->data_layout == ORC_NHWC ? DataLayout::NHWC : DataLayout::NCHW,
                 p->pad_top, p->pad_left, p->stride_x, p->stride_y, p->dilation_x, p->dilation_y,
                 p->depthwise != 0);
    });
}

int ref_fully_connected(const orc_tensor* in, const orc_tensor* weights, const orc_tensor* bias,
                        const orc_tensor* out, int bias_enabled, int transpose_weights, int /*fast*/)
{
    return Guard([&] {
        TensorInfo ii = ToInfo(in), wi = ToInfo(weights), oi = ToInfo(out);
        auto inDec  = MakeDecoder<float>(ii, in->data);
        auto outEnc = MakeEncoder<float>(oi, out->data);
        auto wDec   = MakeDecoder<float>(wi, weights->data);
        std::unique_ptr<Decoder<float>> bDec;
        if (bias_enabled)
        {
            if (!bias) throw InvalidArgumentException("bias enabled without bias tensor");
            bDec = MakeDecoder<float>(ToInfo(bias), bias->data);
        }
        unsigned int numActivations = 1;
        for (unsigned int i = 1; i < ii.GetNumDimensions(); i++) numActivations *= ii.GetShape()[i];
        FullyConnected(ii.GetShape(), *inDec, oi.GetShape(), *outEnc, wi.GetShape(), *wDec, bDec.get(),
                       bias_enabled != 0, numActivations, transpose_weights != 0);
    });
}

int ref_activation(const orc_tensor* in, const orc_tensor* out, int function, float a, float b)
{
    return Guard([&] {
        TensorInfo ii = ToInfo(in), oi = ToInfo(out);
        ActivationFunction fn = function == ORC_ACT_RELU ? ActivationFunction::ReLu
                              : function == ORC_ACT_BOUNDED_RELU ? ActivationFunction::BoundedReLu
                              : ActivationFunction::Linear;
        if (function == ORC_ACT_NONE) { a = 1.0f; b = 0.0f; }
        Activation(*MakeDecoder<float>(ii, in->data), *MakeEncoder<float>(oi, out->data), ii, fn, a, b);
    });
}

int ref_pooling2d(const orc_tensor* in, const orc_tensor* out, const orc_pool_params* p, int data_layout)
{
    return Guard([&] {
        TensorInfo ii = ToInfo(in), oi = ToInfo(out);
        Pooling2dDescriptor d;
        d.m_PoolType = p->pool_type == ORC_POOL_MAX ? PoolingAlgorithm::Max : PoolingAlgorithm::Average;
        d.m_PaddingMethod = p->padding_method == ORC_PAD_EXCLUDE ? PaddingMethod::Exclude : PaddingMethod::IgnoreValue;
        d.m_PadLeft = p->pad_left; d.m_PadRight = p->pad_right; d.m_PadTop = p->pad_top; d.m_PadBottom = p->pad_bottom;
        d.m_PoolWidth = p->pool_w; d.m_PoolHeight = p->pool_h; d.m_StrideX = p->stride_x; d.m_StrideY = p->stride_y;
        d.m_OutputShapeRounding = OutputShapeRounding::Floor;
        d.m_DataLayout = data_layout == ORC_NHWC ? DataLayout::NHWC : DataLayout::NCHW;
        auto dec = MakeDecoder<float>(ii, in->data);
        auto enc = MakeEncoder<float>(oi, out->data);
        Pooling2d(*dec, *enc, ii, oi, d);
    });
}

int ref_softmax(const orc_tensor* in, const orc_tensor* out, float beta, int axis)
{
    return Guard([&] {
        TensorInfo ii = ToInfo(in), oi = ToInfo(out);
        auto dec = MakeDecoder<float>(ii, in->data);
        auto enc = MakeEncoder<float>(oi, out->data);
        Softmax(*dec, *enc, ii, beta, axis);
    });
}

int ref_add(const orc_tensor* in0, const orc_tensor* in1, const orc_tensor* out)
{
    return Guard([&] {
        TensorInfo i0 = ToInfo(in0), i1 = ToInfo(in1), oi = ToInfo(out);
        auto d0 = MakeDecoder<float>(i0, in0->data);
        auto d1 = MakeDecoder<float>(i1, in1->data);
        auto enc = MakeEncoder<float>(oi, out->data);
        ElementwiseBinaryFunction<std::plus<float>>(i0.GetShape(), i1.GetShape(), oi.GetShape(), *d0, *d1, *enc);
    });
}

int ref_pad(const orc_tensor* in, const orc_tensor* out, const uint32_t* pad_before, float pad_value)
{
    return Guard([&] {
        TensorInfo ii = ToInfo(in), oi = ToInfo(out);
        PadQueueDescriptor q;
        for (uint32_t d = 0; d < in->ndim; ++d)
            q.m_Parameters.m_PadList.emplace_back(pad_before[d], out->shape[d] - in->shape[d] - pad_before[d]);
        q.m_Parameters.m_PadValue = pad_value;
        BorrowedHandle ih(in->data, ii.GetShape()), oh(out->data, oi.GetShape());
        Pad(ii, oi, &ih, &oh, q);
    });
}

// Mean over the given axes: RefMeanWorkload::Execute (workloads/RefMeanWorkload.cpp:26-42) -> Reduce(..., ReduceOperation::Mean)
int ref_mean(const orc_tensor* in, const orc_tensor* out, const uint32_t* axes, uint32_t n_axes)
{
    return Guard([&] {
        TensorInfo ii = ToInfo(in), oi = ToInfo(out);
        auto dec = MakeDecoder<float>(ii, in->data);
        auto enc = MakeEncoder<float>(oi, out->data);
        Reduce(ii, oi, *dec, *enc, std::vector<uint32_t>(axes, axes + n_axes), ReduceOperation::Mean);
    });
}

} // extern "C"
