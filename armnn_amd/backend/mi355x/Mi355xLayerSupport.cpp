#include "Mi355xLayerSupport.hpp"
#include "Mi355xDevice.hpp"

#include <armnn/TypesUtils.hpp>
#include <armnn/utility/PolymorphicDowncast.hpp>

#include <algorithm>
#include <cmath>
#include <vector>

namespace armnn
{
namespace
{
bool No(Optional<std::string&> reason, const std::string& why)
{
    if (reason.has_value()) reason.value() = "Mi355x: " + why;
    return false;
}

bool IsActivationType(DataType t) { return t == DataType::QAsymmS8 || t == DataType::QAsymmU8; }

bool GoodScale(const TensorInfo& t)
{
    for (float s : t.GetQuantizationScales())
        if (!(s > 0.0f) || !std::isfinite(s)) return false;
    return !t.GetQuantizationScales().empty();
}

// input/output: same 8-bit asymmetric type, sane scales
bool CheckActivations(const TensorInfo& input, const TensorInfo& output, Optional<std::string&> reason)
{
    if (!IsActivationType(input.GetDataType()))
        return No(reason, std::string("input data type ") + GetDataTypeName(input.GetDataType()) + " is not QAsymmS8 or QAsymmU8");
    if (output.GetDataType() != input.GetDataType()) return No(reason, "input and output data types differ");
    if (input.HasMultipleQuantizationScales() || output.HasMultipleQuantizationScales())
        return No(reason, "per-axis quantization is supported on constant weights and bias only");
    if (!GoodScale(input) || !GoodScale(output)) return No(reason, "quantization scales must be positive and finite");
    return true;
}

// weights + bias rules shared by Convolution2d, DepthwiseConvolution2d and FullyConnected
bool CheckConstants(const TensorInfo& weights, const Optional<TensorInfo>& biases, bool biasEnabled, unsigned int outChannels,
                    unsigned int expectedQuantDim, Optional<std::string&> reason)
{
    const DataType wt = weights.GetDataType();
    if (wt != DataType::QSymmS8 && wt != DataType::QAsymmS8 && wt != DataType::QAsymmU8)
        return No(reason, std::string("weights data type ") + GetDataTypeName(wt) + " is not an 8-bit quantized type");
    if (!weights.IsConstant()) return No(reason, "weights must be constant (the kernels consume a re-laid-out copy made at load time)");
    if (!GoodScale(weights)) return No(reason, "weight scales must be positive and finite");
    if (weights.HasMultipleQuantizationScales())
    {
        if (weights.GetQuantizationScales().size() != outChannels) return No(reason, "per-axis weights must carry one scale per output channel");
        if (weights.GetQuantizationDim().has_value() && weights.GetQuantizationDim().value() != expectedQuantDim)
            return No(reason, "per-axis weights must be quantized along the output-channel dimension");
        if (weights.GetQuantizationOffset() != 0) return No(reason, "per-axis weights must have offset 0");
    }
    if (biasEnabled)
    {
        if (!biases.has_value()) return No(reason, "bias enabled but no bias tensor described");
        const TensorInfo& b = biases.value();
        if (b.GetDataType() != DataType::Signed32) return No(reason, "bias must be Signed32");
        if (!b.IsConstant()) return No(reason, "bias must be constant");
        if (b.GetNumElements() != outChannels) return No(reason, "bias must have one element per output channel");
        if (b.GetQuantizationOffset() != 0) return No(reason, "bias offset must be 0");
        const size_t n = b.GetQuantizationScales().size();
        if (n != 1 && n != outChannels) return No(reason, "bias must carry 1 scale or one per output channel");
    }
    return true;
}

// The device kernels accumulate sum (x - zx)(w - zw) exactly in 32 bits and refuse a plan whose taps could overflow that
// (mi355x_conv2d_create: K * max|x - zx| * max|w - zw| < 2^31, with the true zero points and weights).  Layer support sees
// neither, so it applies the bound that holds for any of them: K * 255 * 255 < 2^31, i.e. K <= 33 025 taps per output.
// A layer beyond that goes to the next backend at optimization time instead of failing at the first inference.
bool CheckTaps(unsigned long long taps, Optional<std::string&> reason)
{
    if (taps * 255ull * 255ull >= (1ull << 31)) return No(reason, "more than 33 025 taps per output could overflow the 32-bit accumulator");
    return true;
}
} // namespace

bool Mi355xLayerSupport::IsConvolution2dSupported(const TensorInfo& input, const TensorInfo& output, const Convolution2dDescriptor& d,
                                                  const TensorInfo& weights, const Optional<TensorInfo>& biases, Optional<std::string&> reason) const
{
    if (d.m_DataLayout != DataLayout::NHWC) return No(reason, "Convolution2d needs DataLayout::NHWC");
    if (input.GetNumDimensions() != 4 || output.GetNumDimensions() != 4 || weights.GetNumDimensions() != 4) return No(reason, "Convolution2d needs 4-D tensors");
    if (!CheckActivations(input, output, reason)) return false;
    if (weights.GetShape()[3] != input.GetShape()[3]) return No(reason, "weights [O,H,W,I]: I differs from the input channels");
    if (weights.GetShape()[0] != output.GetShape()[3]) return No(reason, "weights [O,H,W,I]: O differs from the output channels");
    if (input.GetShape()[0] != output.GetShape()[0]) return No(reason, "batch sizes differ");
    if (d.m_StrideX == 0 || d.m_StrideY == 0 || d.m_DilationX == 0 || d.m_DilationY == 0) return No(reason, "zero stride or dilation");
    if (!CheckTaps(static_cast<unsigned long long>(weights.GetShape()[1]) * weights.GetShape()[2] * weights.GetShape()[3], reason)) return false;
    return CheckConstants(weights, biases, d.m_BiasEnabled, output.GetShape()[3], 0, reason);
}

bool Mi355xLayerSupport::IsDepthwiseConvolutionSupported(const TensorInfo& input, const TensorInfo& output, const DepthwiseConvolution2dDescriptor& d,
                                                         const TensorInfo& weights, const Optional<TensorInfo>& biases, Optional<std::string&> reason) const
{
    if (d.m_DataLayout != DataLayout::NHWC) return No(reason, "DepthwiseConvolution2d needs DataLayout::NHWC");
    if (input.GetNumDimensions() != 4 || output.GetNumDimensions() != 4 || weights.GetNumDimensions() != 4) return No(reason, "DepthwiseConvolution2d needs 4-D tensors");
    if (!CheckActivations(input, output, reason)) return false;
    if (weights.GetShape()[0] != 1) return No(reason, "depthwise weights must be [1,H,W,O]");
    if (weights.GetShape()[3] != output.GetShape()[3]) return No(reason, "depthwise weights [1,H,W,O]: O differs from the output channels");
    if (input.GetShape()[3] == 0 || output.GetShape()[3] % input.GetShape()[3] != 0) return No(reason, "output channels must be a multiple of the input channels");
    if (input.GetShape()[0] != output.GetShape()[0]) return No(reason, "batch sizes differ");
    if (d.m_StrideX == 0 || d.m_StrideY == 0 || d.m_DilationX == 0 || d.m_DilationY == 0) return No(reason, "zero stride or dilation");
    return CheckConstants(weights, biases, d.m_BiasEnabled, output.GetShape()[3], 3, reason);
}

bool Mi355xLayerSupport::IsFullyConnectedSupported(const TensorInfo& input, const TensorInfo& output, const TensorInfo& weights,
                                                   const Optional<TensorInfo>& biases, const FullyConnectedDescriptor& d, Optional<std::string&> reason) const
{
    if (!d.m_ConstantWeights) return No(reason, "FullyConnected needs constant weights");
    if (output.GetNumDimensions() != 2 || weights.GetNumDimensions() != 2) return No(reason, "FullyConnected needs a 2-D output and 2-D weights");
    if (input.GetNumDimensions() < 2 || input.GetShape()[0] == 0) return No(reason, "FullyConnected needs a batched input");
    if (!CheckActivations(input, output, reason)) return false;
    const unsigned int k = input.GetNumElements() / input.GetShape()[0];
    const unsigned int o = output.GetShape()[1];
    const unsigned int wk = d.m_TransposeWeightMatrix ? weights.GetShape()[1] : weights.GetShape()[0];
    const unsigned int wo = d.m_TransposeWeightMatrix ? weights.GetShape()[0] : weights.GetShape()[1];
    if (wk != k || wo != o) return No(reason, "weights shape does not match input width / output width");
    if (output.GetShape()[0] != input.GetShape()[0]) return No(reason, "batch sizes differ");
    if (!CheckTaps(k, reason)) return false;
    return CheckConstants(weights, biases, d.m_BiasEnabled, o, d.m_TransposeWeightMatrix ? 0 : 1, reason);
}

bool Mi355xLayerSupport::IsActivationSupported(const TensorInfo& input, const TensorInfo& output, const ActivationDescriptor& d,
                                               Optional<std::string&> reason) const
{
    if (d.m_Function != ActivationFunction::ReLu && d.m_Function != ActivationFunction::BoundedReLu)
        return No(reason, "only ReLu and BoundedReLu activations run on the device");
    if (input.GetShape() != output.GetShape()) return No(reason, "input and output shapes differ");
    return CheckActivations(input, output, reason);
}

bool Mi355xLayerSupport::IsPooling2dSupported(const TensorInfo& input, const TensorInfo& output, const Pooling2dDescriptor& d,
                                              Optional<std::string&> reason) const
{
    if (d.m_DataLayout != DataLayout::NHWC) return No(reason, "Pooling2d needs DataLayout::NHWC");
    if (d.m_PoolType != PoolingAlgorithm::Max && d.m_PoolType != PoolingAlgorithm::Average) return No(reason, "only Max and Average pooling run on the device");
    if (input.GetNumDimensions() != 4 || output.GetNumDimensions() != 4) return No(reason, "Pooling2d needs 4-D tensors");
    if (d.m_PoolWidth == 0 || d.m_PoolHeight == 0 || d.m_StrideX == 0 || d.m_StrideY == 0) return No(reason, "zero pool size or stride");
    if (input.GetShape()[3] != output.GetShape()[3] || input.GetShape()[0] != output.GetShape()[0]) return No(reason, "batch / channel counts differ");
    return CheckActivations(input, output, reason);
}

bool Mi355xLayerSupport::IsMeanSupported(const TensorInfo& input, const TensorInfo& output, const MeanDescriptor& d,
                                         Optional<std::string&> reason) const
{
    if (input.GetNumDimensions() != 4) return No(reason, "Mean runs on 4-D NHWC tensors");
    std::vector<unsigned int> axes = d.m_Axis;
    std::sort(axes.begin(), axes.end());
    if (axes != std::vector<unsigned int>{1, 2}) return No(reason, "only the mean over height and width (axes 1 and 2) runs on the device");
    const unsigned int n = input.GetShape()[0], c = input.GetShape()[3];
    const bool shapeOk = d.m_KeepDims ? (output.GetNumDimensions() == 4 && output.GetShape()[0] == n && output.GetShape()[1] == 1 &&
                                         output.GetShape()[2] == 1 && output.GetShape()[3] == c)
                                      : (output.GetNumDimensions() == 2 && output.GetShape()[0] == n && output.GetShape()[1] == c);
    if (!shapeOk) return No(reason, "output shape is not [N, 1, 1, C] (kept dimensions) or [N, C]");
    if (input.GetShape()[1] == 0 || input.GetShape()[2] == 0) return No(reason, "empty feature map");
    return CheckActivations(input, output, reason);
}

bool Mi355xLayerSupport::IsPadSupported(const TensorInfo& input, const TensorInfo& output, const PadDescriptor& d,
                                        Optional<std::string&> reason) const
{
    if (d.m_PaddingMode != PaddingMode::Constant) return No(reason, "only constant padding runs on the device");
    const unsigned int rank = input.GetNumDimensions();
    if (rank < 1 || rank > 4) return No(reason, "Pad runs on tensors of 1 to 4 dimensions");
    if (output.GetNumDimensions() != rank || d.m_PadList.size() != rank) return No(reason, "Pad needs one (before, after) pair per dimension");
    for (unsigned int k = 0; k < rank; ++k)
        if (input.GetShape()[k] + d.m_PadList[k].first + d.m_PadList[k].second != output.GetShape()[k])
            return No(reason, "output shape is not the input shape plus the padding");
    if (std::isnan(d.m_PadValue)) return No(reason, "pad value is not a number");
    return CheckActivations(input, output, reason);
}

bool Mi355xLayerSupport::IsSoftmaxSupported(const TensorInfo& input, const TensorInfo& output, const SoftmaxDescriptor& d,
                                            Optional<std::string&> reason) const
{
    const int rank = static_cast<int>(input.GetNumDimensions());
    if (rank < 1) return No(reason, "Softmax needs at least one dimension");
    if (d.m_Axis != -1 && d.m_Axis != rank - 1) return No(reason, "Softmax runs over the innermost axis only");
    if (input.GetShape() != output.GetShape()) return No(reason, "input and output shapes differ");
    return CheckActivations(input, output, reason);
}

bool Mi355xLayerSupport::IsElementwiseBinarySupported(const TensorInfo& in0, const TensorInfo& in1, const TensorInfo& output,
                                                      const ElementwiseBinaryDescriptor& d, Optional<std::string&> reason) const
{
    if (d.m_Operation != BinaryOperation::Add) return No(reason, "only ElementwiseBinary Add runs on the device");
    if (in0.GetShape() != in1.GetShape() || in0.GetShape() != output.GetShape()) return No(reason, "Add needs equally shaped tensors (no broadcast)");
    if (in1.GetDataType() != in0.GetDataType()) return No(reason, "inputs have different data types");
    if (in1.HasMultipleQuantizationScales() || !GoodScale(in1)) return No(reason, "second input: bad quantization");
    return CheckActivations(in0, output, reason);
}

bool Mi355xLayerSupport::IsReshapeSupported(const TensorInfo& input, const TensorInfo& output, Optional<std::string&> reason) const
{
    if (input.GetNumElements() != output.GetNumElements()) return No(reason, "Reshape changes the number of elements");
    if (input.GetDataType() != output.GetDataType()) return No(reason, "Reshape changes the data type");
    return IsTransportSupported(input, reason);
}

bool Mi355xLayerSupport::IsConstantSupported(const TensorInfo& output, Optional<std::string&> reason) const
{
    return IsTransportSupported(output, reason);
}

bool Mi355xLayerSupport::IsTransportSupported(const TensorInfo& t, Optional<std::string&> reason) const
{
    switch (t.GetDataType())
    {
        case DataType::QAsymmS8: case DataType::QAsymmU8: case DataType::QSymmS8: case DataType::Signed32: return true;
        default: return No(reason, std::string("tensors of type ") + GetDataTypeName(t.GetDataType()) + " are not held on the device");
    }
}

bool Mi355xLayerSupport::IsLayerSupported(const LayerType& type, const std::vector<TensorInfo>& infos, const BaseDescriptor& descriptor,
                                          const Optional<LstmInputParamsInfo>&, const Optional<QuantizedLstmInputParamsInfo>&,
                                          Optional<std::string&> reason) const
{
    if (!mi355x::DeviceUsable()) return No(reason, "no MI355X device is visible to this process");
    auto need = [&](size_t n) {
        if (infos.size() < n) throw InvalidArgumentException("Mi355xLayerSupport: too few TensorInfos for " + std::string(GetLayerTypeAsCString(type)));
    };
    // {input, output, weights, biases}: an empty TensorInfo stands for "no bias" (RefLayerSupport.cpp:137-160)
    auto bias = [&](bool enabled) { return enabled ? Optional<TensorInfo>(infos[3]) : Optional<TensorInfo>(); };
    switch (type)
    {
        case LayerType::Convolution2d:
        {
            need(4);
            const auto& d = *PolymorphicDowncast<const Convolution2dDescriptor*>(&descriptor);
            return IsConvolution2dSupported(infos[0], infos[1], d, infos[2], bias(d.m_BiasEnabled), reason);
        }
        case LayerType::DepthwiseConvolution2d:
        {
            need(4);
            const auto& d = *PolymorphicDowncast<const DepthwiseConvolution2dDescriptor*>(&descriptor);
            return IsDepthwiseConvolutionSupported(infos[0], infos[1], d, infos[2], bias(d.m_BiasEnabled), reason);
        }
        case LayerType::FullyConnected:
        {
            need(4);
            const auto& d = *PolymorphicDowncast<const FullyConnectedDescriptor*>(&descriptor);
            return IsFullyConnectedSupported(infos[0], infos[1], infos[2], bias(d.m_BiasEnabled), d, reason);
        }
        case LayerType::Activation:
            need(2);
            return IsActivationSupported(infos[0], infos[1], *PolymorphicDowncast<const ActivationDescriptor*>(&descriptor), reason);
        case LayerType::Pooling2d:
            need(2);
            return IsPooling2dSupported(infos[0], infos[1], *PolymorphicDowncast<const Pooling2dDescriptor*>(&descriptor), reason);
        case LayerType::Mean:
            need(2);
            return IsMeanSupported(infos[0], infos[1], *PolymorphicDowncast<const MeanDescriptor*>(&descriptor), reason);
        case LayerType::Pad:
            need(2);
            return IsPadSupported(infos[0], infos[1], *PolymorphicDowncast<const PadDescriptor*>(&descriptor), reason);
        case LayerType::Softmax:
            need(2);
            return IsSoftmaxSupported(infos[0], infos[1], *PolymorphicDowncast<const SoftmaxDescriptor*>(&descriptor), reason);
        case LayerType::ElementwiseBinary:
            need(3);
            return IsElementwiseBinarySupported(infos[0], infos[1], infos[2], *PolymorphicDowncast<const ElementwiseBinaryDescriptor*>(&descriptor), reason);
        case LayerType::Reshape:
            need(2);
            return IsReshapeSupported(infos[0], infos[1], reason);
        case LayerType::Constant:
            need(1);
            return IsConstantSupported(infos[0], reason);
        case LayerType::Input:
        case LayerType::Output:
            need(1);
            return IsTransportSupported(infos[0], reason);
        case LayerType::MemCopy:
            need(2);
            return IsTransportSupported(infos[0], reason) && IsTransportSupported(infos[1], reason);
        default:
            return No(reason, std::string("layer type ") + GetLayerTypeAsCString(type) + " is not implemented");
    }
}
} // namespace armnn
