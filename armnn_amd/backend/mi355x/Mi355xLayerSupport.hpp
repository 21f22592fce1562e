// ILayerSupport of the Mi355x backend: the envelope the device library accepts.  Everything outside it is answered
// "unsupported" with a reason, so Optimize() assigns the layer to the next backend in the caller's preference list
// (RefLayerSupport::IsLayerSupported, src/backends/reference/RefLayerSupport.cpp:61-540, is the CpuRef counterpart).
#pragma once
#include <armnn/backends/ILayerSupport.hpp>

namespace armnn
{
class Mi355xLayerSupport : public ILayerSupport
{
public:
    bool IsLayerSupported(const LayerType& type, const std::vector<TensorInfo>& infos, const BaseDescriptor& descriptor,
                          const Optional<LstmInputParamsInfo>& lstmParamsInfo = EmptyOptional(),
                          const Optional<QuantizedLstmInputParamsInfo>& quantizedLstmParamsInfo = EmptyOptional(),
                          Optional<std::string&> reasonIfUnsupported = EmptyOptional()) const override;

    bool IsConvolution2dSupported(const TensorInfo& input, const TensorInfo& output, const Convolution2dDescriptor& descriptor,
                                  const TensorInfo& weights, const Optional<TensorInfo>& biases, Optional<std::string&> reason) const;
    bool IsDepthwiseConvolutionSupported(const TensorInfo& input, const TensorInfo& output, const DepthwiseConvolution2dDescriptor& descriptor,
                                         const TensorInfo& weights, const Optional<TensorInfo>& biases, Optional<std::string&> reason) const;
    bool IsFullyConnectedSupported(const TensorInfo& input, const TensorInfo& output, const TensorInfo& weights,
                                   const Optional<TensorInfo>& biases, const FullyConnectedDescriptor& descriptor, Optional<std::string&> reason) const;
    bool IsActivationSupported(const TensorInfo& input, const TensorInfo& output, const ActivationDescriptor& descriptor,
                               Optional<std::string&> reason) const;
    bool IsPooling2dSupported(const TensorInfo& input, const TensorInfo& output, const Pooling2dDescriptor& descriptor,
                              Optional<std::string&> reason) const;
    bool IsMeanSupported(const TensorInfo& input, const TensorInfo& output, const MeanDescriptor& descriptor,
                         Optional<std::string&> reasonIfUnsupported = EmptyOptional()) const;
    bool IsPadSupported(const TensorInfo& input, const TensorInfo& output, const PadDescriptor& descriptor,
                        Optional<std::string&> reasonIfUnsupported = EmptyOptional()) const;
    bool IsSoftmaxSupported(const TensorInfo& input, const TensorInfo& output, const SoftmaxDescriptor& descriptor,
                            Optional<std::string&> reason) const;
    bool IsElementwiseBinarySupported(const TensorInfo& input0, const TensorInfo& input1, const TensorInfo& output,
                                      const ElementwiseBinaryDescriptor& descriptor, Optional<std::string&> reason) const;
    bool IsReshapeSupported(const TensorInfo& input, const TensorInfo& output, Optional<std::string&> reason) const;
    bool IsConstantSupported(const TensorInfo& output, Optional<std::string&> reason) const;
    /// Input, Output and MemCopy: any dense tensor of a type the device tensors can hold
    bool IsTransportSupported(const TensorInfo& tensor, Optional<std::string&> reason) const;
};
} // namespace armnn
