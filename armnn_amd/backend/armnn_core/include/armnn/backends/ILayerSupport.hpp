// Minimal host core: include/armnn/backends/ILayerSupport.hpp:22-40 (the one unified entry point).
#pragma once
#include "../Descriptors.hpp"
#include "../Optional.hpp"
#include "../Tensor.hpp"
#include "../Types.hpp"
#include <string>
#include <vector>

namespace armnn
{
struct LstmInputParamsInfo {};
struct QuantizedLstmInputParamsInfo {};

class ILayerSupport
{
protected:
    ILayerSupport() {}
    virtual ~ILayerSupport() {}
public:
    virtual bool IsLayerSupported(const LayerType& type, const std::vector<TensorInfo>& infos, const BaseDescriptor& descriptor,
                                  const Optional<LstmInputParamsInfo>& lstmParamsInfo = EmptyOptional(),
                                  const Optional<QuantizedLstmInputParamsInfo>& quantizedLstmParamsInfo = EmptyOptional(),
                                  Optional<std::string&> reasonIfUnsupported = EmptyOptional()) const = 0;
};
} // namespace armnn
