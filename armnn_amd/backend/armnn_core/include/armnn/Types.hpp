// Minimal host core: enumerations and small types with the names of include/armnn/Types.hpp.
#pragma once
#include "BackendId.hpp"
#include <cstdint>
#include <functional>
#include <memory>
#include <string>

namespace armnn
{
constexpr unsigned int MaxNumOfTensorDimensions = 5U;

enum class Status { Success = 0, Failure = 1 };

enum class DataType
{
    Float16 = 0, Float32 = 1, QAsymmU8 = 2, Signed32 = 3, Boolean = 4, QSymmS16 = 5, QSymmS8 = 6, QAsymmS8 = 7,
    BFloat16 = 8, Signed64 = 9
};

enum class DataLayout { NCHW = 1, NHWC = 2, NDHWC = 3, NCDHW = 4 };

enum class ActivationFunction
{
    Sigmoid = 0, TanH = 1, Linear = 2, ReLu = 3, BoundedReLu = 4, SoftReLu = 5, LeakyReLu = 6, Abs = 7, Sqrt = 8,
    Square = 9, Elu = 10, HardSwish = 11, Gelu = 12
};

enum class PoolingAlgorithm { Max = 0, Average = 1, L2 = 2 };
enum class PaddingMethod { IgnoreValue = 0, Exclude = 1 };
enum class PaddingMode { Constant = 0, Reflect = 1, Symmetric = 2 };
enum class OutputShapeRounding { Floor = 0, Ceiling = 1 };
enum class BinaryOperation { Add = 0, Div = 1, Maximum = 2, Minimum = 3, Mul = 4, Sub = 5, SqDiff = 6, Power = 7, FloorDiv = 8 };

enum class MemorySource : uint32_t { Undefined = 0, Malloc = 1, DmaBuf = 2, DmaBufProtected = 4, Gralloc = 8 };
using MemorySourceFlags = unsigned int;
enum class MemBlockStrategyType { SingleAxisPacking = 0, MultiAxisPacking = 1 };
enum class ProfilingDetailsMethod { Undefined = 0, DetailsWithEvents = 1, DetailsOnly = 2 };

// the layer kinds this core can hold (names as in include/armnn/Types.hpp:410-500)
enum class LayerType
{
    Activation, Constant, Convolution2d, DepthwiseConvolution2d, ElementwiseBinary, FullyConnected, Input, Mean, MemCopy,
    Output, Pad, Pooling2d, Reshape, Softmax
};
const char* GetLayerTypeAsCString(LayerType type);

using NetworkId = int;
using ImportedInputId = unsigned int;
using ImportedOutputId = unsigned int;
using LayerBindingId = int;
using LayerGuid = uint64_t;

/// Each backend implements this (include/armnn/Types.hpp:273-281)
class IBackend
{
protected:
    IBackend() {}
    virtual ~IBackend() {}
public:
    virtual const BackendId& GetId() const = 0;
};
using IBackendSharedPtr = std::shared_ptr<IBackend>;

/// Device specific knowledge handed to Optimize()
class IDeviceSpec
{
protected:
    IDeviceSpec() {}
    virtual ~IDeviceSpec() {}
public:
    virtual const BackendIdSet& GetSupportedBackends() const = 0;
};

constexpr unsigned int GetDataTypeSize(DataType t)
{
    switch (t)
    {
        case DataType::Float16: case DataType::BFloat16: case DataType::QSymmS16: return 2U;
        case DataType::Float32: case DataType::Signed32: return 4U;
        case DataType::Signed64: return 8U;
        default: return 1U;
    }
}
const char* GetDataTypeName(DataType t);
constexpr bool IsQuantized8BitType(DataType t) { return t == DataType::QAsymmU8 || t == DataType::QAsymmS8 || t == DataType::QSymmS8; }
constexpr bool IsQuantizedType(DataType t) { return IsQuantized8BitType(t) || t == DataType::QSymmS16; }
} // namespace armnn
