// Minimal host core: layer descriptors with the member names of include/armnn/Descriptors.hpp.
#pragma once
#include "Tensor.hpp"
#include "Types.hpp"
#include <utility>
#include <vector>

namespace armnn
{
struct BaseDescriptor
{
    virtual bool IsNull() const { return false; }
    virtual ~BaseDescriptor() = default;
};
struct NullDescriptor : BaseDescriptor
{
    bool IsNull() const override { return true; }
};

struct ActivationDescriptor : BaseDescriptor
{
    ActivationDescriptor() = default;
    ActivationDescriptor(ActivationFunction fn, float a = 0, float b = 0) : m_Function(fn), m_A(a), m_B(b) {}
    bool operator==(const ActivationDescriptor& rhs) const { return m_Function == rhs.m_Function && m_A == rhs.m_A && m_B == rhs.m_B; }
    ActivationFunction m_Function = ActivationFunction::Sigmoid;
    float m_A = 0;   ///< upper bound for BoundedReLu
    float m_B = 0;   ///< lower bound for BoundedReLu
};

struct Convolution2dDescriptor : BaseDescriptor
{
    uint32_t GetNumInputs() const { return m_BiasEnabled ? 3u : 2u; }
    uint32_t m_PadLeft = 0, m_PadRight = 0, m_PadTop = 0, m_PadBottom = 0;
    uint32_t m_StrideX = 1, m_StrideY = 1;
    uint32_t m_DilationX = 1, m_DilationY = 1;
    bool m_BiasEnabled = false;
    DataLayout m_DataLayout = DataLayout::NCHW;
};

struct DepthwiseConvolution2dDescriptor : BaseDescriptor
{
    uint32_t GetNumInputs() const { return m_BiasEnabled ? 3u : 2u; }
    uint32_t m_PadLeft = 0, m_PadRight = 0, m_PadTop = 0, m_PadBottom = 0;
    uint32_t m_StrideX = 1, m_StrideY = 1;
    uint32_t m_DilationX = 1, m_DilationY = 1;
    bool m_BiasEnabled = false;
    DataLayout m_DataLayout = DataLayout::NCHW;
};

struct FullyConnectedDescriptor : BaseDescriptor
{
    uint32_t GetNumInputs() const { return m_BiasEnabled ? 3u : 2u; }
    bool m_BiasEnabled = false;
    bool m_TransposeWeightMatrix = false;
    bool m_ConstantWeights = true;
};

struct Pooling2dDescriptor : BaseDescriptor
{
    PoolingAlgorithm m_PoolType = PoolingAlgorithm::Max;
    uint32_t m_PadLeft = 0, m_PadRight = 0, m_PadTop = 0, m_PadBottom = 0;
    uint32_t m_PoolWidth = 0, m_PoolHeight = 0;
    uint32_t m_StrideX = 0, m_StrideY = 0;
    OutputShapeRounding m_OutputShapeRounding = OutputShapeRounding::Floor;
    PaddingMethod m_PaddingMethod = PaddingMethod::Exclude;
    DataLayout m_DataLayout = DataLayout::NCHW;
};

/// include/armnn/Descriptors.hpp:1172-1193: mean over the listed dimensions, which stay as extents of 1 if m_KeepDims
struct MeanDescriptor : BaseDescriptor
{
    MeanDescriptor() = default;
    MeanDescriptor(const std::vector<unsigned int>& axis, bool keepDims) : m_Axis(axis), m_KeepDims(keepDims) {}
    bool operator==(const MeanDescriptor& rhs) const { return m_Axis == rhs.m_Axis && m_KeepDims == rhs.m_KeepDims; }
    std::vector<unsigned int> m_Axis;
    bool m_KeepDims = false;
};

/// include/armnn/Descriptors.hpp:1196-1229: one (before, after) pair per dimension; for quantized tensors m_PadValue
/// is the stored code itself, not a real number to be quantized (workloads/Pad.cpp:77-84)
struct PadDescriptor : BaseDescriptor
{
    PadDescriptor() = default;
    PadDescriptor(const std::vector<std::pair<unsigned int, unsigned int>>& padList, float padValue = 0,
                  PaddingMode paddingMode = PaddingMode::Constant)
        : m_PadList(padList), m_PadValue(padValue), m_PaddingMode(paddingMode) {}
    bool operator==(const PadDescriptor& rhs) const
    {
        return m_PadList == rhs.m_PadList && m_PadValue == rhs.m_PadValue && m_PaddingMode == rhs.m_PaddingMode;
    }
    std::vector<std::pair<unsigned int, unsigned int>> m_PadList;
    float m_PadValue = 0;
    PaddingMode m_PaddingMode = PaddingMode::Constant;
};

struct SoftmaxDescriptor : BaseDescriptor
{
    float m_Beta = 1.0f;
    int m_Axis = -1;
};

struct ElementwiseBinaryDescriptor : BaseDescriptor
{
    ElementwiseBinaryDescriptor() = default;
    ElementwiseBinaryDescriptor(BinaryOperation op) : m_Operation(op) {}
    BinaryOperation m_Operation = BinaryOperation::Add;
};

struct ReshapeDescriptor : BaseDescriptor
{
    ReshapeDescriptor() = default;
    ReshapeDescriptor(const TensorShape& shape) : m_TargetShape(shape) {}
    TensorShape m_TargetShape;
};
} // namespace armnn
