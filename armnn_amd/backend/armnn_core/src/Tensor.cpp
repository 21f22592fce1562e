// Minimal host core: TensorShape / TensorInfo and the small name tables.
#include <armnn/Tensor.hpp>
#include <armnn/Types.hpp>
#include <armnn/backends/TensorHandle.hpp>

namespace armnn
{
TensorShape::TensorShape(unsigned int numDimensions, const unsigned int* dimensionSizes) : m_NumDimensions(numDimensions)
{
    if (numDimensions > 6) throw InvalidArgumentException("Tensor numDimensions must be <= 6");
    if (numDimensions > 0 && dimensionSizes == nullptr) throw InvalidArgumentException("Tensor dimensionSizes must not be NULL");
    m_Dimensions.fill(0);
    for (unsigned int i = 0; i < numDimensions; ++i) m_Dimensions[i] = dimensionSizes[i];
}

TensorShape::TensorShape(std::initializer_list<unsigned int> l) : m_NumDimensions(static_cast<unsigned int>(l.size()))
{
    if (l.size() > 6) throw InvalidArgumentException("Tensor numDimensions must be <= 6");
    m_Dimensions.fill(0);
    unsigned int i = 0;
    for (unsigned int d : l) m_Dimensions[i++] = d;
}

unsigned int TensorShape::operator[](unsigned int i) const
{
    if (i >= m_NumDimensions) throw InvalidArgumentException("TensorShape: dimension index out of range");
    return m_Dimensions[i];
}

unsigned int& TensorShape::operator[](unsigned int i)
{
    if (i >= m_NumDimensions) throw InvalidArgumentException("TensorShape: dimension index out of range");
    return m_Dimensions[i];
}

bool TensorShape::operator==(const TensorShape& other) const
{
    if (m_NumDimensions != other.m_NumDimensions) return false;
    for (unsigned int i = 0; i < m_NumDimensions; ++i)
        if (m_Dimensions[i] != other.m_Dimensions[i]) return false;
    return true;
}

unsigned int TensorShape::GetNumElements() const
{
    if (m_NumDimensions == 0) return 0;
    unsigned int n = 1;
    for (unsigned int i = 0; i < m_NumDimensions; ++i) n *= m_Dimensions[i];
    return n;
}

TensorInfo::TensorInfo(DataType dataType, float scale, int32_t offset, bool isConstant) : m_DataType(dataType), m_IsConstant(isConstant)
{
    SetQuantizationScale(scale);
    SetQuantizationOffset(offset);
}

TensorInfo::TensorInfo(const TensorShape& shape, DataType dataType, float scale, int32_t offset, bool isConstant)
    : m_Shape(shape), m_DataType(dataType), m_IsConstant(isConstant)
{
    SetQuantizationScale(scale);
    SetQuantizationOffset(offset);
}

TensorInfo::TensorInfo(const TensorShape& shape, DataType dataType, const std::vector<float>& scales, unsigned int quantizationDim,
                       bool isConstant)
    : m_Shape(shape), m_DataType(dataType), m_IsConstant(isConstant)
{
    SetQuantizationScales(scales);
    SetQuantizationDim(MakeOptional<unsigned int>(quantizationDim));
}

float TensorInfo::GetQuantizationScale() const
{
    if (m_Scales.empty()) return 1.0f;     // old default, kept by the reference for backward compatibility
    if (HasMultipleQuantizationScales())
        throw RuntimeException("Invalid call to GetQuantizationScale on a tensor with multiple scale values. Use GetQuantizationScales instead.");
    return m_Scales[0];
}

bool TensorInfo::operator==(const TensorInfo& other) const
{
    return m_Shape == other.m_Shape && m_DataType == other.m_DataType && m_Scales == other.m_Scales &&
           GetQuantizationOffset() == other.GetQuantizationOffset() && m_IsConstant == other.m_IsConstant;
}

bool TensorInfo::IsTypeSpaceMatch(const TensorInfo& other) const
{
    bool match = m_DataType == other.m_DataType;
    if (IsQuantized() && !HasMultipleQuantizationScales())
        match &= GetQuantizationScale() == other.GetQuantizationScale() && GetQuantizationOffset() == other.GetQuantizationOffset();
    return match;
}

TensorShape GetUnpaddedTensorStrides(const TensorInfo& tensorInfo)
{
    TensorShape shape(tensorInfo.GetShape());
    unsigned int stride = GetDataTypeSize(tensorInfo.GetDataType());
    for (unsigned int i = shape.GetNumDimensions(); i-- > 0;)
    {
        const unsigned int extent = shape[i];
        shape[i] = stride;
        stride *= extent;
    }
    return shape;
}

const char* GetDataTypeName(DataType t)
{
    switch (t)
    {
        case DataType::Float16: return "Float16";
        case DataType::Float32: return "Float32";
        case DataType::QAsymmU8: return "QAsymmU8";
        case DataType::Signed32: return "Signed32";
        case DataType::Boolean: return "Boolean";
        case DataType::QSymmS16: return "QSymm16";
        case DataType::QSymmS8: return "QSymmS8";
        case DataType::QAsymmS8: return "QAsymmS8";
        case DataType::BFloat16: return "BFloat16";
        case DataType::Signed64: return "Signed64";
        default: return "Unknown";
    }
}

const char* GetLayerTypeAsCString(LayerType type)
{
    switch (type)
    {
        case LayerType::Activation: return "Activation";
        case LayerType::Constant: return "Constant";
        case LayerType::Convolution2d: return "Convolution2d";
        case LayerType::DepthwiseConvolution2d: return "DepthwiseConvolution2d";
        case LayerType::ElementwiseBinary: return "ElementwiseBinary";
        case LayerType::FullyConnected: return "FullyConnected";
        case LayerType::Input: return "Input";
        case LayerType::MemCopy: return "MemCopy";
        case LayerType::Output: return "Output";
        case LayerType::Pooling2d: return "Pooling2d";
        case LayerType::Reshape: return "Reshape";
        case LayerType::Mean: return "Mean";
        case LayerType::Pad: return "Pad";
        case LayerType::Softmax: return "Softmax";
        default: return "Unknown";
    }
}
} // namespace armnn
