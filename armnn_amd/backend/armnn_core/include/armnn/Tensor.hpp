// Minimal host core: TensorShape / TensorInfo / (Const)Tensor with the interface of include/armnn/Tensor.hpp:20-360
// that quantized convolution paths use (per-tensor and per-axis quantization included).
#pragma once
#include "Exceptions.hpp"
#include "Optional.hpp"
#include "Types.hpp"
#include <array>
#include <initializer_list>
#include <vector>

namespace armnn
{
class TensorShape
{
public:
    TensorShape() : m_NumDimensions(0) { m_Dimensions.fill(0); }
    TensorShape(unsigned int numDimensions, const unsigned int* dimensionSizes);
    TensorShape(std::initializer_list<unsigned int> dimensionSizeList);
    unsigned int operator[](unsigned int i) const;
    unsigned int& operator[](unsigned int i);
    bool operator==(const TensorShape& other) const;
    bool operator!=(const TensorShape& other) const { return !(*this == other); }
    unsigned int GetNumDimensions() const { return m_NumDimensions; }
    unsigned int GetNumElements() const;
private:
    std::array<unsigned int, 6> m_Dimensions{};
    unsigned int m_NumDimensions;
};

class TensorInfo
{
public:
    TensorInfo() = default;
    explicit TensorInfo(DataType dataType, float quantizationScale = 1.0f, int32_t quantizationOffset = 0, bool isConstant = false);
    TensorInfo(const TensorShape& shape, DataType dataType, float quantizationScale = 1.0f, int32_t quantizationOffset = 0,
               bool isConstant = false);
    TensorInfo(const TensorShape& shape, DataType dataType, const std::vector<float>& quantizationScales,
               unsigned int quantizationDim, bool isConstant = false);
    bool operator==(const TensorInfo& other) const;
    bool operator!=(const TensorInfo& other) const { return !(*this == other); }

    const TensorShape& GetShape() const { return m_Shape; }
    TensorShape& GetShape() { return m_Shape; }
    void SetShape(const TensorShape& s) { m_Shape = s; }
    unsigned int GetNumDimensions() const { return m_Shape.GetNumDimensions(); }
    unsigned int GetNumElements() const { return m_Shape.GetNumElements(); }
    DataType GetDataType() const { return m_DataType; }
    void SetDataType(DataType t) { m_DataType = t; }

    bool HasMultipleQuantizationScales() const { return m_Scales.size() > 1; }
    bool HasPerAxisQuantization() const { return HasMultipleQuantizationScales() || m_QuantizationDim.has_value(); }
    std::vector<float> GetQuantizationScales() const { return m_Scales; }
    void SetQuantizationScales(const std::vector<float>& scales) { m_Scales = scales; }
    float GetQuantizationScale() const;
    void SetQuantizationScale(float scale) { m_Scales = {scale}; }
    int32_t GetQuantizationOffset() const { return m_Offset.has_value() ? m_Offset.value() : 0; }
    void SetQuantizationOffset(int32_t offset) { m_Offset = Optional<int32_t>(offset); }
    Optional<unsigned int> GetQuantizationDim() const { return m_QuantizationDim; }
    void SetQuantizationDim(const Optional<unsigned int>& dim) { m_QuantizationDim = dim; }
    bool IsQuantized() const { return IsQuantizedType(m_DataType); }
    bool IsConstant() const { return m_IsConstant; }
    void SetConstant(const bool isConstant = true) { m_IsConstant = isConstant; }
    bool IsTypeSpaceMatch(const TensorInfo& other) const;
    unsigned int GetNumBytes() const { return GetDataTypeSize(m_DataType) * GetNumElements(); }
private:
    TensorShape m_Shape;
    DataType m_DataType = DataType::Float32;
    bool m_IsConstant = false;
    std::vector<float> m_Scales;
    Optional<int32_t> m_Offset;
    Optional<unsigned int> m_QuantizationDim;
};

using BindingPointInfo = std::pair<armnn::LayerBindingId, armnn::TensorInfo>;

template <typename MemoryType>
class BaseTensor
{
public:
    BaseTensor() : m_MemoryArea(nullptr) {}
    BaseTensor(const TensorInfo& info, MemoryType memoryArea) : m_MemoryArea(memoryArea), m_Info(info) {}
    const TensorInfo& GetInfo() const { return m_Info; }
    TensorInfo& GetInfo() { return m_Info; }
    const TensorShape& GetShape() const { return m_Info.GetShape(); }
    DataType GetDataType() const { return m_Info.GetDataType(); }
    unsigned int GetNumDimensions() const { return m_Info.GetNumDimensions(); }
    unsigned int GetNumBytes() const { return m_Info.GetNumBytes(); }
    unsigned int GetNumElements() const { return m_Info.GetNumElements(); }
    MemoryType GetMemoryArea() const { return m_MemoryArea; }
protected:
    MemoryType m_MemoryArea;
private:
    TensorInfo m_Info;
};

class Tensor : public BaseTensor<void*>
{
public:
    using BaseTensor<void*>::BaseTensor;
};

class ConstTensor : public BaseTensor<const void*>
{
public:
    ConstTensor() = default;
    ConstTensor(const TensorInfo& info, const void* memoryArea) : BaseTensor<const void*>(info, memoryArea)
    {
        if (!GetInfo().IsConstant()) throw InvalidArgumentException("Invalid attempt to construct ConstTensor from non-constant TensorInfo.");
    }
    ConstTensor(const Tensor& other) : BaseTensor<const void*>(other.GetInfo(), other.GetMemoryArea()) {}
};

using InputTensors = std::vector<std::pair<LayerBindingId, class ConstTensor>>;
using OutputTensors = std::vector<std::pair<LayerBindingId, class Tensor>>;
} // namespace armnn
