// Minimal host core: ConstTensorHandle / ScopedTensorHandle (include/armnn/backends/TensorHandle.hpp) -- host-memory
// handles that carry a Constant layer's data until the owning backend uploads it.
#pragma once
#include "ITensorHandle.hpp"
#include <cstring>
#include <vector>

namespace armnn
{
TensorShape GetUnpaddedTensorStrides(const TensorInfo& tensorInfo);

class ConstTensorHandle : public ITensorHandle
{
public:
    template <typename T>
    const T* GetConstTensor() const { return reinterpret_cast<const T*>(m_Memory); }
    const TensorInfo& GetTensorInfo() const { return m_TensorInfo; }
    void Manage() override {}
    ITensorHandle* GetParent() const override { return nullptr; }
    const void* Map(bool) const override { return m_Memory; }
    void Unmap() const override {}
    TensorShape GetStrides() const override { return GetUnpaddedTensorStrides(m_TensorInfo); }
    TensorShape GetShape() const override { return m_TensorInfo.GetShape(); }
    void CopyOutTo(void* memory) const override { std::memcpy(memory, m_Memory, m_TensorInfo.GetNumBytes()); }
    void CopyInFrom(const void*) override { throw InvalidArgumentException("ConstTensorHandle is read-only"); }
    void Allocate() override {}
protected:
    ConstTensorHandle(const TensorInfo& tensorInfo) : m_TensorInfo(tensorInfo), m_Memory(nullptr) {}
    ~ConstTensorHandle() {}
    void SetConstMemory(const void* mem) { m_Memory = mem; }
private:
    TensorInfo m_TensorInfo;
    const void* m_Memory;
};

/// owns a copy of the constant data
class ScopedTensorHandle : public ConstTensorHandle
{
public:
    explicit ScopedTensorHandle(const ConstTensor& tensor) : ConstTensorHandle(tensor.GetInfo()), m_Data(tensor.GetNumBytes())
    {
        if (tensor.GetNumBytes()) std::memcpy(m_Data.data(), tensor.GetMemoryArea(), tensor.GetNumBytes());
        SetConstMemory(m_Data.data());
    }
    ~ScopedTensorHandle() {}
private:
    std::vector<unsigned char> m_Data;
};
} // namespace armnn
