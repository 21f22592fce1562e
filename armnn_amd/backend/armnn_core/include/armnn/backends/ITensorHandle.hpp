// Minimal host core: include/armnn/backends/ITensorHandle.hpp:16-103.
#pragma once
#include "../Tensor.hpp"
#include "../Types.hpp"
#include "../utility/IgnoreUnused.hpp"
#include <memory>

namespace armnn
{
class ITensorHandle
{
public:
    virtual ~ITensorHandle() {}
    /// marks the start of the tensor's lifetime for the memory manager; must precede Allocate()
    virtual void Manage() = 0;
    virtual void Allocate() = 0;
    virtual ITensorHandle* GetParent() const = 0;
    virtual const void* Map(bool blocking = true) const = 0;
    virtual void Unmap() const = 0;
    void* Map(bool blocking = true) { return const_cast<void*>(static_cast<const ITensorHandle*>(this)->Map(blocking)); }
    void Unmap() { return static_cast<const ITensorHandle*>(this)->Unmap(); }
    virtual TensorShape GetStrides() const = 0;
    virtual TensorShape GetShape() const = 0;
    virtual void CopyOutTo(void* memory) const = 0;
    virtual void CopyInFrom(const void* memory) = 0;
    virtual unsigned int GetImportFlags() const { return 0; }
    virtual bool Import(void* memory, MemorySource source) { IgnoreUnused(memory, source); return false; }
    virtual bool CanBeImported(void* memory, MemorySource source) { IgnoreUnused(memory, source); return false; }
    virtual void Unimport() {}
    virtual std::shared_ptr<ITensorHandle> DecorateTensorHandle(const TensorInfo& tensorInfo) { IgnoreUnused(tensorInfo); return nullptr; }
};
} // namespace armnn
