// The allocator a caller-side memory plan gets its buffers from when the caller names no allocator of its own
// (IBackendInternal::GetDefaultAllocator; ClBackendDefaultAllocator, src/backends/cl/ClBackendDefaultAllocator.hpp:13-50,
// and DefaultAllocator, src/backends/backendsCommon/DefaultAllocator.hpp:16-45, are the OpenCL and host counterparts).
// Buffers are device memory: the tensors placed in them are adopted in place by Mi355xTensorHandle::Import.
#pragma once
#include "Mi355xDevice.hpp"

#include <armnn/backends/ICustomAllocator.hpp>

namespace armnn
{
class Mi355xDefaultAllocator : public ICustomAllocator
{
public:
    /// device memory is aligned to 256 bytes, more than any alignment the runtime asks for
    void* allocate(size_t size, size_t /*alignment*/) override
    {
        mi355x::EnsureDevice();
        void* p = nullptr;
        mi355x::Check(mi355x_malloc(&p, size ? size : 1), "mi355x_malloc");
        return p;
    }
    void free(void* ptr) override
    {
        if (!ptr) return;
        mi355x::Synchronize();           // no kernel may still be using the buffer
        mi355x_free(ptr);
    }
    MemorySource GetMemorySourceType() override { return MemorySource::Malloc; }
    void* GetMemoryRegionAtOffset(void* buffer, size_t offset, size_t /*alignment*/ = 0) override
    {
        return static_cast<char*>(buffer) + offset;
    }
};
} // namespace armnn
