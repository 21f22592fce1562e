// Minimal host core: include/armnn/backends/ICustomAllocator.hpp:17-60.
#pragma once
#include "../Exceptions.hpp"
#include "../Types.hpp"
#include <cstddef>
#include <memory>
namespace armnn
{
class ICustomAllocator
{
public:
    virtual ~ICustomAllocator() = default;
    virtual void* allocate(size_t size, size_t alignment) = 0;
    virtual void free(void* ptr) = 0;
    /// MemorySource::Malloc, DmaBuf or DmaBufProtected
    virtual armnn::MemorySource GetMemorySourceType() = 0;
    /// the address `offset` bytes into a buffer this allocator returned
    virtual void* GetMemoryRegionAtOffset(void* /*buffer*/, size_t /*offset*/, size_t /*alignment*/ = 0)
    {
        throw armnn::Exception("ICustomerAllocator::GetMemoryRegionAtOffset(): This function should be overridden in subclass.");
    }
};
} // namespace armnn
