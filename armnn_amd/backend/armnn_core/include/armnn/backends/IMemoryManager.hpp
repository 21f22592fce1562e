// Minimal host core: include/armnn/backends/IMemoryManager.hpp:12-22.
#pragma once
namespace armnn
{
class IMemoryManager
{
protected:
    IMemoryManager() {}
public:
    virtual void Acquire() = 0;
    virtual void Release() = 0;
    virtual ~IMemoryManager() {}
};
} // namespace armnn
