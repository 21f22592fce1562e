// Minimal host core: include/armnn/backends/IMemoryOptimizerStrategy.hpp:13-51.  A strategy places blocks (a size and
// the first and last step of the network at which the block is alive) into bins; blocks of one bin whose lifetimes do
// not meet may overlap in address.
#pragma once
#include "../Types.hpp"
#include <string>
#include <vector>
namespace armnn
{
struct MemBlock
{
    MemBlock(unsigned int startOfLife, unsigned int endOfLife, size_t memSize, size_t offset, unsigned int index)
        : m_StartOfLife(startOfLife), m_EndOfLife(endOfLife), m_MemSize(memSize), m_Offset(offset), m_Index(index) {}
    const unsigned int m_StartOfLife;   // inclusive
    const unsigned int m_EndOfLife;     // inclusive
    const size_t m_MemSize;
    size_t m_Offset;
    const unsigned int m_Index;         // keeps the order of the tensors
};
struct MemBin
{
    std::vector<MemBlock> m_MemBlocks;
    size_t m_MemSize;
};
class IMemoryOptimizerStrategy
{
public:
    virtual ~IMemoryOptimizerStrategy() {}
    virtual std::string GetName() const = 0;
    virtual MemBlockStrategyType GetMemBlockStrategyType() const = 0;
    virtual std::vector<MemBin> Optimize(std::vector<MemBlock>& memBlocks) = 0;
};
} // namespace armnn
