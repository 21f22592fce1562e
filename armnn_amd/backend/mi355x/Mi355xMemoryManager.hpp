// IMemoryManager of the Mi355x backend: one device arena for all managed (intermediate) tensors of a network.
//
// Tensor handles reserve a range when their lifetime starts (ITensorHandle::Manage) and give it back when it ends
// (ITensorHandle::Allocate, which the graph calls after the last consumer), so tensors whose lifetimes do not overlap
// share addresses -- the same protocol RefMemoryManager implements with host pools
// (src/backends/reference/RefMemoryManager.cpp:20-101).  Acquire() allocates the arena at its high-water size,
// Release() returns it.  Address reuse is safe when the kernels of a network run in order on one stream; the backend turns
// it off when networks run in lanes.
#pragma once
#include <armnn/backends/IMemoryManager.hpp>

#include <cstddef>
#include <map>

namespace armnn
{
class Mi355xMemoryManager : public IMemoryManager
{
public:
    /// shareAddresses = false gives every tensor a range of its own.  That is what networks running in lanes need: the
    /// lanes are at different layers at the same moment, so a tensor retired for one of them may still be read by another.
    explicit Mi355xMemoryManager(bool shareAddresses = true);
    ~Mi355xMemoryManager() override;

    /// start of a lifetime: returns the offset of a free range of `bytes` (first fit, 256-byte granules)
    size_t Reserve(size_t bytes);
    /// end of a lifetime: the range may be handed out again once the NEXT lifetime has ended (see the definition)
    void Retire(size_t offset, size_t bytes);
    /// device address of `offset`; throws MemoryValidationException before Acquire()
    void* Resolve(size_t offset) const;

    void Acquire() override;
    void Release() override;

    size_t ArenaBytes() const { return m_HighWater; }
    size_t ReservedTotal() const { return m_ReservedTotal; }   ///< sum of all reservations (what no reuse would cost)

private:
    static size_t Granules(size_t bytes) { return (bytes + 255) / 256 * 256; }
    void Free(size_t offset, size_t bytes);
    static constexpr size_t kNothingPending = ~static_cast<size_t>(0);
    size_t m_PendingOffset = 0, m_PendingBytes = kNothingPending;     // the range retired last, not yet free
    const bool m_Share;
    std::map<size_t, size_t> m_Free;     // offset -> length of free ranges below the high-water mark
    size_t m_HighWater = 0;
    size_t m_ReservedTotal = 0;
    void* m_Arena = nullptr;
    size_t m_ArenaSize = 0;
};
} // namespace armnn
