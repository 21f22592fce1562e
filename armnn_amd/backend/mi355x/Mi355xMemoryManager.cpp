#include "Mi355xMemoryManager.hpp"
#include "Mi355xDevice.hpp"

namespace armnn
{
Mi355xMemoryManager::Mi355xMemoryManager(bool shareAddresses) : m_Share(shareAddresses)
{
    if (m_Share) mi355x::CountAddressSharingArena(+1);
}

Mi355xMemoryManager::~Mi355xMemoryManager()
{
    if (m_Share) mi355x::CountAddressSharingArena(-1);
    if (m_Arena) mi355x_free(m_Arena);
}

size_t Mi355xMemoryManager::Reserve(size_t bytes)
{
    const size_t need = Granules(bytes ? bytes : 1);
    m_ReservedTotal += need;
    for (auto it = m_Free.begin(); it != m_Free.end(); ++it)
    {
        if (it->second < need) continue;
        const size_t offset = it->first;
        const size_t rest = it->second - need;
        m_Free.erase(it);
        if (rest) m_Free[offset + need] = rest;
        return offset;
    }
    // grow: a free range that touches the high-water mark is extended instead of left behind
    size_t offset = m_HighWater;
    if (!m_Free.empty())
    {
        auto last = std::prev(m_Free.end());
        if (last->first + last->second == m_HighWater)
        {
            offset = last->first;
            m_Free.erase(last);
        }
    }
    m_HighWater = offset + need;
    return offset;
}

void Mi355xMemoryManager::Retire(size_t offset, size_t bytes)
{
    if (!m_Share) return;
    // A range becomes free one retirement late.  The runtime ends a tensor's lifetime behind its last consumer and starts
    // the next layer's output before it retires anything else, so the output of the layer BEHIND that consumer never lies
    // over the retired tensor: a depthwise layer's input and the output of the pointwise convolution that follows do not
    // overlap, and the convolution workload can run the pair as one launch.
    std::swap(offset, m_PendingOffset);
    std::swap(bytes, m_PendingBytes);
    if (bytes == kNothingPending) return;
    Free(offset, bytes);
}

void Mi355xMemoryManager::Free(size_t offset, size_t bytes)
{
    size_t len = Granules(bytes ? bytes : 1);
    auto next = m_Free.lower_bound(offset);
    if (next != m_Free.begin())
    {
        auto prev = std::prev(next);
        if (prev->first + prev->second == offset)
        {
            offset = prev->first;
            len += prev->second;
            m_Free.erase(prev);
        }
    }
    if (next != m_Free.end() && offset + len == next->first)
    {
        len += next->second;
        m_Free.erase(next);
    }
    m_Free[offset] = len;
}

void* Mi355xMemoryManager::Resolve(size_t offset) const
{
    if (!m_Arena) throw MemoryValidationException("Mi355xMemoryManager: tensor memory used before Acquire()");
    if (offset >= m_ArenaSize) throw MemoryValidationException("Mi355xMemoryManager: tensor lies outside the acquired arena");
    return static_cast<unsigned char*>(m_Arena) + offset;
}

void Mi355xMemoryManager::Acquire()
{
    if (m_Arena && m_ArenaSize >= m_HighWater) return;
    if (m_Arena) { mi355x::Check(mi355x_free(m_Arena), "mi355x_free"); m_Arena = nullptr; }
    mi355x::EnsureDevice();
    m_ArenaSize = m_HighWater ? m_HighWater : 256;
    mi355x::Check(mi355x_malloc(&m_Arena, m_ArenaSize), "mi355x_malloc(arena)");
}

void Mi355xMemoryManager::Release()
{
    if (!m_Arena) return;
    mi355x::Synchronize();
    mi355x::Check(mi355x_free(m_Arena), "mi355x_free");
    m_Arena = nullptr;
    m_ArenaSize = 0;
}
} // namespace armnn
