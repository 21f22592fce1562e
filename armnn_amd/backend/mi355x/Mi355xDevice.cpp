#include "Mi355xDevice.hpp"

#include <atomic>
#include <cstdint>
#include <cstdlib>
#include <map>
#include <mutex>

namespace armnn
{
namespace mi355x
{
namespace
{
std::once_flag g_Once;
mi355x_stream_t g_Streams[kMaxLanes] = {nullptr, nullptr, nullptr, nullptr};
std::atomic<unsigned int> g_Lanes{0};          // 0: not decided yet
std::atomic<int> g_SharingArenas{0};
std::atomic<unsigned long long> g_Epoch{1};
bool g_Ready = false;
std::string g_Why;

// per thread: whether its lanes are running apart, and the events it orders them with
struct LaneState
{
    bool forked = false;
    unsigned int count = 1;         // lanes running since the last Fork()
    mi355x_event_t fork = nullptr;
    mi355x_event_t lane[kMaxLanes] = {nullptr, nullptr, nullptr, nullptr};
    mi355x_event_t Event(mi355x_event_t& e)
    {
        if (!e) Check(mi355x_event_create(&e), "mi355x_event_create");
        return e;
    }
};
thread_local LaneState t_Lanes;
} // namespace

int DeviceCount()
{
    int n = 0;
    if (mi355x_device_count(&n) != 0) return 0;
    return n;
}

namespace
{
std::atomic<bool> g_Assume{false};
}

void AssumeDevice(bool assume) { g_Assume.store(assume); }

bool DeviceUsable()
{
    static const bool present = DeviceCount() > 0;
    return present || g_Assume.load();
}

void EnsureDevice()
{
    std::call_once(g_Once, [] {
        if (DeviceCount() < 1) { g_Why = "no MI355X device is visible to this process"; return; }
        if (mi355x_init(0) != 0) { g_Why = std::string("device initialisation failed: ") + mi355x_last_error(); return; }
        for (mi355x_stream_t& s : g_Streams)
            if (mi355x_stream_create(&s) != 0) { g_Why = std::string("stream creation failed: ") + mi355x_last_error(); return; }
        g_Ready = true;
    });
    if (!g_Ready) throw BackendUnavailableException("Mi355x backend unavailable: " + g_Why);
}

mi355x_stream_t Stream()
{
    EnsureDevice();
    Join();
    return g_Streams[0];
}

unsigned int Lanes()
{
    unsigned int n = g_Lanes.load();
    if (n == 0)
    {
        n = 2;
        if (const char* env = std::getenv("MI355X_LANES"))
        {
            const int v = std::atoi(env);
            if (v >= 1 && v <= static_cast<int>(kMaxLanes)) n = static_cast<unsigned int>(v);
        }
        g_Lanes.store(n);
    }
    return n;
}

void SetLanes(unsigned int lanes)
{
    if (lanes < 1 || lanes > kMaxLanes) throw InvalidArgumentException("Mi355x: the number of lanes must be 1.." + std::to_string(kMaxLanes));
    if (lanes > 1 && g_SharingArenas.load() > 0)
        throw InvalidArgumentException("Mi355x: lanes cannot be turned on while a network loaded for one stream is alive");
    if (g_Ready) Join();
    g_Lanes.store(lanes);
}

void CountAddressSharingArena(int delta) { g_SharingArenas.fetch_add(delta); }

namespace
{
std::mutex g_RangeMutex;
std::multimap<uintptr_t, uintptr_t> g_Ranges;       // begin -> end of every adopted device range alive
std::atomic<int> g_OverlappingRanges{0};
}

bool NoteAdoptedRange(const void* begin, size_t bytes)
{
    const uintptr_t b = reinterpret_cast<uintptr_t>(begin), e = b + (bytes ? bytes : 1);
    std::lock_guard<std::mutex> lock(g_RangeMutex);
    bool overlap = false;
    for (const auto& r : g_Ranges)
    {
        if (r.first >= e) break;
        if (r.second > b) { overlap = true; break; }
    }
    g_Ranges.emplace(b, e);
    if (overlap) g_OverlappingRanges.fetch_add(1);
    return overlap;
}

void ForgetAdoptedRange(const void* begin, size_t bytes, bool overlapped)
{
    const uintptr_t b = reinterpret_cast<uintptr_t>(begin), e = b + (bytes ? bytes : 1);
    std::lock_guard<std::mutex> lock(g_RangeMutex);
    auto range = g_Ranges.equal_range(b);
    for (auto it = range.first; it != range.second; ++it)
        if (it->second == e) { g_Ranges.erase(it); break; }
    if (overlapped) g_OverlappingRanges.fetch_sub(1);
}

unsigned int LanesFor(unsigned int batch)
{
    const unsigned int n = Lanes();
    if (g_OverlappingRanges.load() != 0) return 1u;
    return (n > 1 && batch % n == 0 && batch / n >= kMinLaneBatch) ? n : 1u;
}

mi355x_stream_t LaneStream(unsigned int lane)
{
    EnsureDevice();
    if (lane >= kMaxLanes) throw InvalidArgumentException("Mi355x: no such lane");
    return g_Streams[lane];
}

void Fork()
{
    EnsureDevice();
    LaneState& st = t_Lanes;
    if (st.forked) return;
    const unsigned int n = Lanes();
    if (n > 1)
    {
        Check(mi355x_event_record(st.Event(st.fork), g_Streams[0]), "mi355x_event_record");
        for (unsigned int k = 1; k < n; ++k) Check(mi355x_stream_wait_event(g_Streams[k], st.fork), "mi355x_stream_wait_event");
    }
    st.forked = true;
    st.count = n;
}

void Join()
{
    LaneState& st = t_Lanes;
    if (!st.forked) return;
    for (unsigned int k = 1; k < st.count; ++k)
    {
        Check(mi355x_event_record(st.Event(st.lane[k]), g_Streams[k]), "mi355x_event_record");
        Check(mi355x_stream_wait_event(g_Streams[0], st.lane[k]), "mi355x_stream_wait_event");
    }
    st.forked = false;
}

void UploadInLanes(void* dstDevice, const void* srcHost, size_t bytes, unsigned int lanes)
{
    if (lanes <= 1 || bytes % lanes != 0)
    {
        Check(mi355x_memcpy_h2d_async(dstDevice, srcHost, bytes, Stream()), "mi355x_memcpy_h2d_async");
        return;
    }
    Fork();
    LaneState& st = t_Lanes;
    const size_t part = bytes / lanes;
    mi355x_stream_t queue = g_Streams[lanes - 1];
    for (unsigned int k = 0; k < lanes; ++k)
    {
        Check(mi355x_memcpy_h2d_async(static_cast<unsigned char*>(dstDevice) + k * part, static_cast<const unsigned char*>(srcHost) + k * part, part, queue),
              "mi355x_memcpy_h2d");
        if (k + 1 < lanes)
        {
            Check(mi355x_event_record(st.Event(st.lane[k]), queue), "mi355x_event_record");
            Check(mi355x_stream_wait_event(g_Streams[k], st.lane[k]), "mi355x_stream_wait_event");
        }
    }
}

void Synchronize()
{
    Check(mi355x_stream_synchronize(Stream()), "mi355x_stream_synchronize");
    g_Epoch.fetch_add(1);
}

unsigned long long SyncEpoch() { return g_Epoch.load(); }

void Check(int status, const char* what)
{
    if (status != 0)
        throw RuntimeException(std::string(what) + " failed (" + std::to_string(status) + "): " + mi355x_last_error());
}

int32_t ToDType(DataType t)
{
    switch (t)
    {
        case DataType::QAsymmS8: return MI355X_QASYMM_S8;
        case DataType::QAsymmU8: return MI355X_QASYMM_U8;
        case DataType::QSymmS8: return MI355X_QSYMM_S8;
        case DataType::Signed32: return MI355X_SIGNED32;
        default: throw InvalidArgumentException(std::string("Mi355x: unsupported data type ") + GetDataTypeName(t));
    }
}

mi355x_quant ToQuant(const TensorInfo& info)
{
    if (info.GetDataType() != DataType::QAsymmS8 && info.GetDataType() != DataType::QAsymmU8)
        throw InvalidArgumentException(std::string("Mi355x: activation tensors must be QAsymmS8 or QAsymmU8, got ") + GetDataTypeName(info.GetDataType()));
    mi355x_quant q;
    q.dtype = ToDType(info.GetDataType());
    q.scale = info.GetQuantizationScale();
    q.offset = info.GetQuantizationOffset();
    return q;
}
} // namespace mi355x
} // namespace armnn
