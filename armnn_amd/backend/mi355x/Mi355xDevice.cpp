#include "Mi355xDevice.hpp"

#include <mutex>

namespace armnn
{
namespace mi355x
{
namespace
{
std::once_flag g_Once;
mi355x_stream_t g_Stream = nullptr;
bool g_Ready = false;
std::string g_Why;
} // namespace

int DeviceCount()
{
    int n = 0;
    if (mi355x_device_count(&n) != 0) return 0;
    return n;
}

void EnsureDevice()
{
    std::call_once(g_Once, [] {
        if (DeviceCount() < 1) { g_Why = "no MI355X device is visible to this process"; return; }
        if (mi355x_init(0) != 0) { g_Why = std::string("device initialisation failed: ") + mi355x_last_error(); return; }
        if (mi355x_stream_create(&g_Stream) != 0) { g_Why = std::string("stream creation failed: ") + mi355x_last_error(); return; }
        g_Ready = true;
    });
    if (!g_Ready) throw BackendUnavailableException("Mi355x backend unavailable: " + g_Why);
}

mi355x_stream_t Stream()
{
    EnsureDevice();
    return g_Stream;
}

void Synchronize() { Check(mi355x_stream_synchronize(Stream()), "mi355x_stream_synchronize"); }

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
