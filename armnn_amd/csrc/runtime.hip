// Device runtime part of the C ABI: device selection, memory, streams, events, graphs.
#include "common.h"

#include <cmath>
#include <mutex>

namespace mi355x
{

char* ErrorBuffer()
{
    static thread_local char buf[512] = {0};
    return buf;
}

int SetError(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(ErrorBuffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

namespace
{
char* KernelNameBuffer()
{
    static thread_local char buf[192] = {0};
    return buf;
}
} // namespace

void NoteKernel(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(KernelNameBuffer(), 192, fmt, ap);
    va_end(ap);
}

int UploadNow(void* dst_dev, const void* src_host, size_t bytes)
{
    // one stream per calling thread, so concurrent plan creations do not wait for each other
    struct Own
    {
        hipStream_t s = nullptr;
        ~Own() { if (s) (void)hipStreamDestroy(s); }
    };
    thread_local Own own;
    if (!own.s) MI355X_HIP(hipStreamCreateWithFlags(&own.s, hipStreamNonBlocking));
    MI355X_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, own.s));
    MI355X_HIP(hipStreamSynchronize(own.s));
    return 0;
}

Options& GlobalOptions()
{
    static Options o;
    return o;
}

int32_t QuantizeHost(float value, float scale, int32_t offset, int32_t dtype)
{
    const float lo = dtype == MI355X_QASYMM_U8 ? 0.0f : -128.0f;
    const float hi = dtype == MI355X_QASYMM_U8 ? 255.0f : 127.0f;
    float q = value / scale;
    float r = static_cast<float>(std::round(static_cast<double>(q)));
    float v = static_cast<float>(offset) + r;
    v = v > lo ? v : lo;
    v = v < hi ? v : hi;
    return static_cast<int32_t>(v);
}

void ActivationClamp(int32_t activation, float a, float b, const mi355x_quant& out, int32_t* lo, int32_t* hi)
{
    const int32_t tmin = out.dtype == MI355X_QASYMM_U8 ? 0 : -128;
    const int32_t tmax = out.dtype == MI355X_QASYMM_U8 ? 255 : 127;
    *lo = tmin;
    *hi = tmax;
    if (activation == MI355X_ACT_RELU)
    {
        *lo = QuantizeHost(0.0f, out.scale, out.offset, out.dtype);
    }
    else if (activation == MI355X_ACT_BOUNDED_RELU)
    {
        *lo = QuantizeHost(b, out.scale, out.offset, out.dtype);
        *hi = QuantizeHost(a, out.scale, out.offset, out.dtype);
    }
}

Requant MakeRequant(const mi355x_quant& out, int32_t activation, float a, float b)
{
    Requant rq;
    rq.out_scale    = out.scale;
    rq.out_offset_f = static_cast<float>(out.offset);
    rq.type_min_f   = out.dtype == MI355X_QASYMM_U8 ? 0.0f : -128.0f;
    rq.type_max_f   = out.dtype == MI355X_QASYMM_U8 ? 255.0f : 127.0f;
    rq.out_is_u8    = out.dtype == MI355X_QASYMM_U8;
    ActivationClamp(activation, a, b, out, &rq.act_lo, &rq.act_hi);
    rq.inv_scale = 1.0f / out.scale;
    rq.act_lo_f  = static_cast<float>(rq.act_lo);
    rq.act_hi_f  = static_cast<float>(rq.act_hi);
    // The tie window argument needs |offset| <= 255 (so that |value/scale| > 512 always clamps) and a normal,
    // finite reciprocal.
    rq.pk_bias = rq.out_is_u8 ? 0 : 128;
    rq.pk_xor  = rq.out_is_u8 ? 0u : 0x80808080u;
    rq.pk_lo_f = static_cast<float>(rq.act_lo + rq.pk_bias);
    rq.pk_hi_f = static_cast<float>(rq.act_hi + rq.pk_bias);
    rq.pk_full = (rq.act_lo + rq.pk_bias == 0 && rq.act_hi + rq.pk_bias == 255) ? 1 : 0;
    rq.fast_ok = !GlobalOptions().exact_division_epilogue && std::isnormal(rq.inv_scale) && std::isnormal(out.scale) && out.offset >= -255 && out.offset <= 255 &&
                 rq.act_lo <= rq.act_hi;
    return rq;
}

__global__ void FillU8Kernel(uint8_t* dst, uint8_t value, size_t n)
{
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) dst[i] = value;
}

} // namespace mi355x

using namespace mi355x;

extern "C" {

const char* mi355x_last_error(void) { return ErrorBuffer(); }

const char* mi355x_last_kernel(void) { return KernelNameBuffer(); }

int mi355x_abi_version(void) { return MI355X_ABI_VERSION; }

int mi355x_set_option(const char* name, int value)
{
    if (!name) return SetError(MI355X_ERR_INVALID_ARGUMENT, "option name is null");
    if (std::strcmp(name, "exact_division_epilogue") == 0) { GlobalOptions().exact_division_epilogue = value != 0; return 0; }
    if (std::strcmp(name, "stem_dot4") == 0) { GlobalOptions().stem_dot4 = value != 0; return 0; }
    if (std::strcmp(name, "chain_stages") == 0)
    {
        if (value < 2 || value > 4) return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain_stages must be 2, 3 or 4");
        GlobalOptions().chain_stages = value;
        return 0;
    }
    if (std::strcmp(name, "igemm_xcd_cols") == 0)
    {
        if (value < 0 || value > 2) return SetError(MI355X_ERR_INVALID_ARGUMENT, "igemm_xcd_cols must be 0, 1 or 2");
        GlobalOptions().igemm_xcd_cols = value;
        return 0;
    }
    if (std::strcmp(name, "dwpw_stream") == 0) { GlobalOptions().dwpw_stream = value != 0; return 0; }
    if (std::strcmp(name, "pwdw_auto") == 0) { GlobalOptions().pwdw_auto = value != 0; return 0; }
    if (std::strcmp(name, "pwdw_mf") == 0)
    {
        if (value != 0 && value != 2 && value != 4 && value != 7) return SetError(MI355X_ERR_INVALID_ARGUMENT, "pwdw_mf must be 0, 2, 4 or 7");
        GlobalOptions().pwdw_mf = value;
        return 0;
    }
    if (std::strcmp(name, "pool_small") == 0) { GlobalOptions().pool_small = value != 0; return 0; }
    if (std::strcmp(name, "pwpool_auto") == 0) { GlobalOptions().pwpool_auto = value != 0; return 0; }
    if (std::strcmp(name, "dwpw_panel") == 0) { GlobalOptions().dwpw_panel = value != 0; return 0; }
    if (std::strcmp(name, "chain_defer_signal") == 0) { GlobalOptions().chain_defer_signal = value != 0; return 0; }
    if (std::strcmp(name, "chain_panel") == 0) { GlobalOptions().chain_panel = value != 0; return 0; }
    if (std::strcmp(name, "chain_blocks_per_cu") == 0)
    {
        if (value < 0 || value > 16) return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain_blocks_per_cu must be 0 .. 16");
        GlobalOptions().chain_blocks_per_cu = value;
        return 0;
    }
    if (std::strcmp(name, "dw_rows") == 0)
    {
        if (value < 0 || value > 2) return SetError(MI355X_ERR_INVALID_ARGUMENT, "dw_rows must be 0, 1 or 2");
        GlobalOptions().dw_rows = value;
        return 0;
    }
    if (std::strcmp(name, "pw_slab") == 0)
    {
        if (value != 0 && value != 32 && value != 64 && value != 128) return SetError(MI355X_ERR_INVALID_ARGUMENT, "pw_slab must be 0, 32, 64 or 128");
        GlobalOptions().pw_slab = value;
        return 0;
    }
    if (std::strcmp(name, "dw_mfma") == 0)
    {
        if (value != 0 && value != 1 && value != 7 && value != 8 && value != 14 && value != 16) return SetError(MI355X_ERR_INVALID_ARGUMENT, "dw_mfma must be 0, 1, 7, 8, 14 or 16");
        GlobalOptions().dw_mfma = value;
        return 0;
    }
    if (std::strcmp(name, "dw_cb") == 0)
    {
        if (value != 0 && value != 32) return SetError(MI355X_ERR_INVALID_ARGUMENT, "dw_cb must be 0 or 32");
        GlobalOptions().dw_cb = value;
        return 0;
    }
    if (std::strcmp(name, "igemm_lds") == 0)
    {
        if (value != 0 && value != 2 && value != 3) return SetError(MI355X_ERR_INVALID_ARGUMENT, "igemm_lds must be 0, 2 or 3");
        GlobalOptions().igemm_lds = value;
        return 0;
    }
    if (std::strcmp(name, "igemm_tile") == 0)
    {
        // 2256, 2128, 1256: the large-tile kernel at 256x256, 256x128, 128x256; 2064 / 4064: 64x64 tiles with K split over 2 / 4
        // groups of waves; 3000 / 3001: the resident-tile kernel (3001: half-height tiles for narrow outputs) where its shape
        // rules allow it (any other forced tile keeps a convolution off that kernel)
        if (value != 0 && value != 64 && value != 96 && value != 128 && value != 256 && value != 512 && value != 2256 && value != 2128 && value != 1256 &&
            value != 3000 && value != 3001 && value != 4064 && value != 2064)
            return SetError(MI355X_ERR_INVALID_ARGUMENT, "igemm_tile must be 0, 64, 96, 128, 256, 512, 2256, 2128, 1256, 3000, 3001, 2064 or 4064");
        GlobalOptions().igemm_tile = value;
        return 0;
    }
    return SetError(MI355X_ERR_INVALID_ARGUMENT, "unknown option '%s'", name);
}

int mi355x_device_count(int* count)
{
    if (!count) return SetError(MI355X_ERR_INVALID_ARGUMENT, "count is null");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess)
    {
        // no driver / no device is not an error for a caller that only wants to know
        (void)hipGetLastError();
        n = 0;
    }
    *count = n;
    return 0;
}

int mi355x_init(int device)
{
    int n = 0;
    mi355x_device_count(&n);
    if (n <= 0) return SetError(MI355X_ERR_NO_DEVICE, "no HIP device available");
    if (device < 0 || device >= n) return SetError(MI355X_ERR_INVALID_ARGUMENT, "device %d out of range [0,%d)", device, n);
    MI355X_HIP(hipSetDevice(device));
    MI355X_HIP(hipFree(nullptr));   // force context creation
    hipDeviceProp_t prop;
    MI355X_HIP(hipGetDeviceProperties(&prop, device));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    {
        return SetError(MI355X_ERR_UNSUPPORTED, "device %d is %s; this library contains gfx950 code only", device,
                        prop.gcnArchName);
    }
    return 0;
}

int mi355x_device_name(char* buf, size_t buf_len)
{
    if (!buf || buf_len == 0) return SetError(MI355X_ERR_INVALID_ARGUMENT, "buffer is null");
    int dev = 0;
    MI355X_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    MI355X_HIP(hipGetDeviceProperties(&prop, dev));
    snprintf(buf, buf_len, "%s", prop.gcnArchName);
    return 0;
}

int mi355x_device_props(int* compute_units, int* clock_khz, size_t* total_mem, size_t* lds_per_cu)
{
    int dev = 0;
    MI355X_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    MI355X_HIP(hipGetDeviceProperties(&prop, dev));
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (total_mem) *total_mem = prop.totalGlobalMem;
    if (lds_per_cu) *lds_per_cu = prop.maxSharedMemoryPerMultiProcessor;
    return 0;
}

int mi355x_malloc(void** ptr_dev, size_t bytes)
{
    if (!ptr_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "ptr is null");
    *ptr_dev = nullptr;
    if (bytes == 0) return 0;
    MI355X_HIP(hipMalloc(ptr_dev, bytes));
    return 0;
}

int mi355x_free(void* ptr_dev)
{
    if (!ptr_dev) return 0;
    MI355X_HIP(hipFree(ptr_dev));
    return 0;
}

int mi355x_host_alloc(void** ptr_host, size_t bytes)
{
    if (!ptr_host) return SetError(MI355X_ERR_INVALID_ARGUMENT, "ptr is null");
    *ptr_host = nullptr;
    if (bytes == 0) return 0;
    MI355X_HIP(hipHostMalloc(ptr_host, bytes, hipHostMallocDefault));
    return 0;
}

int mi355x_host_device_pointer(const void* host_ptr, void** device_ptr, int* is_device_memory)
{
    if (!host_ptr || !device_ptr || !is_device_memory) return SetError(MI355X_ERR_INVALID_ARGUMENT, "null pointer");
    *device_ptr = nullptr;
    *is_device_memory = 0;
    hipPointerAttribute_t attr;
    const hipError_t e = hipPointerGetAttributes(&attr, host_ptr);
    if (e != hipSuccess)
    {
        (void)hipGetLastError();      // an unknown (pageable) pointer is an answer here, not a sticky error
        return SetError(MI355X_ERR_UNSUPPORTED, "pageable host memory is not reachable from the device; allocate it with mi355x_host_alloc");
    }
    if (attr.type == hipMemoryTypeDevice) { *device_ptr = const_cast<void*>(host_ptr); *is_device_memory = 1; return 0; }
    if (attr.type != hipMemoryTypeHost || !attr.devicePointer)
        return SetError(MI355X_ERR_UNSUPPORTED, "memory of this kind is not reachable from the device; allocate it with mi355x_host_alloc");
    *device_ptr = attr.devicePointer;
    return 0;
}

int mi355x_host_free(void* ptr_host)
{
    if (!ptr_host) return 0;
    MI355X_HIP(hipHostFree(ptr_host));
    return 0;
}

static int Copy(void* dst, const void* src, size_t bytes, hipMemcpyKind kind, mi355x_stream_t stream)
{
    if (bytes == 0) return 0;
    if (!dst || !src) return SetError(MI355X_ERR_INVALID_ARGUMENT, "null pointer in copy of %zu bytes", bytes);
    MI355X_HIP(hipMemcpyAsync(dst, src, bytes, kind, ToHip(stream)));
    if (kind != hipMemcpyDeviceToDevice)
    {
        // host buffers may be pageable and reused by the caller right away: complete the copy before returning
        MI355X_HIP(hipStreamSynchronize(ToHip(stream)));
    }
    return 0;
}

int mi355x_memcpy_h2d(void* d, const void* s, size_t n, mi355x_stream_t st) { return Copy(d, s, n, hipMemcpyHostToDevice, st); }
int mi355x_memcpy_d2h(void* d, const void* s, size_t n, mi355x_stream_t st) { return Copy(d, s, n, hipMemcpyDeviceToHost, st); }
int mi355x_memcpy_d2d(void* d, const void* s, size_t n, mi355x_stream_t st) { return Copy(d, s, n, hipMemcpyDeviceToDevice, st); }

static int CopyAsync(void* dst, const void* src, const void* host, size_t bytes, hipMemcpyKind kind, mi355x_stream_t stream)
{
    if (bytes == 0) return 0;
    if (!dst || !src) return SetError(MI355X_ERR_INVALID_ARGUMENT, "null pointer in copy of %zu bytes", bytes);
    void* device_alias = nullptr;
    int is_device = 0;
    if (int rc = mi355x_host_device_pointer(host, &device_alias, &is_device)) return rc;
    MI355X_HIP(hipMemcpyAsync(dst, src, bytes, kind, ToHip(stream)));
    return 0;
}
int mi355x_memcpy_h2d_async(void* d, const void* s, size_t n, mi355x_stream_t st) { return CopyAsync(d, s, s, n, hipMemcpyHostToDevice, st); }
int mi355x_memcpy_d2h_async(void* d, const void* s, size_t n, mi355x_stream_t st) { return CopyAsync(d, s, d, n, hipMemcpyDeviceToHost, st); }

int mi355x_fill_u8(void* dst_dev, uint8_t value, size_t bytes, mi355x_stream_t stream)
{
    if (bytes == 0) return 0;
    if (!dst_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "dst is null");
    size_t blocks = (bytes + 255) / 256;
    if (blocks > 65535) blocks = 65535;
    NoteKernel("FillU8Kernel");
    hipLaunchKernelGGL(FillU8Kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, ToHip(stream),
                       static_cast<uint8_t*>(dst_dev), value, bytes);
    MI355X_HIP(hipGetLastError());
    return 0;
}

int mi355x_stream_create(mi355x_stream_t* stream)
{
    if (!stream) return SetError(MI355X_ERR_INVALID_ARGUMENT, "stream is null");
    hipStream_t s;
    MI355X_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));   // default priority
    *stream = reinterpret_cast<mi355x_stream_t>(s);
    return 0;
}

int mi355x_stream_destroy(mi355x_stream_t stream)
{
    if (!stream) return 0;
    MI355X_HIP(hipStreamDestroy(ToHip(stream)));
    return 0;
}

int mi355x_stream_synchronize(mi355x_stream_t stream)
{
    MI355X_HIP(hipStreamSynchronize(ToHip(stream)));
    return 0;
}

int mi355x_device_synchronize(void)
{
    MI355X_HIP(hipDeviceSynchronize());
    return 0;
}

int mi355x_event_create(mi355x_event_t* event)
{
    if (!event) return SetError(MI355X_ERR_INVALID_ARGUMENT, "event is null");
    hipEvent_t e;
    MI355X_HIP(hipEventCreate(&e));
    *event = reinterpret_cast<mi355x_event_t>(e);
    return 0;
}

int mi355x_event_destroy(mi355x_event_t event)
{
    if (!event) return 0;
    MI355X_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
    return 0;
}

int mi355x_event_record(mi355x_event_t event, mi355x_stream_t stream)
{
    MI355X_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), ToHip(stream)));
    return 0;
}

int mi355x_stream_wait_event(mi355x_stream_t stream, mi355x_event_t event)
{
    MI355X_HIP(hipStreamWaitEvent(ToHip(stream), reinterpret_cast<hipEvent_t>(event), 0));
    return 0;
}

int mi355x_event_synchronize(mi355x_event_t event)
{
    MI355X_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
    return 0;
}

int mi355x_event_elapsed_ms(mi355x_event_t start, mi355x_event_t stop, float* ms)
{
    if (!ms) return SetError(MI355X_ERR_INVALID_ARGUMENT, "ms is null");
    MI355X_HIP(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start), reinterpret_cast<hipEvent_t>(stop)));
    return 0;
}

struct mi355x_graph_s
{
    hipGraph_t     graph = nullptr;
    hipGraphExec_t exec  = nullptr;
};

int mi355x_graph_capture_begin(mi355x_stream_t stream)
{
    if (!stream) return SetError(MI355X_ERR_INVALID_ARGUMENT, "graph capture needs a non-default stream");
    MI355X_HIP(hipStreamBeginCapture(ToHip(stream), hipStreamCaptureModeThreadLocal));
    return 0;
}

int mi355x_graph_capture_end(mi355x_stream_t stream, mi355x_graph_t* graph)
{
    if (!graph) return SetError(MI355X_ERR_INVALID_ARGUMENT, "graph is null");
    *graph = nullptr;
    hipGraph_t g = nullptr;
    MI355X_HIP(hipStreamEndCapture(ToHip(stream), &g));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    if (e != hipSuccess)
    {
        (void)hipGraphDestroy(g);
        return HipFail(e, "hipGraphInstantiate");
    }
    auto* out = new mi355x_graph_s;
    out->graph = g;
    out->exec = exec;
    *graph = out;
    return 0;
}

int mi355x_graph_launch(mi355x_graph_t graph, mi355x_stream_t stream)
{
    if (!graph) return SetError(MI355X_ERR_INVALID_ARGUMENT, "graph is null");
    MI355X_HIP(hipGraphLaunch(graph->exec, ToHip(stream)));
    return 0;
}

int mi355x_graph_destroy(mi355x_graph_t graph)
{
    if (!graph) return 0;
    if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph) (void)hipGraphDestroy(graph->graph);
    delete graph;
    return 0;
}

} // extern "C"
