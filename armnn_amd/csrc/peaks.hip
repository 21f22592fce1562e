// Micro-benchmarks that measure what this device delivers at its actual clocks, for reading roofline fractions:
//   * int8 MFMA issue rate: every wave runs independent v_mfma_i32_32x32x32_i8 chains on register operands only;
//   * the same with the operands read from LDS every step (2 + 4 fragments per 8 MFMAs, as a GEMM wave tile does):
//     the clock the device sustains with the matrix cores and LDS busy together is lower, and so is this rate;
//   * HBM copy rate: 16-byte loads and stores over buffers far larger than the caches.
// Measurement support for the benchmark scripts; not part of the inference ABI.
#include <hip/hip_runtime.h>
#include <cstdint>

namespace
{
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// ops per wave and iteration: 4 MFMAs x 32*32*32 MACs x 2
__global__ __launch_bounds__(256) void MfmaPeakKernel(int iters, int* sink)
{
    const int lane = threadIdx.x;
    v4i a = {lane, lane + 1, lane + 2, lane + 3};
    v4i b = {lane ^ 5, lane ^ 9, lane ^ 17, lane ^ 33};
    v16i c0 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, c1 = c0, c2 = c0, c3 = c0;
    for (int i = 0; i < iters; ++i)
    {
        c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c3, 0, 0, 0);
    }
    const v16i s = c0 + c1 + c2 + c3;
    int t = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) t += s[i];
    if (t == 0x7fffffff) sink[0] = t;          // keeps the chains alive; practically never taken
}

// The same chains with operands whose bytes are either all small (as above) or spread over the whole int8 range, and
// with the shader clock read at both ends: the matrix cores' power draw depends on how many operand bits toggle, and the
// clock the device sustains follows it.  cyc[0] receives block 0's cycle count, cyc[1] its 100 MHz wall-clock ticks.
__global__ __launch_bounds__(256) void MfmaDataKernel(int iters, int spread, int* sink, long long* cyc)
{
    const int lane = threadIdx.x;
    const unsigned h = (static_cast<unsigned>(lane) + 1u) * 2654435761u;
    v4i a = {lane, lane + 1, lane + 2, lane + 3};
    v4i b = {lane ^ 5, lane ^ 9, lane ^ 17, lane ^ 33};
    if (spread)
    {
        a = v4i{static_cast<int>(h), static_cast<int>(h * 40503u + 7u), static_cast<int>(h ^ 0x9e3779b9u), static_cast<int>(h * 2246822519u)};
        b = v4i{static_cast<int>(h * 3266489917u), static_cast<int>(~h), static_cast<int>(h * 668265263u + 1u), static_cast<int>(h ^ 0x85ebca6bu)};
    }
    v16i c0 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, c1 = c0, c2 = c0, c3 = c0;
    const long long t0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    for (int i = 0; i < iters; ++i)
    {
        c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c3, 0, 0, 0);
    }
    const v16i s = c0 + c1 + c2 + c3;
    int t = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) t += s[i];
    if (t == 0x7fffffff) sink[0] = t;
    if (blockIdx.x == 0 && threadIdx.x == 0)
    {
        cyc[0] = __builtin_readcyclecounter() - t0;
        cyc[1] = wall_clock64() - w0;
    }
}

// four 16-byte loads in flight per thread, non-temporal both ways (the fastest of the variants tried on this device)
// ops per wave and iteration: 8 MFMAs x 32*32*32 MACs x 2; 6 ds_read_b128 per iteration
__global__ __launch_bounds__(256) void MfmaLdsFedKernel(int iters, int* sink)
{
    __shared__ __attribute__((aligned(16))) int lds[16384];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < 16384; i += 256) lds[i] = static_cast<int>(i * 2654435761u);
    __syncthreads();
    v16i c[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) c[i][j] = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const int base = wave * 4096 + lane * 4;
    for (int it = 0; it < iters; ++it)
    {
        const int o = (it & 3) * 1024;
        v4i fa[2], fb[4];
#pragma unroll
        for (int i = 0; i < 2; ++i) fa[i] = *reinterpret_cast<const v4i*>(&lds[(base + o + 256 * i) & 16383]);
#pragma unroll
        for (int j = 0; j < 4; ++j) fb[j] = *reinterpret_cast<const v4i*>(&lds[(base + o + 256 * (2 + j)) & 16383]);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) c[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], c[i][j], 0, 0, 0);
    }
    int t = 0;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int k = 0; k < 16; ++k) t += c[i][j][k];
    if (t == 0x7fffffff) sink[0] = t;
}

__global__ __launch_bounds__(256) void CopyKernel(const v4i* __restrict__ src, v4i* __restrict__ dst, size_t n16)
{
    size_t i = static_cast<size_t>(blockIdx.x) * 1024 + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * 1024;
    for (; i + 768 < n16; i += stride)
    {
        v4i t[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) t[u] = __builtin_nontemporal_load(src + i + u * 256);
#pragma unroll
        for (int u = 0; u < 4; ++u) __builtin_nontemporal_store(t[u], dst + i + u * 256);
    }
}

// four loads in flight per thread and pass; the xor keeps them alive
__global__ __launch_bounds__(256) void ReadKernel(const v4i* __restrict__ src, size_t n16, int* sink)
{
    size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    v4i acc = {0, 0, 0, 0};
    for (; i + 3 * stride < n16; i += 4 * stride)
    {
        const v4i a = __builtin_nontemporal_load(src + i), b = __builtin_nontemporal_load(src + i + stride),
                  c = __builtin_nontemporal_load(src + i + 2 * stride), d = __builtin_nontemporal_load(src + i + 3 * stride);
        acc ^= a ^ b ^ c ^ d;
    }
    for (; i < n16; i += stride) acc ^= src[i];
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678) sink[0] = 1;
}

struct Events
{
    hipEvent_t e0 = nullptr, e1 = nullptr;
    bool ok = false;
    Events() { ok = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess; }
    ~Events()
    {
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
    }
};
} // namespace

extern "C"
{
// Dense int8 MFMA rate in ops/s (2 ops per multiply-accumulate) with `waves_per_simd` waves on every SIMD.
int mi355x_peak_mfma_i8(int waves_per_simd, double* ops_per_s)
{
    if (!ops_per_s || waves_per_simd < 1 || waves_per_simd > 8) return 1;
    int dev = 0, n_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 2;
    if (hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 2;
    int* sink = nullptr;
    if (hipMalloc(&sink, 64) != hipSuccess) return 2;
    Events ev;
    const int iters = 20000;
    const dim3 grid(static_cast<unsigned>(n_cu * waves_per_simd));      // 256 threads = 4 waves = one per SIMD
    int rc = ev.ok ? 0 : 2;
    if (rc == 0)
    {
        hipLaunchKernelGGL(MfmaPeakKernel, grid, dim3(256), 0, nullptr, 200, sink);      // warm-up
        (void)hipEventRecord(ev.e0, nullptr);
        hipLaunchKernelGGL(MfmaPeakKernel, grid, dim3(256), 0, nullptr, iters, sink);
        (void)hipEventRecord(ev.e1, nullptr);
        float ms = 0.0f;
        if (hipEventSynchronize(ev.e1) != hipSuccess || hipEventElapsedTime(&ms, ev.e0, ev.e1) != hipSuccess || ms <= 0.0f) rc = 2;
        else *ops_per_s = static_cast<double>(grid.x) * 4.0 * iters * 4.0 * 65536.0 / (ms * 1e-3);
    }
    (void)hipFree(sink);
    return rc;
}

// Register-only int8 MFMA rate in ops/s, one wave per SIMD, with small operand bytes (spread = 0) or operand bytes over
// the whole range (spread = 1), and the shader clock in GHz that block 0 saw meanwhile.
int mi355x_peak_mfma_i8_data(int spread, double* ops_per_s, double* clock_ghz)
{
    if (!ops_per_s || !clock_ghz) return 1;
    int dev = 0, n_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 2;
    if (hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 2;
    int* sink = nullptr;
    long long* cyc = nullptr;
    if (hipMalloc(&sink, 64) != hipSuccess) return 2;
    if (hipMalloc(&cyc, 16) != hipSuccess) { (void)hipFree(sink); return 2; }
    Events ev;
    const int iters = 40000;
    const dim3 grid(static_cast<unsigned>(n_cu));
    int rc = ev.ok ? 0 : 2;
    if (rc == 0)
    {
        hipLaunchKernelGGL(MfmaDataKernel, grid, dim3(256), 0, nullptr, 4000, spread, sink, cyc);      // warm-up
        (void)hipEventRecord(ev.e0, nullptr);
        hipLaunchKernelGGL(MfmaDataKernel, grid, dim3(256), 0, nullptr, iters, spread, sink, cyc);
        (void)hipEventRecord(ev.e1, nullptr);
        float ms = 0.0f;
        long long host[2] = {0, 0};
        if (hipEventSynchronize(ev.e1) != hipSuccess || hipEventElapsedTime(&ms, ev.e0, ev.e1) != hipSuccess || ms <= 0.0f ||
            hipMemcpy(host, cyc, sizeof(host), hipMemcpyDeviceToHost) != hipSuccess || host[1] <= 0) rc = 2;
        else
        {
            *ops_per_s = static_cast<double>(grid.x) * 4.0 * iters * 4.0 * 65536.0 / (ms * 1e-3);
            *clock_ghz = static_cast<double>(host[0]) / (static_cast<double>(host[1]) * 10.0);      // cycles per 10 ns tick
        }
    }
    (void)hipFree(sink);
    (void)hipFree(cyc);
    return rc;
}

// Dense int8 MFMA rate in ops/s when every operand fragment comes from LDS (two waves per SIMD).
int mi355x_peak_mfma_i8_lds_fed(double* ops_per_s)
{
    if (!ops_per_s) return 1;
    int dev = 0, n_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 2;
    if (hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 2;
    int* sink = nullptr;
    if (hipMalloc(&sink, 64) != hipSuccess) return 2;
    Events ev;
    const int iters = 10000;
    const dim3 grid(static_cast<unsigned>(n_cu * 2));
    int rc = ev.ok ? 0 : 2;
    if (rc == 0)
    {
        hipLaunchKernelGGL(MfmaLdsFedKernel, grid, dim3(256), 0, nullptr, 100, sink);
        (void)hipEventRecord(ev.e0, nullptr);
        hipLaunchKernelGGL(MfmaLdsFedKernel, grid, dim3(256), 0, nullptr, iters, sink);
        (void)hipEventRecord(ev.e1, nullptr);
        float ms = 0.0f;
        if (hipEventSynchronize(ev.e1) != hipSuccess || hipEventElapsedTime(&ms, ev.e0, ev.e1) != hipSuccess || ms <= 0.0f) rc = 2;
        else *ops_per_s = static_cast<double>(grid.x) * 4.0 * iters * 8.0 * 65536.0 / (ms * 1e-3);
    }
    (void)hipFree(sink);
    return rc;
}

// HBM read rate in bytes/s over a buffer of `bytes`.
int mi355x_peak_hbm_read(size_t bytes, double* bytes_per_s)
{
    if (!bytes_per_s || bytes < (1u << 20) || (bytes & 15) != 0) return 1;
    void* src = nullptr;
    int* sink = nullptr;
    if (hipMalloc(&src, bytes) != hipSuccess) return 2;
    if (hipMalloc(&sink, 64) != hipSuccess) { (void)hipFree(src); return 2; }
    Events ev;
    int rc = ev.ok && hipMemset(src, 1, bytes) == hipSuccess ? 0 : 2;
    if (rc == 0)
    {
        const size_t n16 = bytes / 16;
        const dim3 grid(256 * 16);
        const int reps = 10;
        hipLaunchKernelGGL(ReadKernel, grid, dim3(256), 0, nullptr, static_cast<const v4i*>(src), n16, sink);
        (void)hipEventRecord(ev.e0, nullptr);
        for (int r = 0; r < reps; ++r)
            hipLaunchKernelGGL(ReadKernel, grid, dim3(256), 0, nullptr, static_cast<const v4i*>(src), n16, sink);
        (void)hipEventRecord(ev.e1, nullptr);
        float ms = 0.0f;
        if (hipEventSynchronize(ev.e1) != hipSuccess || hipEventElapsedTime(&ms, ev.e0, ev.e1) != hipSuccess || ms <= 0.0f) rc = 2;
        else *bytes_per_s = static_cast<double>(bytes) * reps / (ms * 1e-3);
    }
    (void)hipFree(src);
    (void)hipFree(sink);
    return rc;
}

// HBM copy rate in bytes/s, counting the bytes read plus the bytes written, over `bytes` per buffer (a multiple of 16 KiB).
int mi355x_peak_hbm_copy(size_t bytes, double* bytes_per_s)
{
    if (!bytes_per_s || bytes < (1u << 20) || (bytes & 16383) != 0) return 1;
    void *src = nullptr, *dst = nullptr;
    if (hipMalloc(&src, bytes) != hipSuccess) return 2;
    if (hipMalloc(&dst, bytes) != hipSuccess) { (void)hipFree(src); return 2; }
    Events ev;
    int rc = ev.ok && hipMemset(src, 1, bytes) == hipSuccess ? 0 : 2;
    if (rc == 0)
    {
        const size_t n16 = bytes / 16;
        const dim3 grid(256 * 16);
        const int reps = 10;
        hipLaunchKernelGGL(CopyKernel, grid, dim3(256), 0, nullptr, static_cast<const v4i*>(src), static_cast<v4i*>(dst), n16);
        (void)hipEventRecord(ev.e0, nullptr);
        for (int r = 0; r < reps; ++r)
            hipLaunchKernelGGL(CopyKernel, grid, dim3(256), 0, nullptr, static_cast<const v4i*>(src), static_cast<v4i*>(dst), n16);
        (void)hipEventRecord(ev.e1, nullptr);
        float ms = 0.0f;
        if (hipEventSynchronize(ev.e1) != hipSuccess || hipEventElapsedTime(&ms, ev.e0, ev.e1) != hipSuccess || ms <= 0.0f) rc = 2;
        else *bytes_per_s = 2.0 * static_cast<double>(bytes) * reps / (ms * 1e-3);
    }
    (void)hipFree(src);
    (void)hipFree(dst);
    return rc;
}
} // extern "C"
