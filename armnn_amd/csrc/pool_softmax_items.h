// Global pooling of one (image, 256-channel group) and Softmax of one row as device functions of a 256-thread block:
// the per-layer kernels are thin wrappers around them, and the classifier-tail kernel (pooling -> FullyConnected ->
// Softmax in one launch) calls the same functions, so both give the same bytes.
#pragma once

#include <hip/hip_runtime.h>

#include <cfloat>
#include <climits>

#include "common.h"
#include "device_math.h"

namespace mi355x
{

struct PoolArgs
{
    int H, W, C, Ho, Wo;
    int pool_w, pool_h, stride_x, stride_y;
    int pad_left, pad_right, pad_top, pad_bottom;
    int is_max, exclude;
};

constexpr int kGlobalPoolMaxTaps = 196;

// Item = image * groups + group, groups = ceil(C / 256); C must be a multiple of 4 and the tensors dword aligned (THROUGH:
// the output 16-byte aligned).
// All threads fetch the image's taps as dwords into LDS (`raw`, taps * 64 dwords) at once; then thread c walks channel
// c's taps in the reference's order (row by row), so the fp32 sum is the reference's sum (Pooling2d.cpp:186-300 with a
// window that is the whole image).  `taps` = H * W, at most kGlobalPoolMaxTaps.  THROUGH: the byte is written through L2
// as it is stored, for a caller that hands it to other blocks of the same launch.
// The function ends with reads of `raw`: a barrier must separate it from the next use of that memory.
template <bool THROUGH>
__device__ __forceinline__ void GlobalPoolItem(const PoolArgs& p, const QIn& qin, const Requant& rq, const uint8_t* __restrict__ x,
                                               uint8_t* __restrict__ y, int item, uint32_t* raw)
{
    const int taps = p.H * p.W;
    const int groups = (p.C + 255) >> 8;
    const long long n = item / groups;
    const int c0 = (item % groups) * 256;
    const int quads = min(64, (p.C - c0) >> 2);
    const uint8_t* xn = x + n * taps * p.C + c0;
    for (int i = threadIdx.x; i < taps * 64; i += 256)
    {
        const int tap = i >> 6, q = i & 63;
        if (q < quads) raw[i] = *reinterpret_cast<const uint32_t*>(xn + static_cast<long long>(tap) * p.C + q * 4);
    }
    __syncthreads();
    const int c = threadIdx.x;
    if constexpr (!THROUGH)
    {
        if (c0 + c >= p.C) return;
    }
    const bool inside = c0 + c < p.C;
    const uint8_t* col = reinterpret_cast<const uint8_t*>(raw) + (inside ? c : 0);
    float res;
    if (p.is_max)
    {
        int best = INT_MIN;
        for (int t = 0; t < taps; ++t)
        {
            const int code = qin.is_u8 ? static_cast<int>(col[t * 256]) : static_cast<int>(static_cast<int8_t>(col[t * 256]));
            best = max(best, code);
        }
        res = __fmul_rn(static_cast<float>(best - qin.offset), qin.scale);
    }
    else
    {
        float sum = 0.0f;
#pragma unroll 7
        for (int t = 0; t < taps; ++t)
        {
            const int code = qin.is_u8 ? static_cast<int>(col[t * 256]) : static_cast<int>(static_cast<int8_t>(col[t * 256]));
            sum = __fadd_rn(sum, __fmul_rn(static_cast<float>(code - qin.offset), qin.scale));
        }
        res = __fdiv_rn(sum, static_cast<float>(taps));
    }
    const uint8_t out = static_cast<uint8_t>(QuantizeFastDev(res, rq));
    if constexpr (THROUGH)
    {
        // Single bytes written through one by one are slow: the group's bytes meet in LDS (behind the taps, which every
        // thread has finished reading at the barrier) and leave as dwords, one per four channels.
        __syncthreads();
        reinterpret_cast<uint8_t*>(raw)[c] = out;
        __syncthreads();
        // the image's 256-channel group as the buffer: uniform base, offsets below 256
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(y + n * p.C + c0, 0, min(256, p.C - c0), 0x00020000);
        if (c < 16)
        {
            typedef unsigned int U4 __attribute__((ext_vector_type(4)));
            const U4 v = *reinterpret_cast<const U4*>(raw + c * 4);
            if (c * 16 + 16 <= p.C - c0) __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, c * 16, 0, kStoreAuxSc1);
            else
            {
#pragma unroll
                for (int d = 0; d < 4; ++d) __builtin_amdgcn_raw_buffer_store_b32(v[d], rsrc, c * 16 + d * 4, 0, kStoreAuxSc1);   // past the end: dropped
            }
        }
    }
    else y[n * p.C + c0 + c] = out;
}

// Softmax of one row of `cols` <= 256 * V codes, held in registers: one pass over memory, one exp per element
// (Softmax.cpp:16-69: maximum, exp((v - max) * beta), sum, division).  `red`: 8 floats of LDS; a barrier must separate
// two calls.
template <int V>
__device__ __forceinline__ void SoftmaxRowItem(int cols, float beta, const QIn& qin, const Requant& rq, const uint8_t* __restrict__ xr,
                                               uint8_t* __restrict__ yr, float* red)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint8_t raw[V];
#pragma unroll
    for (int k = 0; k < V; ++k) raw[k] = xr[min(tid + 256 * k, cols - 1)];
    float v[V];
    float mx = -FLT_MAX;
#pragma unroll
    for (int k = 0; k < V; ++k)
    {
        v[k] = DequantDev(raw[k], qin);
        if (tid + 256 * k < cols) mx = fmaxf(mx, v[k]);
    }
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float sum = 0.0f;
#pragma unroll
    for (int k = 0; k < V; ++k)
    {
        v[k] = tid + 256 * k < cols ? expf(__fmul_rn(__fsub_rn(v[k], mx), beta)) : 0.0f;
        sum += v[k];
    }
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    if (lane == 0) red[4 + wave] = sum;
    __syncthreads();
    sum = (red[4] + red[5]) + (red[6] + red[7]);
#pragma unroll
    for (int k = 0; k < V; ++k)
        if (tid + 256 * k < cols) yr[tid + 256 * k] = static_cast<uint8_t>(QuantizeDev(__fdiv_rn(v[k], sum), rq));
}

} // namespace mi355x
