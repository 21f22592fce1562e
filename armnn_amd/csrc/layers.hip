// Bandwidth-bound layers that keep a network resident on the device between the convolutions:
// Activation, Pooling2d, ElementwiseBinary Add, Softmax.  All follow the reference's float formulation
// (dequantize -> float op -> armnn::Quantize) element for element.
#include "common.h"
#include "device_math.h"
#include "pool_softmax_items.h"

#include <algorithm>
#include <cfloat>
#include <climits>
#include <cmath>

using namespace mi355x;

typedef unsigned int v4u __attribute__((ext_vector_type(4)));

namespace
{

__device__ __forceinline__ float ActivationDev(float in, int fn, float a, float b)
{
    if (fn == MI355X_ACT_RELU) return fmaxf(0.0f, in);
    if (fn == MI355X_ACT_BOUNDED_RELU) return fminf(a, fmaxf(b, in));
    return in;
}


// A per-element function of one 8-bit code: build the 256-entry table once per block, then stream.
__global__ __launch_bounds__(256) void ActivationKernel(QIn qin, Requant rq, int fn, float a, float b,
                                                        const uint8_t* __restrict__ x, uint8_t* __restrict__ y, size_t n)
{
    __shared__ uint8_t lut[256];
    lut[threadIdx.x] = static_cast<uint8_t>(QuantizeDev(ActivationDev(DequantDev(static_cast<uint8_t>(threadIdx.x), qin), fn, a, b), rq));
    __syncthreads();
    size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (; i < n; i += stride) y[i] = lut[x[i]];
}

// One thread per output element; same window clamping and divisor rules as Pooling2d.cpp:186-300.
__global__ __launch_bounds__(256) void Pool2dKernel(PoolArgs p, QIn qin, Requant rq, const uint8_t* __restrict__ x,
                                                    uint8_t* __restrict__ y, long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    const int c = static_cast<int>(idx % p.C);
    long long pix = idx / p.C;
    const int ox = static_cast<int>(pix % p.Wo);
    pix /= p.Wo;
    const int oy = static_cast<int>(pix % p.Ho);
    const long long n = pix / p.Ho;

    int hstart = oy * p.stride_y - p.pad_top;
    int hend = min(hstart + p.pool_h, p.H + p.pad_bottom);
    const int height = hend - hstart;
    bool clamped = hstart < 0 || hend > p.H;
    hstart = min(max(hstart, 0), p.H);
    hend = min(max(hend, 0), p.H);
    int wstart = ox * p.stride_x - p.pad_left;
    int wend = min(wstart + p.pool_w, p.W + p.pad_right);
    float area = static_cast<float>(height * (wend - wstart));
    float result;
    if (hend <= 0 || hstart > p.H || wend <= 0 || wstart > p.W)
    {
        result = 0.0f;      // window covers padding only
    }
    else
    {
        clamped = clamped || wstart < 0 || wend > p.W;
        wstart = min(max(wstart, 0), p.W);
        wend = min(max(wend, 0), p.W);
        // The reference's clamp flag carries along a row, but with Exclude the divisor it selects equals
        // the unclamped one whenever this window itself is unclamped, so the per-window flag is equivalent.
        if (clamped && p.exclude) area = static_cast<float>((hend - hstart) * (wend - wstart));
        result = p.is_max ? -FLT_MAX : 0.0f;
        const uint8_t* xn = x + n * p.H * p.W * p.C + c;
        if (hend - hstart <= 8 && wend - wstart <= 8)
        {
            // up to 8 x 8 taps: all loads are issued before the first one is used (an element outside the window reads
            // the window's first element and is ignored), then accumulated in the reference's row-major order
            uint8_t raw[64];
            const long long first = (static_cast<long long>(hstart) * p.W + wstart) * p.C;
#pragma unroll
            for (int dy = 0; dy < 8; ++dy)
#pragma unroll
                for (int dx = 0; dx < 8; ++dx)
                {
                    const bool in = hstart + dy < hend && wstart + dx < wend;
                    raw[dy * 8 + dx] = xn[in ? (static_cast<long long>(hstart + dy) * p.W + wstart + dx) * p.C : first];
                }
#pragma unroll
            for (int dy = 0; dy < 8; ++dy)
#pragma unroll
                for (int dx = 0; dx < 8; ++dx)
                {
                    if (hstart + dy < hend && wstart + dx < wend)
                    {
                        const float v = DequantDev(raw[dy * 8 + dx], qin);
                        if (p.is_max) { if (v > result) result = v; }
                        else result = __fadd_rn(result, v);
                    }
                }
        }
        else
        {
            for (int iy = hstart; iy < hend; ++iy)
                for (int ix = wstart; ix < wend; ++ix)
                {
                    const float v = DequantDev(xn[(static_cast<long long>(iy) * p.W + ix) * p.C], qin);
                    if (p.is_max) { if (v > result) result = v; }
                    else result = __fadd_rn(result, v);
                }
        }
        if (!p.is_max) result = __fdiv_rn(result, area);
    }
    y[idx] = static_cast<uint8_t>(QuantizeFastDev(result, rq));
}

// Four channels per thread (one dword per tap), windows of at most WB x WB taps with all loads issued up front.
// Max pooling compares the raw codes: dequantization is strictly increasing, so the largest code is the largest value.
template <int WB>
__global__ __launch_bounds__(256) void Pool2dC4Kernel(PoolArgs p, QIn qin, Requant rq, const uint8_t* __restrict__ x,
                                                      uint8_t* __restrict__ y, long long total4)
{
    const long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total4) return;
    const int C4 = p.C >> 2;
    const int c = static_cast<int>(idx % C4) * 4;
    long long pix = idx / C4;
    const int ox = static_cast<int>(pix % p.Wo);
    pix /= p.Wo;
    const int oy = static_cast<int>(pix % p.Ho);
    const long long n = pix / p.Ho;

    int hstart = oy * p.stride_y - p.pad_top;
    int hend = min(hstart + p.pool_h, p.H + p.pad_bottom);
    const int height = hend - hstart;
    bool clamped = hstart < 0 || hend > p.H;
    hstart = min(max(hstart, 0), p.H);
    hend = min(max(hend, 0), p.H);
    int wstart = ox * p.stride_x - p.pad_left;
    int wend = min(wstart + p.pool_w, p.W + p.pad_right);
    float area = static_cast<float>(height * (wend - wstart));
    float res[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (!(hend <= 0 || hstart > p.H || wend <= 0 || wstart > p.W))
    {
        clamped = clamped || wstart < 0 || wend > p.W;
        wstart = min(max(wstart, 0), p.W);
        wend = min(max(wend, 0), p.W);
        if (clamped && p.exclude) area = static_cast<float>((hend - hstart) * (wend - wstart));
        const uint8_t* xn = x + n * p.H * p.W * p.C + c;
        uint32_t raw[WB * WB];
        const long long first = (static_cast<long long>(hstart) * p.W + wstart) * p.C;
#pragma unroll
        for (int dy = 0; dy < WB; ++dy)
#pragma unroll
            for (int dx = 0; dx < WB; ++dx)
            {
                const bool in = hstart + dy < hend && wstart + dx < wend;
                raw[dy * WB + dx] = *reinterpret_cast<const uint32_t*>(xn + (in ? (static_cast<long long>(hstart + dy) * p.W + wstart + dx) * p.C : first));
            }
        int best[4] = {INT_MIN, INT_MIN, INT_MIN, INT_MIN};
#pragma unroll
        for (int dy = 0; dy < WB; ++dy)
#pragma unroll
            for (int dx = 0; dx < WB; ++dx)
            {
                if (hstart + dy < hend && wstart + dx < wend)
                {
                    const uint32_t w = raw[dy * WB + dx];
#pragma unroll
                    for (int ch = 0; ch < 4; ++ch)
                    {
                        const int code = qin.is_u8 ? static_cast<int>((w >> (8 * ch)) & 0xffu)
                                                   : static_cast<int>(static_cast<int8_t>((w >> (8 * ch)) & 0xffu));
                        if (p.is_max) best[ch] = max(best[ch], code);
                        else res[ch] = __fadd_rn(res[ch], __fmul_rn(static_cast<float>(code - qin.offset), qin.scale));
                    }
                }
            }
#pragma unroll
        for (int ch = 0; ch < 4; ++ch)
        {
            if (p.is_max) res[ch] = best[ch] == INT_MIN ? -FLT_MAX : __fmul_rn(static_cast<float>(best[ch] - qin.offset), qin.scale);
            else res[ch] = __fdiv_rn(res[ch], area);
        }
    }
    *reinterpret_cast<uint32_t*>(y + idx * 4) = QuantizePack4Dev(res[0], res[1], res[2], res[3], rq);
}

// Max pooling over windows of at most WB x WB taps, sixteen channels per thread: 16-byte loads, and the maximum taken on
// pairs of bytes at a time (v_pk_max_u16 on the even and on the odd bytes of a dword; int8 codes are first mapped to
// unsigned order by flipping the sign bit).  The window arithmetic is spent once per sixteen outputs instead of once per
// four.  The largest code is the largest value (dequantization is strictly increasing); it is dequantized and requantized
// like every pooling result.
template <int WB>
__global__ __launch_bounds__(256) void MaxPool2dC16Kernel(PoolArgs p, QIn qin, Requant rq, const uint8_t* __restrict__ x,
                                                          uint8_t* __restrict__ y, long long total16)
{
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    const long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total16) return;
    const int C16 = p.C >> 4;
    const int c = static_cast<int>(idx % C16) * 16;
    long long pix = idx / C16;
    const int ox = static_cast<int>(pix % p.Wo);
    pix /= p.Wo;
    const int oy = static_cast<int>(pix % p.Ho);
    const long long n = pix / p.Ho;

    int hstart = oy * p.stride_y - p.pad_top;
    int hend = min(hstart + p.pool_h, p.H + p.pad_bottom);
    hstart = min(max(hstart, 0), p.H);
    hend = min(max(hend, 0), p.H);
    int wstart = ox * p.stride_x - p.pad_left;
    int wend = min(wstart + p.pool_w, p.W + p.pad_right);
    const bool empty = hend <= 0 || hstart > p.H || wend <= 0 || wstart > p.W;
    wstart = min(max(wstart, 0), p.W);
    wend = min(max(wend, 0), p.W);
    us2 blo[4], bhi[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) { blo[d] = us2{0, 0}; bhi[d] = us2{0, 0}; }
    bool any = false;
    if (!empty)
    {
        const uint8_t* xn = x + n * p.H * p.W * p.C + c;
        v4u raw[WB * WB];
        const long long first = (static_cast<long long>(min(hstart, p.H - 1)) * p.W + min(wstart, p.W - 1)) * p.C;
#pragma unroll
        for (int dy = 0; dy < WB; ++dy)
#pragma unroll
            for (int dx = 0; dx < WB; ++dx)
            {
                const bool in = hstart + dy < hend && wstart + dx < wend;
                raw[dy * WB + dx] = *reinterpret_cast<const v4u*>(xn + (in ? (static_cast<long long>(hstart + dy) * p.W + wstart + dx) * p.C : first));
            }
        const uint32_t flip = qin.is_u8 ? 0u : 0x80808080u;
#pragma unroll
        for (int dy = 0; dy < WB; ++dy)
#pragma unroll
            for (int dx = 0; dx < WB; ++dx)
            {
                if (hstart + dy < hend && wstart + dx < wend)
                {
                    any = true;
#pragma unroll
                    for (int d = 0; d < 4; ++d)
                    {
                        const uint32_t w = raw[dy * WB + dx][d] ^ flip;
                        const uint32_t lo = w & 0x00ff00ffu, hi = (w >> 8) & 0x00ff00ffu;
                        blo[d] = __builtin_elementwise_max(blo[d], __builtin_bit_cast(us2, lo));
                        bhi[d] = __builtin_elementwise_max(bhi[d], __builtin_bit_cast(us2, hi));
                    }
                }
            }
    }
    v4u out;
    const int unflip = qin.is_u8 ? 0 : 128;
#pragma unroll
    for (int d = 0; d < 4; ++d)
    {
        const int code[4] = {static_cast<int>(blo[d].x) - unflip, static_cast<int>(bhi[d].x) - unflip, static_cast<int>(blo[d].y) - unflip,
                             static_cast<int>(bhi[d].y) - unflip};
        float res[4];
#pragma unroll
        // a window wholly outside the padded extent gives 0.0 ("nothing to pool"), one that only covers padding the lowest value
        for (int ch = 0; ch < 4; ++ch)
            res[ch] = any ? __fmul_rn(static_cast<float>(code[ch] - qin.offset), qin.scale) : empty ? 0.0f : -FLT_MAX;
        out[d] = QuantizePack4Dev(res[0], res[1], res[2], res[3], rq);
    }
    *reinterpret_cast<v4u*>(y + idx * 16) = out;
}

// The window is the whole image (global pooling): a block owns 256 channels of one image (GlobalPoolItem).
__global__ __launch_bounds__(256) void GlobalPoolKernel(PoolArgs p, QIn qin, Requant rq, const uint8_t* __restrict__ x,
                                                        uint8_t* __restrict__ y)
{
    __shared__ uint32_t raw[kGlobalPoolMaxTaps * 64];
    GlobalPoolItem<false>(p, qin, rq, x, y, static_cast<int>(blockIdx.x), raw);
}

// The same pooling for images of at most MAXT pixels: a thread owns one channel of one image and asks for all of its taps
// before it uses the first, so the launch waits for memory once; the taps are then summed in GlobalPoolItem's order with
// GlobalPoolItem's arithmetic (same bytes).  Any channel count, no alignment rule.
template <int MAXT>
__global__ __launch_bounds__(64) void GlobalPoolSmallKernel(PoolArgs p, QIn qin, Requant rq, const uint8_t* __restrict__ x,
                                                            uint8_t* __restrict__ y, long long total)
{
    const long long i = static_cast<long long>(blockIdx.x) * 64 + threadIdx.x;
    if (i >= total) return;
    const int taps = p.H * p.W;
    const long long n = i / p.C;
    const int c = static_cast<int>(i - n * p.C);
    const uint8_t* src = x + n * taps * p.C + c;
    uint8_t v[MAXT];
#pragma unroll
    for (int t = 0; t < MAXT; ++t) v[t] = t < taps ? src[static_cast<long long>(t) * p.C] : 0;
    float res;
    if (p.is_max)
    {
        int best = INT_MIN;
#pragma unroll
        for (int t = 0; t < MAXT; ++t)
            if (t < taps) best = max(best, qin.is_u8 ? static_cast<int>(v[t]) : static_cast<int>(static_cast<int8_t>(v[t])));
        res = __fmul_rn(static_cast<float>(best - qin.offset), qin.scale);
    }
    else
    {
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < MAXT; ++t)
            if (t < taps)
            {
                const int code = qin.is_u8 ? static_cast<int>(v[t]) : static_cast<int>(static_cast<int8_t>(v[t]));
                sum = __fadd_rn(sum, __fmul_rn(static_cast<float>(code - qin.offset), qin.scale));
            }
        res = __fdiv_rn(sum, static_cast<float>(taps));
    }
    y[i] = static_cast<uint8_t>(QuantizeFastDev(res, rq));
}

// 16 elements per thread, 16-byte loads and stores
template <bool CLAMP>
__global__ __launch_bounds__(256) void AddVec16Kernel(AddFuse f, const v4u* __restrict__ x0,
                                                      const v4u* __restrict__ x1, v4u* __restrict__ y, size_t n16)
{
    const OutPtr outp = MakeOutPtr(reinterpret_cast<uint8_t*>(y), static_cast<long long>(n16) * 16);
    size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (; i < n16; i += stride)
    {
        const v4u a = x0[i], b = x1[i];
        v4u o;
#pragma unroll
        for (int d = 0; d < 4; ++d) o[d] = AddQuantize4Dev<CLAMP>(a[d], b[d], f);
        StoreOut16(outp, static_cast<long long>(i) * 16, StoreVec4{static_cast<int>(o[0]), static_cast<int>(o[1]), static_cast<int>(o[2]), static_cast<int>(o[3])});
    }
}

__global__ __launch_bounds__(256) void AddKernel(QIn q0, QIn q1, Requant rq, int fn, float a, float b,
                                                 const uint8_t* __restrict__ x0, const uint8_t* __restrict__ x1,
                                                 uint8_t* __restrict__ y, size_t n)
{
    size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (; i < n; i += stride)
    {
        const float s = __fadd_rn(DequantDev(x0[i], q0), DequantDev(x1[i], q1));
        int q = QuantizeFastDev(s, rq);   // rq carries the fused activation as an integer clamp
        y[i] = static_cast<uint8_t>(q);
    }
    (void)fn; (void)a; (void)b;
}

// One wave per row. exp((x - max) * beta) / sum, Softmax.cpp:41-64.
__global__ __launch_bounds__(64) void SoftmaxKernel(int cols, float beta, QIn qin, Requant rq,
                                                    const uint8_t* __restrict__ x, uint8_t* __restrict__ y)
{
    const uint8_t* xr = x + static_cast<long long>(blockIdx.x) * cols;
    uint8_t* yr = y + static_cast<long long>(blockIdx.x) * cols;
    const int lane = threadIdx.x;
    float mx = -FLT_MAX;
    for (int i = lane; i < cols; i += 64) mx = fmaxf(mx, DequantDev(xr[i], qin));
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    float sum = 0.0f;
    for (int i = lane; i < cols; i += 64) sum += expf(__fmul_rn(__fsub_rn(DequantDev(xr[i], qin), mx), beta));
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    for (int i = lane; i < cols; i += 64)
    {
        const float e = expf(__fmul_rn(__fsub_rn(DequantDev(xr[i], qin), mx), beta));
        yr[i] = static_cast<uint8_t>(QuantizeDev(__fdiv_rn(e, sum), rq));
    }
}

// One block per row, the row held in registers (cols <= 256 * V): SoftmaxRowItem.
template <int V>
__global__ __launch_bounds__(256) void SoftmaxRowKernel(int cols, float beta, QIn qin, Requant rq,
                                                         const uint8_t* __restrict__ x, uint8_t* __restrict__ y)
{
    __shared__ float red[8];
    SoftmaxRowItem<V>(cols, beta, qin, rq, x + static_cast<long long>(blockIdx.x) * cols, y + static_cast<long long>(blockIdx.x) * cols, red);
}

// Constant padding.  The host merges every unpadded dimension into the one outside it, so a row of the canonical
// innermost dimension is one contiguous run of output bytes whose middle part is one contiguous run of input bytes.
struct PadArgs
{
    uint32_t out[4], in[4], before[4];   // canonical shapes, right-aligned (leading extents 1)
    uint32_t fill;                       // the pad code in all four bytes
    int identity;                        // equal quantizations: elements are copied, not re-quantized
};

__device__ __forceinline__ uint32_t Recode4(uint32_t w, const uint8_t* lut)
{
    return static_cast<uint32_t>(lut[w & 0xffu]) | (static_cast<uint32_t>(lut[(w >> 8) & 0xffu]) << 8) |
           (static_cast<uint32_t>(lut[(w >> 16) & 0xffu]) << 16) | (static_cast<uint32_t>(lut[w >> 24]) << 24);
}

// One block per 256 units of V bytes of one output row; V divides the innermost extents and the front padding, so a
// unit lies either wholly inside the input or wholly in the padding.  grid.x = rows * chunks.
template <int V>
__global__ __launch_bounds__(256) void PadKernel(PadArgs p, QIn qin, Requant rq, uint32_t chunks,
                                                 const uint8_t* __restrict__ x, uint8_t* __restrict__ y)
{
    __shared__ uint8_t lut[256];
    if (!p.identity)
    {
        lut[threadIdx.x] = static_cast<uint8_t>(QuantizeDev(DequantDev(static_cast<uint8_t>(threadIdx.x), qin), rq));
        __syncthreads();
    }
    const uint32_t row = blockIdx.x / chunks;
    const uint32_t unit = (blockIdx.x - row * chunks) * 256 + threadIdx.x;
    if (unit >= p.out[3] / V) return;
    const uint32_t d2 = row % p.out[2];
    const uint32_t r1 = row / p.out[2];
    const uint32_t d1 = r1 % p.out[1];
    const uint32_t d0 = r1 / p.out[1];
    // unsigned wrap-around turns "in front of the input" into "beyond it"
    const uint32_t s0 = d0 - p.before[0], s1 = d1 - p.before[1], s2 = d2 - p.before[2], s3 = unit * V - p.before[3];
    const bool inside = s0 < p.in[0] && s1 < p.in[1] && s2 < p.in[2] && s3 < p.in[3];
    const size_t src = ((static_cast<size_t>(s0) * p.in[1] + s1) * p.in[2] + s2) * p.in[3] + s3;
    const size_t dst = static_cast<size_t>(row) * p.out[3] + static_cast<size_t>(unit) * V;
    if constexpr (V == 1)
    {
        uint8_t v = static_cast<uint8_t>(p.fill);
        if (inside) v = p.identity ? x[src] : lut[x[src]];
        y[dst] = v;
    }
    else if constexpr (V == 4)
    {
        uint32_t w = p.fill;
        if (inside)
        {
            w = *reinterpret_cast<const uint32_t*>(x + src);
            if (!p.identity) w = Recode4(w, lut);
        }
        *reinterpret_cast<uint32_t*>(y + dst) = w;
    }
    else
    {
        v4u w = {p.fill, p.fill, p.fill, p.fill};
        if (inside)
        {
            w = *reinterpret_cast<const v4u*>(x + src);
            if (!p.identity) { w.x = Recode4(w.x, lut); w.y = Recode4(w.y, lut); w.z = Recode4(w.z, lut); w.w = Recode4(w.w, lut); }
        }
        *reinterpret_cast<v4u*>(y + dst) = w;
    }
}

int CheckQ(const mi355x_quant* q, const char* what)
{
    if (!q) return SetError(MI355X_ERR_INVALID_ARGUMENT, "%s quantization is null", what);
    if (!IsActivationDtype(q->dtype)) return SetError(MI355X_ERR_UNSUPPORTED, "%s: data type %d is not QAsymmS8/QAsymmU8", what, q->dtype);
    if (!(q->scale > 0.0f) || !std::isfinite(q->scale)) return SetError(MI355X_ERR_INVALID_ARGUMENT, "%s: scale must be positive and finite", what);
    return 0;
}

unsigned GridFor(size_t n)
{
    size_t b = (n + 255) / 256;
    return static_cast<unsigned>(b > 16384 ? 16384 : b);
}

} // namespace

extern "C" {

int mi355x_activation_run(size_t n, const mi355x_quant* in_q, const mi355x_quant* out_q, int32_t activation, float a,
                          float b, const void* input_dev, void* output_dev, mi355x_stream_t stream)
{
    if (int rc = CheckQ(in_q, "input")) return rc;
    if (int rc = CheckQ(out_q, "output")) return rc;
    if (activation < MI355X_ACT_NONE || activation > MI355X_ACT_BOUNDED_RELU) return SetError(MI355X_ERR_UNSUPPORTED, "activation %d", activation);
    if (n == 0) return 0;
    if (!input_dev || !output_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "null tensor pointer");
    Requant rq = MakeRequant(*out_q, MI355X_ACT_NONE, 0.0f, 0.0f);
    NoteKernel("ActivationKernel");
    hipLaunchKernelGGL(ActivationKernel, dim3(GridFor(n)), dim3(256), 0, ToHip(stream), MakeQIn(*in_q), rq, activation, a, b,
                       static_cast<const uint8_t*>(input_dev), static_cast<uint8_t*>(output_dev), n);
    MI355X_HIP(hipGetLastError());
    return 0;
}

int mi355x_pool2d_run(const mi355x_pool2d_desc* d, uint32_t batch, const void* input_dev, void* output_dev,
                      mi355x_stream_t stream)
{
    if (!d) return SetError(MI355X_ERR_INVALID_ARGUMENT, "descriptor is null");
    if (int rc = CheckQ(&d->input, "input")) return rc;
    if (int rc = CheckQ(&d->output, "output")) return rc;
    if (d->pool_type != 0 && d->pool_type != 1) return SetError(MI355X_ERR_UNSUPPORTED, "Unsupported pooling algorithm %d", d->pool_type);
    if (d->padding_method != 0 && d->padding_method != 1) return SetError(MI355X_ERR_UNSUPPORTED, "Unsupported padding type %d", d->padding_method);
    if (d->pool_w == 0 || d->pool_h == 0 || d->stride_x == 0 || d->stride_y == 0 || d->channels == 0)
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "zero pool size / stride / channels");
    if (batch == 0 || d->out_h == 0 || d->out_w == 0) return 0;
    if (!input_dev || !output_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "null tensor pointer");
    PoolArgs p;
    p.H = d->in_h; p.W = d->in_w; p.C = d->channels; p.Ho = d->out_h; p.Wo = d->out_w;
    p.pool_w = d->pool_w; p.pool_h = d->pool_h; p.stride_x = d->stride_x; p.stride_y = d->stride_y;
    p.pad_left = d->pad_left; p.pad_right = d->pad_right; p.pad_top = d->pad_top; p.pad_bottom = d->pad_bottom;
    p.is_max = d->pool_type == 0;
    p.exclude = d->padding_method == 1;
    Requant rq = MakeRequant(d->output, MI355X_ACT_NONE, 0.0f, 0.0f);
    const long long total = static_cast<long long>(batch) * p.Ho * p.Wo * p.C;
    const bool vec4 = (p.C % 4) == 0 && (reinterpret_cast<uintptr_t>(input_dev) & 3) == 0 && (reinterpret_cast<uintptr_t>(output_dev) & 3) == 0;
    const bool global = p.Ho == 1 && p.Wo == 1 && p.pad_top == 0 && p.pad_left == 0 && p.pool_h == p.H && p.pool_w == p.W &&
                        p.H * p.W <= kGlobalPoolMaxTaps;
    if (global && p.H * p.W <= 64 && GlobalOptions().pool_small != 0)
    {
        NoteKernel("GlobalPoolSmallKernel<64>");
        const long long n = static_cast<long long>(batch) * p.C;
        hipLaunchKernelGGL(GlobalPoolSmallKernel<64>, dim3(static_cast<unsigned>((n + 63) / 64)), dim3(64), 0, ToHip(stream), p, MakeQIn(d->input), rq,
                           static_cast<const uint8_t*>(input_dev), static_cast<uint8_t*>(output_dev), n);
    }
    else if (vec4 && global)
    {
        NoteKernel("GlobalPoolKernel");
        hipLaunchKernelGGL(GlobalPoolKernel, dim3(static_cast<unsigned>(batch * ((p.C + 255) / 256))), dim3(256), 0, ToHip(stream), p,
                           MakeQIn(d->input), rq, static_cast<const uint8_t*>(input_dev), static_cast<uint8_t*>(output_dev));
    }
    else if (p.is_max && (p.C % 16) == 0 && p.pool_w <= 3 && p.pool_h <= 3 && (reinterpret_cast<uintptr_t>(input_dev) & 15) == 0 &&
             (reinterpret_cast<uintptr_t>(output_dev) & 15) == 0)
    {
        NoteKernel("MaxPool2dC16Kernel<3>");
        hipLaunchKernelGGL(MaxPool2dC16Kernel<3>, dim3(static_cast<unsigned>((total / 16 + 255) / 256)), dim3(256), 0, ToHip(stream), p,
                           MakeQIn(d->input), rq, static_cast<const uint8_t*>(input_dev), static_cast<uint8_t*>(output_dev), total / 16);
    }
    else if (vec4 && p.pool_w <= 3 && p.pool_h <= 3)
    {
        NoteKernel("Pool2dC4Kernel<3>");
        hipLaunchKernelGGL(Pool2dC4Kernel<3>, dim3(static_cast<unsigned>((total / 4 + 255) / 256)), dim3(256), 0, ToHip(stream), p,
                           MakeQIn(d->input), rq, static_cast<const uint8_t*>(input_dev), static_cast<uint8_t*>(output_dev), total / 4);
    }
    else if (vec4 && p.pool_w <= 8 && p.pool_h <= 8)
    {
        NoteKernel("Pool2dC4Kernel<8>");
        hipLaunchKernelGGL(Pool2dC4Kernel<8>, dim3(static_cast<unsigned>((total / 4 + 255) / 256)), dim3(256), 0, ToHip(stream), p,
                           MakeQIn(d->input), rq, static_cast<const uint8_t*>(input_dev), static_cast<uint8_t*>(output_dev), total / 4);
    }
    else
    {
        NoteKernel("Pool2dKernel");
        hipLaunchKernelGGL(Pool2dKernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, ToHip(stream), p,
                           MakeQIn(d->input), rq, static_cast<const uint8_t*>(input_dev), static_cast<uint8_t*>(output_dev), total);
    }
    MI355X_HIP(hipGetLastError());
    return 0;
}

int mi355x_add_run(size_t n, const mi355x_quant* in0_q, const mi355x_quant* in1_q, const mi355x_quant* out_q,
                   int32_t activation, float a, float b, const void* input0_dev, const void* input1_dev,
                   void* output_dev, mi355x_stream_t stream)
{
    if (int rc = CheckQ(in0_q, "input0")) return rc;
    if (int rc = CheckQ(in1_q, "input1")) return rc;
    if (int rc = CheckQ(out_q, "output")) return rc;
    if (activation < MI355X_ACT_NONE || activation > MI355X_ACT_BOUNDED_RELU) return SetError(MI355X_ERR_UNSUPPORTED, "activation %d", activation);
    if (n == 0) return 0;
    if (!input0_dev || !input1_dev || !output_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "null tensor pointer");
    Requant rq = MakeRequant(*out_q, activation, a, b);
    const bool vec16 = (n % 16) == 0 && ((reinterpret_cast<uintptr_t>(input0_dev) | reinterpret_cast<uintptr_t>(input1_dev) |
                                           reinterpret_cast<uintptr_t>(output_dev)) & 15) == 0;
    if (vec16)
    {
        NoteKernel("AddVec16Kernel");
        const AddFuse f = MakeAddFuse(*in0_q, *in1_q, *out_q, activation, a, b);
        if (f.rq.pk_full)
            hipLaunchKernelGGL(AddVec16Kernel<false>, dim3(GridFor(n / 16)), dim3(256), 0, ToHip(stream), f,
                               static_cast<const v4u*>(input0_dev), static_cast<const v4u*>(input1_dev), static_cast<v4u*>(output_dev), n / 16);
        else
            hipLaunchKernelGGL(AddVec16Kernel<true>, dim3(GridFor(n / 16)), dim3(256), 0, ToHip(stream), f,
                               static_cast<const v4u*>(input0_dev), static_cast<const v4u*>(input1_dev), static_cast<v4u*>(output_dev), n / 16);
    }
    else
    {
        NoteKernel("AddKernel");
        hipLaunchKernelGGL(AddKernel, dim3(GridFor(n)), dim3(256), 0, ToHip(stream), MakeQIn(*in0_q), MakeQIn(*in1_q), rq,
                           activation, a, b, static_cast<const uint8_t*>(input0_dev), static_cast<const uint8_t*>(input1_dev),
                           static_cast<uint8_t*>(output_dev), n);
    }
    MI355X_HIP(hipGetLastError());
    return 0;
}

int mi355x_softmax_run(uint32_t rows, uint32_t cols, float beta, const mi355x_quant* in_q, const mi355x_quant* out_q,
                       const void* input_dev, void* output_dev, mi355x_stream_t stream)
{
    if (int rc = CheckQ(in_q, "input")) return rc;
    if (int rc = CheckQ(out_q, "output")) return rc;
    if (rows == 0 || cols == 0) return 0;
    if (!input_dev || !output_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "null tensor pointer");
    Requant rq = MakeRequant(*out_q, MI355X_ACT_NONE, 0.0f, 0.0f);
    const uint8_t* xin = static_cast<const uint8_t*>(input_dev);
    uint8_t* yout = static_cast<uint8_t*>(output_dev);
    if (cols <= 1024)
    {
        NoteKernel("SoftmaxRowKernel<4>");
        hipLaunchKernelGGL(SoftmaxRowKernel<4>, dim3(rows), dim3(256), 0, ToHip(stream), static_cast<int>(cols), beta, MakeQIn(*in_q), rq, xin, yout);
    }
    else if (cols <= 2048)
    {
        NoteKernel("SoftmaxRowKernel<8>");
        hipLaunchKernelGGL(SoftmaxRowKernel<8>, dim3(rows), dim3(256), 0, ToHip(stream), static_cast<int>(cols), beta, MakeQIn(*in_q), rq, xin, yout);
    }
    else
    {
        NoteKernel("SoftmaxKernel");
        hipLaunchKernelGGL(SoftmaxKernel, dim3(rows), dim3(64), 0, ToHip(stream), static_cast<int>(cols), beta, MakeQIn(*in_q), rq, xin, yout);
    }
    MI355X_HIP(hipGetLastError());
    return 0;
}

int mi355x_pad_run(const mi355x_pad_desc* d, const void* input_dev, void* output_dev, mi355x_stream_t stream)
{
    if (!d) return SetError(MI355X_ERR_INVALID_ARGUMENT, "descriptor is null");
    if (d->rank < 1 || d->rank > 4) return SetError(MI355X_ERR_UNSUPPORTED, "Pad of rank %u (1..4 run on the device)", d->rank);
    if (int rc = CheckQ(&d->input, "input")) return rc;
    if (int rc = CheckQ(&d->output, "output")) return rc;
    if (d->input.dtype != d->output.dtype) return SetError(MI355X_ERR_INVALID_ARGUMENT, "input and output data types differ");
    if (std::isnan(d->pad_value)) return SetError(MI355X_ERR_INVALID_ARGUMENT, "pad value is not a number");

    // merge every unpadded dimension into its outer neighbour
    unsigned long long out[4], in[4], before[4];
    int n = 0;
    for (uint32_t k = 0; k < d->rank; ++k)
    {
        const unsigned long long o = static_cast<unsigned long long>(d->in_shape[k]) + d->pad_before[k] + d->pad_after[k];
        const bool unpadded = d->pad_before[k] == 0 && d->pad_after[k] == 0;
        if (n > 0 && unpadded)
        {
            out[n - 1] *= o; in[n - 1] *= o; before[n - 1] *= o;
        }
        else
        {
            out[n] = o; in[n] = d->in_shape[k]; before[n] = d->pad_before[k];
            ++n;
        }
    }
    unsigned long long total = 1, in_total = 1, rows = 1;
    for (int k = 0; k < n; ++k) { total *= out[k]; in_total *= in[k]; }
    if (total == 0) return 0;
    if ((!input_dev && in_total != 0) || !output_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "null tensor pointer");
    PadArgs p;
    for (int k = 0; k < 4; ++k) { p.out[k] = 1; p.in[k] = 1; p.before[k] = 0; }
    for (int k = 0; k < n; ++k)
    {
        if (out[k] > 0xffffffffull) return SetError(MI355X_ERR_UNSUPPORTED, "Pad: a merged extent exceeds 32 bits");
        p.out[4 - n + k] = static_cast<uint32_t>(out[k]);
        p.in[4 - n + k] = static_cast<uint32_t>(in[k]);
        p.before[4 - n + k] = static_cast<uint32_t>(before[k]);
    }
    for (int k = 0; k < 3; ++k) rows *= p.out[k];

    // Quantize<T>(value, 1, 0): round half away from zero, then saturate (TypesUtils.cpp:29-45)
    const bool u8 = d->output.dtype == MI355X_QASYMM_U8;
    float code = std::round(d->pad_value);
    code = std::min(std::max(code, u8 ? 0.0f : -128.0f), u8 ? 255.0f : 127.0f);
    const uint32_t byte = static_cast<uint32_t>(static_cast<int>(code)) & 0xffu;
    p.fill = byte * 0x01010101u;
    p.identity = d->input.scale == d->output.scale && d->input.offset == d->output.offset;

    const uintptr_t align = reinterpret_cast<uintptr_t>(input_dev) | reinterpret_cast<uintptr_t>(output_dev);
    const uint32_t inner = p.out[3] | p.in[3] | p.before[3];
    const int v = ((inner | align) & 15) == 0 ? 16 : ((inner | align) & 3) == 0 ? 4 : 1;
    const unsigned long long chunks = (p.out[3] / v + 255) / 256;
    if (rows * chunks > 0x7fffffffull) return SetError(MI355X_ERR_UNSUPPORTED, "Pad: tensor too large for one launch");
    Requant rq = MakeRequant(d->output, MI355X_ACT_NONE, 0.0f, 0.0f);
    const dim3 grid(static_cast<unsigned>(rows * chunks));
    const uint8_t* xin = static_cast<const uint8_t*>(input_dev);
    uint8_t* yout = static_cast<uint8_t*>(output_dev);
    if (v == 16)
    {
        NoteKernel("PadKernel<16>");
        hipLaunchKernelGGL(PadKernel<16>, grid, dim3(256), 0, ToHip(stream), p, MakeQIn(d->input), rq, static_cast<uint32_t>(chunks), xin, yout);
    }
    else if (v == 4)
    {
        NoteKernel("PadKernel<4>");
        hipLaunchKernelGGL(PadKernel<4>, grid, dim3(256), 0, ToHip(stream), p, MakeQIn(d->input), rq, static_cast<uint32_t>(chunks), xin, yout);
    }
    else
    {
        NoteKernel("PadKernel<1>");
        hipLaunchKernelGGL(PadKernel<1>, grid, dim3(256), 0, ToHip(stream), p, MakeQIn(d->input), rq, static_cast<uint32_t>(chunks), xin, yout);
    }
    MI355X_HIP(hipGetLastError());
    return 0;
}

} // extern "C"
