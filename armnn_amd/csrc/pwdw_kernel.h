// Pointwise 1x1 convolution + the depthwise 3x3 that follows it as ONE kernel, for feature maps small enough that a block
// can hold whole images: the 1x1 layer's output tile never leaves the CU.
//
//   * A block owns G whole images (G * H * W <= 32 * MF pixel rows) and BN = 64 of the channels.  A depthwise layer
//     mixes nothing across channels, so those 64 channels of the intermediate tensor are all the block needs: there is
//     no halo to recompute and no channel is computed twice.
//   phase A  the 1x1 GEMM out[pixel][c] = sum_k x[pixel][k] * W[c][k] on v_mfma_i32_32x32x32_i8, k-tiles of 128 bytes
//            travelling global -> LDS directly (global_load_lds_dwordx4, the xor-swizzled dense layout of
//            IgemmLdsKernel), ST stages.  Wave w owns 32-channel column (w & 1) and the 32-pixel fragments
//            (w >> 1), (w >> 1) + 2, ... of the MF.
//   phase B  requantize with the 1x1 layer's constants (+ its fused activation) and write the int8 codes -- exactly the
//            bytes the separate layer would have stored -- into the LDS tile T[image][halo row][halo column][channel],
//            whose border cells hold the depthwise layer's padding value.
//   phase C  the v_dot4 depthwise arithmetic of Depthwise3x3Kernel over T (a thread: 4 channels x 2 neighbouring output
//            pixels per step), requantize with the depthwise layer's constants, store.
//
// Both layers' arithmetic is untouched, so the result is byte-identical to running them one after the other; what
// disappears is a kernel launch with its ramp and drain, and the intermediate tensor's round trip.
#pragma once

#include <hip/hip_runtime.h>

#include <climits>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"
#include "dw_stem_kernels.h"
#include "igemm_lds_kernel.h"

namespace mi355x
{

struct PwDwArgs
{
    // pointwise stage
    const uint8_t* x;           // [N][H][W][Ci]
    const int8_t*  w;           // [C_pad][K_pad]
    int            K_pad;       // multiple of 128, >= Ci
    ChanTab        pw_ct;
    const int32_t* pw_corr;
    uint32_t       pw_xor;      // 0x80808080 for uint8 input
    Requant        pw_rq;
    int N, H, W, Ci, C;         // C: channels of the intermediate tensor (multiple of 64)
    int G;                      // images per block
    int tiles_n;                // C / 64
    int total_blocks, xcd_chunk;
    // depthwise stage
    const uint32_t* dw_grp;     // [C/4][8][4] dwords per group of 4 channels: w row 0, w row 1, w row 2, corr, m+, b+, m-, b-
    ChanTab         dw_ct;
    Requant         dw_rq;
    uint32_t        dw_xor;     // 0x80808080 when the intermediate tensor is uint8: T holds the signed-shifted codes
    uint32_t        dw_pad;     // the depthwise padding value, already shifted, replicated in 4 bytes
    int Ho, Wo, pad_top, pad_left;
    int HR, HC;                 // halo tile: (Ho - 1) * S + 3 rows, 2 * S * pairs + 2 columns
    int pairs;                  // (Wo + 1) / 2 output pixel pairs per row
    uint8_t*        y;          // [N][Ho][Wo][C]; with global pooling as the second stage [N][C]
    // global pooling as the second stage (POOL) in place of the depthwise layer
    QIn             pool_in;    // the intermediate tensor's quantization as the pooling reads it
    Requant         pool_rq;
    int             pool_is_max;
};

constexpr int kPwDwBN = 64;
constexpr int kPwDwPitch = kPwDwBN + 16;

template <int MF, int ST>
constexpr int PwDwStageBytes()
{
    return ST * (MF * 32 + kPwDwBN) * 128;
}

// s_waitcnt vmcnt(n) for a wave-uniform run-time n: the instruction takes an immediate, so the even counts a k-tile
// pipeline produces are enumerated and anything else waits for the next smaller one (stricter, never wrong).
__device__ __forceinline__ void WaitVmcntAtMost(int n)
{
    if (n >= 40) __builtin_amdgcn_s_waitcnt(VmcntImm(40));
    else if (n >= 36) __builtin_amdgcn_s_waitcnt(VmcntImm(36));
    else if (n >= 32) __builtin_amdgcn_s_waitcnt(VmcntImm(32));
    else if (n >= 30) __builtin_amdgcn_s_waitcnt(VmcntImm(30));
    else if (n >= 28) __builtin_amdgcn_s_waitcnt(VmcntImm(28));
    else if (n >= 24) __builtin_amdgcn_s_waitcnt(VmcntImm(24));
    else if (n >= 20) __builtin_amdgcn_s_waitcnt(VmcntImm(20));
    else if (n >= 18) __builtin_amdgcn_s_waitcnt(VmcntImm(18));
    else if (n >= 16) __builtin_amdgcn_s_waitcnt(VmcntImm(16));
    else if (n >= 12) __builtin_amdgcn_s_waitcnt(VmcntImm(12));
    else if (n >= 10) __builtin_amdgcn_s_waitcnt(VmcntImm(10));
    else if (n >= 8) __builtin_amdgcn_s_waitcnt(VmcntImm(8));
    else if (n >= 6) __builtin_amdgcn_s_waitcnt(VmcntImm(6));
    else if (n >= 4) __builtin_amdgcn_s_waitcnt(VmcntImm(4));
    else __builtin_amdgcn_s_waitcnt(VmcntImm(0));
}

// MF: 32-pixel fragments per block; ST: LDS stages of the GEMM; S: depthwise stride (1 or 2); NW: waves (4 or 8).
// POOL: the second stage is a pooling whose window is the whole image instead of the depthwise layer: T holds the
// images' pixels back to back without a border, and thread (image, channel) walks its column in the order of
// GlobalPoolItem, so the pooled bytes are those of the two layers run one after the other (Pooling2d.cpp:186-300).
template <int MF, int ST, int S, int NW, bool POOL = false>
__global__ __launch_bounds__(64 * NW) void PwDwKernel(PwDwArgs a)
{
    constexpr int BK = 128, BN = kPwDwBN, BM = MF * 32, PITCH = kPwDwPitch;
    constexpr int UA = BM / 16;                  // 16-row units of the activation tile, dealt to the waves round robin
    constexpr int RAU = (UA + NW - 1) / NW;      // ... units per wave at most
    constexpr int RB = 8 / NW;                   // 8-row groups of the weight tile per wave
    constexpr int FSTEP = NW / 2;                // a wave's fragments are FSTEP apart
    static_assert(NW == 4 || NW == 8, "4 or 8 waves");
    constexpr int STAGE = (BM + BN) * BK;
    constexpr int TP = (MF + FSTEP - 1) / FSTEP; // fragments per wave at most
    typedef __attribute__((address_space(3))) void* LdsPtr;
    typedef const __attribute__((address_space(1))) void* GlobalPtr;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int tile = XcdContiguousWorkItem(blockIdx.x, a.xcd_chunk);
    if ((static_cast<int>(blockIdx.x) >> 3) >= a.xcd_chunk || tile >= a.total_blocks) return;
    const int tn = tile % a.tiles_n;
    const int grp = tile / a.tiles_n;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int HW = a.H * a.W;
    const int n0 = grp * a.G;
    const int images = min(a.G, a.N - n0);
    const int rows = images * HW;                // valid pixel rows of this block

    // ---- phase A ----------------------------------------------------------------------------------------------------
    const int lrow = lane >> 3;
    const int lchunk[2] = {(lane & 7) ^ (lrow >> 1), (lane & 7) ^ ((lrow >> 1) + 4)};
    const uint8_t* xbase = a.x + static_cast<long long>(n0) * HW * a.Ci;
    const uint8_t* xrow[RAU][2];
#pragma unroll
    for (int u = 0; u < RAU; ++u)
#pragma unroll
        for (int h = 0; h < 2; ++h)
        {
            const int r = (u * NW + wave) * 16 + h * 8 + lrow;
            // rows past the block's images re-read its first row; their products are never stored
            xrow[u][h] = xbase + static_cast<long long>(r < rows ? r : 0) * a.Ci + lchunk[h] * 16;
        }
    const int8_t* wrow[RB];
#pragma unroll
    for (int j = 0; j < RB; ++j)
    {
        const int hu = wave * RB + j;            // 8-row group of the weight tile
        wrow[j] = a.w + static_cast<long long>(tn * BN + hu * 8 + lrow) * a.K_pad + lchunk[hu & 1] * 16;
    }
    const int my_units = wave < UA ? (UA - wave + NW - 1) / NW : 0;     // wave-uniform

    auto load_tile = [&](int kt, int stage) {
        uint8_t* As = smem + stage * STAGE;
        uint8_t* Bs = As + BM * BK;
#pragma unroll
        for (int u = 0; u < RAU; ++u)
            if (u < my_units)
            {
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    __builtin_amdgcn_global_load_lds((GlobalPtr)(xrow[u][h] + kt * BK), (LdsPtr)(As + ((u * NW + wave) * 16 + h * 8) * BK), 16, 0, 0);
            }
#pragma unroll
        for (int j = 0; j < RB; ++j)
            __builtin_amdgcn_global_load_lds((GlobalPtr)(wrow[j] + kt * BK), (LdsPtr)(Bs + (wave * RB + j) * 8 * BK), 16, 0, 0);
    };

    const int tc = wave & 1;                     // this wave's 32-channel column
    const int f0 = wave >> 1;                    // ... and its fragments f0, f0 + FSTEP, ...
    const int lane_c = 4 * (lane >> 5);
    const int cbase = tn * BN + tc * 32;
    v16i acc[TP];
    {
        v16i init;
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const v4i c4 = *reinterpret_cast<const v4i*>(a.pw_corr + cbase + 8 * q + lane_c);
            init[4 * q + 0] = c4[0]; init[4 * q + 1] = c4[1]; init[4 * q + 2] = c4[2]; init[4 * q + 3] = c4[3];
        }
#pragma unroll
        for (int tp = 0; tp < TP; ++tp) acc[tp] = init;
    }
    const int frag_row = lane & 31, frag_half = lane >> 5;
    const int xm = static_cast<int>(a.pw_xor);
    auto compute = [&](int stage) {
        const uint8_t* As = smem + stage * STAGE;
        const uint8_t* Bs = As + BM * BK;
#pragma unroll
        for (int ks = 0; ks < BK / 32; ++ks)
        {
            const int slot = ((ks * 2 + frag_half) ^ ((frag_row >> 1) & 7)) * 16;
            const v4i fw = *reinterpret_cast<const v4i*>(Bs + (tc * 32 + frag_row) * BK + slot);
#pragma unroll
            for (int tp = 0; tp < TP; ++tp)
            {
                const int f = f0 + FSTEP * tp;
                if (f < MF)
                {
                    v4i fa = *reinterpret_cast<const v4i*>(As + (f * 32 + frag_row) * BK + slot);
                    fa ^= xm;
                    acc[tp] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw, fa, acc[tp], 0, 0, 0);
                }
            }
        }
    };

    // ---- depthwise constants of this thread's 4 channels, requested before the GEMM's tiles ---------------------------
    const int c4 = tid & 15;
    v4i w0 = {}, w1 = {}, w2 = {}, corr4 = {};
    float4 dmp = {}, dbp = {}, dmm = {}, dbm = {};
    if constexpr (!POOL)
    {
        const v4i* gc = reinterpret_cast<const v4i*>(a.dw_grp + (tn * (BN / 4) + c4) * 32);
        w0 = gc[0]; w1 = gc[1]; w2 = gc[2]; corr4 = gc[3];
        dmp = *reinterpret_cast<const float4*>(gc + 4);
        dbp = *reinterpret_cast<const float4*>(gc + 5);
        dmm = *reinterpret_cast<const float4*>(gc + 6);
        dbm = *reinterpret_cast<const float4*>(gc + 7);
    }

    const int nk = a.K_pad / BK;
#pragma unroll
    for (int s = 0; s < ST - 1; ++s)
        if (s < nk) load_tile(s, s);

    int stage = 0;
    for (int kt = 0; kt < nk; ++kt)
    {
        // Tile kt has landed when at most the requests of the younger tiles (up to ST - 2 of them, 2 per 16-row unit of
        // this wave) are outstanding; any other load the wave has issued since only makes the wait stricter.
        WaitVmcntAtMost(min(ST - 2, nk - 1 - kt) * (2 * my_units + RB));
        __syncthreads();
        if (kt + ST - 1 < nk)
        {
            int ls = stage + ST - 1;
            if (ls >= ST) ls -= ST;
            load_tile(kt + ST - 1, ls);
        }
        compute(stage);
        if (++stage == ST) stage = 0;
    }
    __syncthreads();

    // ---- phase B: T <- padding value, then the requantized 1x1 outputs ---------------------------------------------------
    uint8_t* T = smem;
    if constexpr (!POOL)
    {
        const int cells = a.G * a.HR * a.HC;
        const v4i padv = {static_cast<int>(a.dw_pad), static_cast<int>(a.dw_pad), static_cast<int>(a.dw_pad), static_cast<int>(a.dw_pad)};
        for (int i = tid; i < cells * (PITCH / 16); i += 64 * NW) *reinterpret_cast<v4i*>(T + i * 16) = padv;
        __syncthreads();
    }
#pragma unroll
    for (int tp = 0; tp < TP; ++tp)
    {
        const int f = f0 + FSTEP * tp;
        const int ml = f * 32 + frag_row;
        if (f < MF && ml < rows)
        {
            bool inside = true;
            uint8_t* cell = T + ml * PITCH + tc * 32 + lane_c;         // POOL: pixel rows as they come
            if constexpr (!POOL)
            {
                const int g = ml / HW, p = ml - g * HW;
                const int iy = p / a.W, ix = p - iy * a.W;
                const int hy = iy + a.pad_top, hx = ix + a.pad_left;
                inside = hy < a.HR && hx < a.HC;
                cell = T + ((g * a.HR + hy) * a.HC + hx) * PITCH + tc * 32 + lane_c;
            }
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const int cg = cbase + 8 * q + lane_c;
                const Fast4 f4 = LoadFast4(a.pw_ct, cg);
                const v16i& v = acc[tp];
                const uint32_t out = Requant4Dev(v[4 * q + 0], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3], f4, a.pw_ct, cg, a.pw_rq);
                if (inside) *reinterpret_cast<uint32_t*>(cell + 8 * q) = POOL ? out : out ^ a.dw_xor;
            }
        }
    }
    __syncthreads();

    // ---- phase C, pooling: thread (image, channel) walks its column of T ------------------------------------------------
    if constexpr (POOL)
    {
        for (int it = tid; it < images * BN; it += 64 * NW)
        {
            const int g = it / BN, c = it - g * BN;
            const uint8_t* col = T + g * HW * PITCH + c;
            float res;
            if (a.pool_is_max)
            {
                int best = INT_MIN;
                for (int t = 0; t < HW; ++t)
                {
                    const int code = a.pool_in.is_u8 ? static_cast<int>(col[t * PITCH]) : static_cast<int>(static_cast<int8_t>(col[t * PITCH]));
                    best = max(best, code);
                }
                res = __fmul_rn(static_cast<float>(best - a.pool_in.offset), a.pool_in.scale);
            }
            else
            {
                float sum = 0.0f;
#pragma unroll 7
                for (int t = 0; t < HW; ++t)
                {
                    const int code = a.pool_in.is_u8 ? static_cast<int>(col[t * PITCH]) : static_cast<int>(static_cast<int8_t>(col[t * PITCH]));
                    sum = __fadd_rn(sum, __fmul_rn(static_cast<float>(code - a.pool_in.offset), a.pool_in.scale));
                }
                res = __fdiv_rn(sum, static_cast<float>(HW));
            }
            a.y[static_cast<long long>(n0 + g) * a.C + tn * BN + c] = static_cast<uint8_t>(QuantizeFastDev(res, a.pool_rq));
        }
        return;
    }

    // ---- phase C: depthwise 3x3 over T ---------------------------------------------------------------------------------
    constexpr int NPX = S == 1 ? 4 : 6;
    const int per_image = a.Ho * a.pairs;
    const int items = images * per_image;
    const int cglob = tn * BN + c4 * 4;
    for (int it = tid >> 4; it < items; it += 4 * NW)
    {
        const int g = it / per_image, r = it - g * per_image;
        const int oy = r / a.pairs, xg = r - oy * a.pairs;
        int o[2][4];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int ch = 0; ch < 4; ++ch) o[j][ch] = corr4[ch];
#pragma unroll
        for (int kr = 0; kr < 3; ++kr)
        {
            const v4i wr = kr == 0 ? w0 : kr == 1 ? w1 : w2;
            const uint8_t* base = T + ((g * a.HR + oy * S + kr) * a.HC + xg * 2 * S) * PITCH + c4 * 4;
            uint32_t px[NPX];
#pragma unroll
            for (int j = 0; j < NPX; ++j) px[j] = *reinterpret_cast<const uint32_t*>(base + j * PITCH);
            uint32_t lo[NPX / 2], hi[NPX / 2];
#pragma unroll
            for (int q = 0; q < NPX / 2; ++q)
            {
                lo[q] = __builtin_amdgcn_perm(px[2 * q + 1], px[2 * q], 0x05010400u);
                hi[q] = __builtin_amdgcn_perm(px[2 * q + 1], px[2 * q], 0x07030602u);
            }
#pragma unroll
            for (int gq = 0; gq < NPX / 2 - 1; ++gq)
            {
                uint32_t chv[4];
                chv[0] = __builtin_amdgcn_perm(lo[gq + 1], lo[gq], 0x05040100u);
                chv[1] = __builtin_amdgcn_perm(lo[gq + 1], lo[gq], 0x07060302u);
                chv[2] = __builtin_amdgcn_perm(hi[gq + 1], hi[gq], 0x05040100u);
                chv[3] = __builtin_amdgcn_perm(hi[gq + 1], hi[gq], 0x07060302u);
#pragma unroll
                for (int ch = 0; ch < 4; ++ch)
                {
                    if (S == 1)
                    {
                        // pixels x .. x + 3 of one channel: output x takes weights (w0, w1, w2, 0), output x + 1 the same
                        // weights one byte up
                        o[0][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), wr[ch], o[0][ch], false);
                        o[1][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), static_cast<int>(static_cast<uint32_t>(wr[ch]) << 8), o[1][ch], false);
                    }
                    else
                    {
                        o[gq][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), wr[ch], o[gq][ch], false);
                    }
                }
            }
        }
        uint8_t* yrow = a.y + ((static_cast<long long>(n0 + g) * a.Ho + oy) * a.Wo) * a.C + cglob;
#pragma unroll
        for (int j = 0; j < 2; ++j)
        {
            const uint32_t q = Requant4Dev(o[j][0], o[j][1], o[j][2], o[j][3], dmp, dbp, dmm, dbm, a.dw_ct, nullptr, cglob, a.dw_rq);
            const int ox = xg * 2 + j;
            if (ox < a.Wo) *reinterpret_cast<uint32_t*>(yrow + static_cast<long long>(ox) * a.C) = q;
        }
    }
}

} // namespace mi355x
