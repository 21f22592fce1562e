// Depthwise 3x3 + pointwise 1x1 as ONE kernel: the depthwise layer's output tile never leaves the CU.
//
//   phase A  for every block of 32 channels: stage the input halo tile in LDS (double buffered, next block's loads in
//            flight while this one is computed), run the v_dot4 depthwise arithmetic of Depthwise3x3Kernel, requantize
//            with the depthwise layer's own constants (+ its fused activation) and write the resulting int8 codes --
//            exactly the bytes the separate layer would have stored -- to the LDS tile T[pixel][channel].
//   phase B  T is the "activation" operand of the pointwise GEMM: out[pixel][co] = sum_c T[pixel][c] * W[co][c] on
//            v_mfma_i32_32x32x32_i8.  A wave owns pairs of 32-channel sub-tiles; it reads its weight fragments straight
//            from global memory (lane = output channel row, 16 contiguous K bytes; every weight byte is read once per
//            block) and the pixel fragments from T, requantizes with the pointwise layer's constants and writes 64
//            contiguous channel bytes per pixel.
//
// The two layers' arithmetic is untouched, so the result is byte-identical to running them one after the other; what
// disappears is the intermediate tensor's round trip through HBM, one kernel launch and the second kernel's load phase.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"
#include "dw_stem_kernels.h"

namespace mi355x
{

struct DwPwArgs
{
    // depthwise stage
    const uint8_t*  x;
    const uint8_t*  pad16;      // 16 bytes that become the depthwise padding value under dw_xor
    const uint32_t* dw_grp;     // [C/4][8][4] dwords per group of 4 channels: w row 0, w row 1, w row 2, corr, m+, b+, m-, b-
    ChanTab         dw_ct;      // exact-path constants of the depthwise layer
    int N, H, W, C, Ho, Wo;
    int pad_top, pad_left;
    int tiles_x, tiles_y;
    int total_blocks, xcd_chunk;
    uint32_t dw_xor;            // 0x80808080 for uint8 input
    Requant dw_rq;
    // pointwise stage
    const int8_t*  pw_w;        // [Co_pad][pw_wstride]
    int            pw_wstride;
    ChanTab        pw_ct;       // rows 2, 5, 6 on the fast path (accumulators start at zero)
    const int32_t* pw_corr;
    uint8_t*       y;
    int            Co;
    uint32_t       mid_xor;     // 0x80808080 when the intermediate tensor is uint8: T holds the signed-shifted codes
    Requant        pw_rq;
};

// S: depthwise stride (1 or 2).  P: output pixels per thread along x, so a tile is 8 rows x 4P pixels (stride 1: P = 4
// or 2; stride 2: P = 2).  The narrow stride-1 tile gives small images enough blocks to fill the device.
template <int S, int P>
struct DwPwGeom
{
    static_assert((S == 1 && (P == 4 || P == 2)) || (S == 2 && P == 2), "supported tile shapes");
    static constexpr int CB = 32, TH = 8, XG = 4;
    static constexpr int TW = P * XG;
    static constexpr int TP = TH * TW;                 // pixels per tile: 128, 64 (stride 1) or 64 (stride 2)
    static constexpr int HR = TH * S + 2;
    static constexpr int HC = TW * S + 2;
    static constexpr int PITCH = 48;
    static constexpr int HALO = HR * HC * PITCH;
    static constexpr int NST = (HR * HC * 2 + 255) / 256;   // 16-byte staging chunks per thread and channel block
    static constexpr int OST = 4 * 32 * (64 + 16);          // output staging, aliases the halo buffers
    static constexpr int SCRATCH = 2 * HALO > OST ? 2 * HALO : OST;
    static constexpr int G = S == 1 ? P / 2 : P;            // dot-product groups per thread and kernel row
    static constexpr int NPX = 2 * (G + 1);                 // halo pixels a thread reads per kernel row
};

template <int S, int P>
inline int DwPwSmemBytes(int C)
{
    using G = DwPwGeom<S, P>;
    return G::TP * (C + 16) + G::SCRATCH + (C / 4) * 128;
}

// D: channel blocks whose halo loads are in flight (register slots); KC: k-steps per weight chunk of phase B, the next
// chunk being loaded while the current one is multiplied.
template <int S, int P, int D>
__global__ __launch_bounds__(256) void DwPwKernel(DwPwArgs a)
{
    using G = DwPwGeom<S, P>;
    constexpr int TW = G::TW, TH = G::TH, HC = G::HC, PITCH = G::PITCH, NST = G::NST;
    constexpr int TPS = G::TP / 32;                    // 32-pixel sub-tiles
    constexpr int NC = 2;                              // 32-channel sub-tiles a wave accumulates together
    constexpr int KC = 4;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int LDT = a.C + 16;
    uint8_t* T = smem;
    uint8_t* scratch = smem + G::TP * LDT;
    uint32_t* grp = reinterpret_cast<uint32_t*>(scratch + G::SCRATCH);

    int b = XcdContiguousWorkItem(blockIdx.x, a.xcd_chunk);
    if ((static_cast<int>(blockIdx.x) >> 3) >= a.xcd_chunk || b >= a.total_blocks) return;
    const int tx = b % a.tiles_x; b /= a.tiles_x;
    const int ty = b % a.tiles_y;
    const int n = b / a.tiles_y;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;

    // ---- depthwise constants of all channels -> LDS ----------------------------------------------------------------
    for (int i = tid; i < a.C * 2; i += 256)           // C/4 groups x 8 rows of 16 bytes
        *reinterpret_cast<v4i*>(grp + i * 4) = *reinterpret_cast<const v4i*>(a.dw_grp + i * 4);

    // ---- phase A ----------------------------------------------------------------------------------------------------
    const int iy_org = ty * TH * S - a.pad_top;
    const int ix_org = tx * TW * S - a.pad_left;
    const uint8_t* xn = a.x + static_cast<long long>(n) * a.H * a.W * a.C;
    const int xm = static_cast<int>(a.dw_xor);
    // this thread's staging chunks: halo pixel + 16-byte half, fixed over the channel blocks
    int st_off[NST];            // byte offset of the chunk inside the image (channel block 0), -1: outside, -2: none
#pragma unroll
    for (int k = 0; k < NST; ++k)
    {
        const int i = tid + k * 256;
        st_off[k] = -2;
        if (i < G::HR * HC * 2)
        {
            const int half = i & 1, pix = i >> 1;
            const int col = pix % HC, row = pix / HC;
            const int iy = iy_org + row, ix = ix_org + col;
            const bool ok = static_cast<unsigned>(iy) < static_cast<unsigned>(a.H) && static_cast<unsigned>(ix) < static_cast<unsigned>(a.W);
            st_off[k] = ok ? (iy * a.W + ix) * a.C + half * 16 : -1;
        }
    }
    v4i st[D][NST];
    auto stage_load = [&](int cb, auto slot) {
        constexpr int SL = decltype(slot)::value;
#pragma unroll
        for (int k = 0; k < NST; ++k)
        {
            // outside the image (or no chunk): 16 prepared padding bytes, so that every load is unconditional
            const uint8_t* src = st_off[k] >= 0 ? xn + st_off[k] + cb * 32 : a.pad16;
            st[SL][k] = *reinterpret_cast<const v4i*>(src);
        }
    };
    auto stage_store = [&](int buf, auto slot) {
        constexpr int SL = decltype(slot)::value;
        uint8_t* halo = scratch + buf * G::HALO;
#pragma unroll
        for (int k = 0; k < NST; ++k)
        {
            const int i = tid + k * 256;
            if (i < G::HR * HC * 2) *reinterpret_cast<v4i*>(halo + (i >> 1) * PITCH + (i & 1) * 16) = st[SL][k] ^ xm;
        }
    };

    const int c4 = tid & 7;
    const int xg = (tid >> 3) & 3;
    const int row = tid >> 5;
    const int ncb = a.C >> 5;
    const uint32_t mid = a.mid_xor;
    using std::integral_constant;
    stage_load(0, integral_constant<int, 0>{});
    if constexpr (D > 1) { if (1 < ncb) stage_load(1, integral_constant<int, 1>{}); }
    if constexpr (D > 2) { if (2 < ncb) stage_load(2, integral_constant<int, 2>{}); }
    if constexpr (D > 3) { if (3 < ncb) stage_load(3, integral_constant<int, 3>{}); }
    // channel block cb (cb % D == J): its halo goes from slot J to LDS, slot J is refilled with block cb + D
    auto dw_block = [&](int cb, auto jc) {
        stage_store(cb & 1, jc);
        __syncthreads();        // also orders the constants' LDS writes before their first use
        if (cb + D < ncb) stage_load(cb + D, jc);

        const uint8_t* halo = scratch + (cb & 1) * G::HALO;
        const v4i* gc = reinterpret_cast<const v4i*>(grp + (cb * 8 + c4) * 32);   // this thread's group of 4 channels
        const v4i w0 = gc[0], w1 = gc[1], w2 = gc[2], corr4 = gc[3];
        int acc[P][4];
#pragma unroll
        for (int j = 0; j < P; ++j)
#pragma unroll
            for (int ch = 0; ch < 4; ++ch) acc[j][ch] = corr4[ch];
#pragma unroll
        for (int r = 0; r < 3; ++r)
        {
            const v4i wr = r == 0 ? w0 : r == 1 ? w1 : w2;
            const uint8_t* base = halo + ((row * S + r) * HC + xg * P * S) * PITCH + c4 * 4;
            uint32_t px[G::NPX];
#pragma unroll
            for (int j = 0; j < G::NPX; ++j) px[j] = *reinterpret_cast<const uint32_t*>(base + j * PITCH);
            uint32_t lo[G::G + 1], hi[G::G + 1];
#pragma unroll
            for (int q = 0; q < G::G + 1; ++q)
            {
                lo[q] = __builtin_amdgcn_perm(px[2 * q + 1], px[2 * q], 0x05010400u);
                hi[q] = __builtin_amdgcn_perm(px[2 * q + 1], px[2 * q], 0x07030602u);
            }
#pragma unroll
            for (int g = 0; g < G::G; ++g)
            {
                uint32_t chv[4];
                chv[0] = __builtin_amdgcn_perm(lo[g + 1], lo[g], 0x05040100u);
                chv[1] = __builtin_amdgcn_perm(lo[g + 1], lo[g], 0x07060302u);
                chv[2] = __builtin_amdgcn_perm(hi[g + 1], hi[g], 0x05040100u);
                chv[3] = __builtin_amdgcn_perm(hi[g + 1], hi[g], 0x07060302u);
#pragma unroll
                for (int ch = 0; ch < 4; ++ch)
                {
                    if (S == 1)
                    {
                        acc[2 * g][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), wr[ch], acc[2 * g][ch], false);
                        acc[2 * g + 1][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), static_cast<int>(static_cast<uint32_t>(wr[ch]) << 8), acc[2 * g + 1][ch], false);
                    }
                    else
                    {
                        acc[g][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), wr[ch], acc[g][ch], false);
                    }
                }
            }
        }
        const float4 mp = *reinterpret_cast<const float4*>(gc + 4);
        const float4 bp = *reinterpret_cast<const float4*>(gc + 5);
        const float4 mm = *reinterpret_cast<const float4*>(gc + 6);
        const float4 bm = *reinterpret_cast<const float4*>(gc + 7);
        const int c = cb * 32 + c4 * 4;
#pragma unroll
        for (int j = 0; j < P; ++j)
        {
            const uint32_t q = Requant4Dev(acc[j][0], acc[j][1], acc[j][2], acc[j][3], mp, bp, mm, bm, a.dw_ct, nullptr, c, a.dw_rq);
            *reinterpret_cast<uint32_t*>(T + (row * TW + xg * P + j) * LDT + c) = q ^ mid;
        }
    };
    for (int cb = 0; cb < ncb; cb += D)
    {
        dw_block(cb, integral_constant<int, 0>{});
        if constexpr (D > 1) { if (cb + 1 < ncb) dw_block(cb + 1, integral_constant<int, 1>{}); }
        if constexpr (D > 2) { if (cb + 2 < ncb) dw_block(cb + 2, integral_constant<int, 2>{}); }
        if constexpr (D > 3) { if (cb + 3 < ncb) dw_block(cb + 3, integral_constant<int, 3>{}); }
    }
    __syncthreads();            // T complete; the halo buffers are free and become the output staging area

    // ---- phase B ----------------------------------------------------------------------------------------------------
    constexpr int LDO = 64 + 16;
    uint8_t* ostage = scratch + wave * 32 * LDO;
    const int frag_row = lane & 31;
    const int frag_k = (lane >> 5) * 16;
    const int lane_c = 4 * (lane >> 5);
    const int ksteps = a.C >> 5;
    const int nct = a.Co >> 5;
    for (int ct = wave * NC; ct < nct; ct += 4 * NC)
    {
        v16i acc[NC][TPS];
        const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        const int8_t* wbase = a.pw_w + static_cast<long long>(ct * 32 + frag_row) * a.pw_wstride + frag_k;
        const uint8_t* tbase = T + frag_row * LDT + frag_k;
        // weights in chunks of KC k-steps, two register slots: chunk q + 1 is on its way while chunk q is multiplied
        const int nchunk = (ksteps + KC - 1) / KC;
        v4i wv[2][KC][NC];
        auto load_w = [&](int q, auto slot) {
            constexpr int SL = decltype(slot)::value;
#pragma unroll
            for (int kk = 0; kk < KC; ++kk)
            {
                const int k = min(q * KC + kk, ksteps - 1);     // a short last chunk re-reads the last step (not used)
#pragma unroll
                for (int i = 0; i < NC; ++i)
                    wv[SL][kk][i] = *reinterpret_cast<const v4i*>(wbase + static_cast<long long>(i) * 32 * a.pw_wstride + k * 32);
            }
        };
        auto mul_w = [&](int q, auto slot) {
            constexpr int SL = decltype(slot)::value;
#pragma unroll
            for (int kk = 0; kk < KC; ++kk)
            {
                const int k = q * KC + kk;
                if (k < ksteps)
                {
#pragma unroll
                    for (int p = 0; p < TPS; ++p)
                    {
                        const v4i av = *reinterpret_cast<const v4i*>(tbase + p * 32 * LDT + k * 32);
#pragma unroll
                        for (int i = 0; i < NC; ++i)
                            acc[i][p] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wv[SL][kk][i], av, acc[i][p], 0, 0, 0);
                    }
                }
            }
        };
#pragma unroll
        for (int i = 0; i < NC; ++i)
#pragma unroll
            for (int p = 0; p < TPS; ++p) acc[i][p] = zero;
        load_w(0, integral_constant<int, 0>{});
        for (int q = 0; q < nchunk; q += 2)
        {
            if (q + 1 < nchunk) load_w(q + 1, integral_constant<int, 1>{});
            mul_w(q, integral_constant<int, 0>{});
            if (q + 1 < nchunk)
            {
                if (q + 2 < nchunk) load_w(q + 2, integral_constant<int, 0>{});
                mul_w(q + 1, integral_constant<int, 1>{});
            }
        }
        // epilogue: one 32-pixel sub-tile at a time through the wave's staging rows
#pragma unroll
        for (int p = 0; p < TPS; ++p)
        {
#pragma unroll
            for (int i = 0; i < NC; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                {
                    const int cl = i * 32 + 8 * q + lane_c;
                    const int cg = ct * 32 + cl;
                    const float4 mp = *reinterpret_cast<const float4*>(a.pw_ct.p + 2 * a.pw_ct.stride + cg);
                    const float4 bp = *reinterpret_cast<const float4*>(a.pw_ct.p + 6 * a.pw_ct.stride + cg);
                    const float4 mm = *reinterpret_cast<const float4*>(a.pw_ct.p + 4 * a.pw_ct.stride + cg);
                    const float4 bm = *reinterpret_cast<const float4*>(a.pw_ct.p + 7 * a.pw_ct.stride + cg);
                    const v16i& v = acc[i][p];
                    const uint32_t out = Requant4Dev(v[4 * q + 0], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3], mp, bp, mm, bm, a.pw_ct, a.pw_corr, cg, a.pw_rq);
                    *reinterpret_cast<uint32_t*>(ostage + frag_row * LDO + cl) = out;
                }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            // 32 pixels x 64 bytes: 4 chunks of 16 bytes per pixel, 2 per lane
#pragma unroll
            for (int j = lane; j < 32 * 4; j += 64)
            {
                const int r = j >> 2, cc = j & 3;
                const int pix = p * 32 + r;
                const int oy = ty * TH + pix / TW, ox = tx * TW + pix % TW;
                if (oy < a.Ho && ox < a.Wo)
                    *reinterpret_cast<v4i*>(a.y + ((static_cast<long long>(n) * a.Ho + oy) * a.Wo + ox) * a.Co + ct * 32 + cc * 16) =
                        *reinterpret_cast<const v4i*>(ostage + r * LDO + cc * 16);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    }
}

} // namespace mi355x
