// VALU kernels built on v_dot4_i32_i8 with LDS-staged halo tiles:
//
//   Depthwise3x3Kernel<S>   DepthwiseConvolution2d 3x3, multiplier 1, stride S in {1,2}, channels % 32 == 0.
//   SmallCiConvKernel<..>   Convolution2d with <= 4 input channels (network stems): too little K per tap for MFMA.
//
// Both bring the input to signed int8 while staging (uint8: x ^ 0x80) and fill out-of-image positions with the
// shifted zero point, so that   sum (x - zx) w  =  sum x' w  -  zx' * sum_taps w ;   the second term is a
// per-channel constant (`corr`) that initialises the accumulators.  Weights must be symmetric int8 (offset 0).
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"

namespace mi355x
{

struct Dw3x3Args
{
    const uint8_t*  x;
    const uint32_t* wpack;    // [C][4] dwords; dword r (r < 3) = bytes { w[r][0][c], w[r][1][c], w[r][2][c], 0 }
    ChanTab         ct;
    const int32_t*  corr;     // [C]  -zx' * sum of the 9 taps
    uint8_t*        y;
    int N, H, W, C, Ho, Wo;
    int pad_top, pad_left;
    int tiles_x, tiles_y, cblocks;
    uint32_t xor_mask, pad_word;
    Requant rq;
};

// Block: 8 output rows x (4 groups of P pixels) x 32 channels; thread = (4 channels, P pixels of one row).
// A thread reads 6 consecutive input pixels per kernel row (one dword = 4 channels each), transposes them with
// v_perm_b32 into per-channel dwords of 4 consecutive pixels, and each such dword feeds
//   stride 1: two outputs  (weights {w0,w1,w2,0} and {0,w0,w1,w2})
//   stride 2: one output   (weights {w0,w1,w2,0})
// through one v_dot4 per channel.
template <int S>
__global__ __launch_bounds__(256) void Depthwise3x3Kernel(Dw3x3Args a)
{
    constexpr int CB = 32, TH = 8, XG = 4;
    constexpr int P = S == 1 ? 4 : 2;            // outputs per thread
    constexpr int TW = P * XG;                   // outputs per tile row
    constexpr int HR = TH * S + 2;               // halo rows held in LDS
    constexpr int HC = TW * S + 2;               // halo columns
    constexpr int PITCH = 48;                    // bytes per pixel in LDS: 32 used; 48 spreads dword reads over banks
    __shared__ __attribute__((aligned(16))) uint8_t tile[HR * HC * PITCH];

    int b = blockIdx.x;
    const int cb = b % a.cblocks; b /= a.cblocks;
    const int tx = b % a.tiles_x; b /= a.tiles_x;
    const int ty = b % a.tiles_y;
    const int n = b / a.tiles_y;
    const int tid = threadIdx.x;

    // ---- stage the halo tile: 16-byte chunks, two per pixel ------------------------------------------------
    const int iy_org = ty * TH * S - a.pad_top;
    const int ix_org = tx * TW * S - a.pad_left;
    const uint8_t* xn = a.x + static_cast<long long>(n) * a.H * a.W * a.C + cb * CB;
    const v4i padv = {static_cast<int>(a.pad_word), static_cast<int>(a.pad_word), static_cast<int>(a.pad_word),
                      static_cast<int>(a.pad_word)};
    const int xm = static_cast<int>(a.xor_mask);
    for (int i = tid; i < HR * HC * 2; i += 256)
    {
        const int half = i & 1;
        const int pix = i >> 1;
        const int col = pix % HC;
        const int row = pix / HC;
        const int iy = iy_org + row, ix = ix_org + col;
        v4i v = padv;
        if (static_cast<unsigned>(iy) < static_cast<unsigned>(a.H) && static_cast<unsigned>(ix) < static_cast<unsigned>(a.W))
            v = *reinterpret_cast<const v4i*>(xn + (static_cast<long long>(iy) * a.W + ix) * a.C + half * 16) ^ xm;
        *reinterpret_cast<v4i*>(tile + pix * PITCH + half * 16) = v;
    }

    // ---- per-thread constants ---------------------------------------------------------------------------------
    const int c4 = tid & 7;
    const int xg = (tid >> 3) & 3;
    const int row = tid >> 5;
    const int c = cb * CB + c4 * 4;
    uint32_t wA[3][4];
#pragma unroll
    for (int ch = 0; ch < 4; ++ch)
    {
        const uint4 w4 = *reinterpret_cast<const uint4*>(a.wpack + (c + ch) * 4);
        wA[0][ch] = w4.x; wA[1][ch] = w4.y; wA[2][ch] = w4.z;
    }
    const v4i corr4 = *reinterpret_cast<const v4i*>(a.corr + c);
    int acc[P][4];
#pragma unroll
    for (int j = 0; j < P; ++j)
#pragma unroll
        for (int ch = 0; ch < 4; ++ch) acc[j][ch] = corr4[ch];

    __syncthreads();

#pragma unroll
    for (int r = 0; r < 3; ++r)
    {
        const uint8_t* base = tile + ((row * S + r) * HC + xg * P * S) * PITCH + c4 * 4;
        uint32_t px[6];
#pragma unroll
        for (int j = 0; j < 6; ++j) px[j] = *reinterpret_cast<const uint32_t*>(base + j * PITCH);
        // level 1: pixel pairs -> {p0.c0,p1.c0,p0.c1,p1.c1} and {p0.c2,p1.c2,p0.c3,p1.c3}
        uint32_t lo[3], hi[3];
#pragma unroll
        for (int q = 0; q < 3; ++q)
        {
            lo[q] = __builtin_amdgcn_perm(px[2 * q + 1], px[2 * q], 0x05010400u);
            hi[q] = __builtin_amdgcn_perm(px[2 * q + 1], px[2 * q], 0x07030602u);
        }
        // level 2: two pairs -> one dword per channel holding 4 consecutive pixels
#pragma unroll
        for (int g = 0; g < 2; ++g)
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
                    acc[2 * g][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), static_cast<int>(wA[r][ch]), acc[2 * g][ch], false);
                    acc[2 * g + 1][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), static_cast<int>(wA[r][ch] << 8), acc[2 * g + 1][ch], false);
                }
                else
                {
                    acc[g][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), static_cast<int>(wA[r][ch]), acc[g][ch], false);
                }
            }
        }
    }

    // ---- epilogue ------------------------------------------------------------------------------------------------
    const int oy = ty * TH + row;
    if (oy >= a.Ho) return;
    const Fast4 f4 = LoadFast4(a.ct, c);
    uint8_t* yrow = a.y + (static_cast<long long>(n) * a.Ho + oy) * a.Wo * a.C + c;
#pragma unroll
    for (int j = 0; j < P; ++j)
    {
        const int ox = tx * TW + xg * P + j;
        if (ox < a.Wo)
        {
            *reinterpret_cast<uint32_t*>(yrow + static_cast<long long>(ox) * a.C) =
                Requant4Dev(acc[j][0], acc[j][1], acc[j][2], acc[j][3], f4, a.ct, c, a.rq);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
struct SmallCiArgs
{
    const uint8_t*  x;
    const uint32_t* wpack;    // [Co][KH][RD] dwords: row r of filter co as consecutive (kx, ci) bytes, zero padded
    ChanTab         ct;
    const int32_t*  corr;     // [Co]
    uint8_t*        y;
    int N, H, W, Ci, Ho, Wo, Co;
    int Kw, stride, pad_top, pad_left;
    int tiles_x, tiles_y;
    uint32_t xor_mask, pad_byte;
    uint32_t ci_recip;        // ceil(65536 / Ci): (b * ci_recip) >> 16 == b / Ci for the small b used here
    Requant rq;
};

// Block: 16 x 16 output pixels; thread = one pixel, all output channels.  The input halo is staged byte by byte
// (rows start at arbitrary byte addresses when Ci is 3), each thread then reads its KH rows of Kw*Ci contiguous
// bytes as aligned dwords + v_alignbyte, and walks the output channels with wave-uniform (scalar-loaded) weights.
template <int KH, int RD>
__global__ __launch_bounds__(256) void SmallCiConvKernel(SmallCiArgs a)
{
    constexpr int TW = 16, TH = 16;
    constexpr int HRMAX = (TH - 1) * 2 + KH;
    constexpr int LP = (TW - 1) * 2 * 4 + RD * 4 + 8;       // LDS row pitch in bytes (multiple of 4)
    __shared__ __attribute__((aligned(16))) uint8_t tile[HRMAX * LP + 16];

    int b = blockIdx.x;
    const int tx = b % a.tiles_x; b /= a.tiles_x;
    const int ty = b % a.tiles_y;
    const int n = b / a.tiles_y;
    const int tid = threadIdx.x;
    const int S = a.stride;
    const int HR = (TH - 1) * S + KH;
    const int RB = ((TW - 1) * S + a.Kw) * a.Ci;            // bytes per halo row that carry data

    const int iy_org = ty * TH * S - a.pad_top;
    const int ix_org = tx * TW * S - a.pad_left;
    const uint8_t* xn = a.x + static_cast<long long>(n) * a.H * a.W * a.Ci;
    const uint8_t xm = static_cast<uint8_t>(a.xor_mask);
    for (int row = tid >> 6; row < HR; row += 4)
    {
        const int iy = iy_org + row;
        const bool row_ok = static_cast<unsigned>(iy) < static_cast<unsigned>(a.H);
        const uint8_t* xrow = xn + static_cast<long long>(iy) * a.W * a.Ci;
        for (int bcol = tid & 63; bcol < LP; bcol += 64)
        {
            uint8_t v = static_cast<uint8_t>(a.pad_byte);
            if (row_ok && bcol < RB)
            {
                const int pix = static_cast<int>((static_cast<uint32_t>(bcol) * a.ci_recip) >> 16);
                const int ix = ix_org + pix;
                if (static_cast<unsigned>(ix) < static_cast<unsigned>(a.W))
                    v = xrow[ix_org * a.Ci + bcol] ^ xm;
            }
            tile[row * LP + bcol] = v;
        }
    }
    __syncthreads();

    const int lx = tid & 15, ly = tid >> 4;
    uint32_t xr[KH][RD];
#pragma unroll
    for (int r = 0; r < KH; ++r)
    {
        const int off = (ly * S + r) * LP + lx * S * a.Ci;
        const uint32_t* p = reinterpret_cast<const uint32_t*>(tile + (off & ~3));
        const int sh = off & 3;
        uint32_t d[RD + 1];
#pragma unroll
        for (int i = 0; i <= RD; ++i) d[i] = p[i];
#pragma unroll
        for (int i = 0; i < RD; ++i) xr[r][i] = __builtin_amdgcn_alignbyte(d[i + 1], d[i], sh);
    }

    const int oy = ty * TH + ly, ox = tx * TW + lx;
    if (oy >= a.Ho || ox >= a.Wo) return;
    uint8_t* yp = a.y + ((static_cast<long long>(n) * a.Ho + oy) * a.Wo + ox) * a.Co;
    for (int co = 0; co < a.Co; co += 4)
    {
        int q[4];
        const Fast4 f4 = LoadFast4(a.ct, co);
#pragma unroll
        for (int u = 0; u < 4; ++u)
        {
            const uint32_t* w = a.wpack + static_cast<long long>(co + u) * KH * RD;
            int acc = a.corr[co + u];
#pragma unroll
            for (int r = 0; r < KH; ++r)
#pragma unroll
                for (int i = 0; i < RD; ++i)
                    acc = __builtin_amdgcn_sdot4(static_cast<int>(xr[r][i]), static_cast<int>(w[r * RD + i]), acc, false);
            q[u] = acc;
        }
        *reinterpret_cast<uint32_t*>(yp + co) = Requant4Dev(q[0], q[1], q[2], q[3], f4, a.ct, co, a.rq);
    }
}

} // namespace mi355x
