// Convolution2d with a small filter and stride 1 whose input tile stays in LDS for all taps.
//
// The implicit GEMM re-reads every input pixel once per tap (nine times for 3x3) through the CU's vector L1, and for
// 64..256 channels that path -- not MFMA, not HBM -- sets its speed.  Here a block takes R whole output rows of one
// image and
//   * brings the (R + Kh - 1) x (Wo + Kw - 1) input pixels those rows need into LDS once (global_load_lds_dwordx4, out-of-
//     image positions from 16 prepared padding bytes), dense, pixel after pixel, Ci bytes each;
//   * walks K = taps x Ci in 128-byte k-tiles: the weights of a tile travel global -> LDS as in IgemmLdsKernel (ST
//     stages), the activation fragment of tap (ky, kx) is read straight from the resident tile at the tap's pixel offset;
//   * requantizes and writes the R x Wo x BN output bytes, which are contiguous rows of the output tensor.
// A 16-byte chunk c of pixel p lives at slot c ^ swz(p), swz(p) = (p >> SH) & (Ci / 16 - 1) with SH = 2, 1, 0 for
// Ci = 64, 128, 256: an MFMA fragment read takes the same chunk of consecutive pixels, and 16 consecutive pixels then
// cover sixteen different 4-bank groups whatever pixel they start at (a tap only shifts the start).
// Rows of the output tile are 32-pixel fragments of the flattened (row, column) index, so any Wo up to 32 * MF / R fits.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"
#include "igemm_lds_kernel.h"

namespace mi355x
{

struct HaloArgs
{
    const uint8_t* x;
    const uint8_t* pad16;   // 16 bytes of (padding value ^ input xor)
    const int8_t*  w;       // [Co_pad][K_pad], K = (ky, kx, ci), zero padded to whole 128-byte k-tiles
    ChanTab        ct;
    const int32_t* corr;    // [Co_pad]
    uint8_t*       y;
    int H, W, Ho, Wo, Co;
    int Kh, Kw;
    int pad_top, pad_left;
    int K_pad;
    int R;                  // output rows per tile
    int tiles_y;            // tiles per image
    int tiles_m, tiles_n;   // tiles_m = batch * tiles_y
    int WP;                 // Wo + Kw - 1: pixels per row of the resident tile
    int HP;                 // (R + Kh - 1) * WP: its pixels
    uint32_t wo_magic, wp_magic;   // ceil(2^32 / Wo), ceil(2^32 / WP): exact quotients for dividends below 2^16
    uint32_t xor_mask;
    Requant rq;
};

template <int CI>
constexpr int HaloTileBytes(int hp)
{
    return (hp * CI + 1023) / 1024 * 1024;       // whole 1 KB load instructions
}

// resident tile, weight stages, the block's slice of the channel table; the output byte tile is staged over the first two
// once the k-loop is done
template <int CI, int BN, int MF, int ST>
constexpr int HaloSmemBytes(int hp)
{
    constexpr int stages = ST * BN * 128;
    constexpr int out = MF * 32 * (BN + 16);
    const int work = HaloTileBytes<CI>(hp) + stages;
    return (work > out ? work : out) + 4 * BN * 4;
}

// WM x WN = 4 waves; a wave owns TP 32-pixel fragments and 32 output channels: block tile (32 * WM * TP) pixels x
// (32 * WN) channels.
template <int CI, int WM, int WN, int TP, int ST, bool U8>
__global__ __launch_bounds__(256) void HaloConvKernel(HaloArgs a)
{
    static_assert(WM * WN == 4, "four waves");
    static_assert(CI == 64 || CI == 128 || CI == 256, "64, 128 or 256 input channels");
    constexpr int BN = 32 * WN;
    constexpr int NCH = CI / 16;                               // 16-byte chunks per pixel
    constexpr int SH = CI == 64 ? 2 : CI == 128 ? 1 : 0;
    constexpr int RB = BN / 32;                                // weight load instructions per wave and k-tile (8 rows each)
    constexpr int WSTAGE = BN * 128;
    constexpr int LDO = BN + 16;
    typedef __attribute__((address_space(3))) void* LdsPtr;
    typedef const __attribute__((address_space(1))) void* GlobalPtr;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int MF = WM * TP;
    uint8_t* halo = smem;
    uint8_t* wst = smem + HaloTileBytes<CI>(a.HP);
    const int work = HaloTileBytes<CI>(a.HP) + ST * WSTAGE;
    float* tab_lds = reinterpret_cast<float*>(smem + (work > MF * 32 * LDO ? work : MF * 32 * LDO));   // rows 2..5 of the channel table, BN channels

    const int nblocks = a.tiles_m * a.tiles_n;
    const int per_xcd = (nblocks + 7) >> 3;
    const int tile = static_cast<int>(blockIdx.x & 7) * per_xcd + static_cast<int>(blockIdx.x >> 3);
    if (tile >= nblocks) return;
    const int tn = tile % a.tiles_n;
    const int tm = tile / a.tiles_n;
    const int n = tm / a.tiles_y;
    const int y0 = (tm - n * a.tiles_y) * a.R;
    const int rows = min(a.R, a.Ho - y0);
    const int mt = rows * a.Wo;                                // output pixels of this tile

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    // ---- the resident tile: instruction i of the block moves chunks 64 i .. 64 i + 63 --------------------------------
    {
        const int nchunks = a.HP * NCH;
        const int iy_org = y0 - a.pad_top, ix_org = -a.pad_left;
        const uint8_t* xn = a.x + static_cast<long long>(n) * a.H * a.W * CI;
        for (int i = wave; i * 64 < nchunks; i += 4)
        {
            const int e = i * 64 + lane;
            const int p = e / NCH, slot = e % NCH;
            const int chunk = slot ^ ((p >> SH) & (NCH - 1));
            const int hy = static_cast<int>(__umulhi(static_cast<uint32_t>(p), a.wp_magic));
            const int hx = p - hy * a.WP;
            const int iy = iy_org + hy, ix = ix_org + hx;
            const bool ok = (e < nchunks) & (static_cast<unsigned>(iy) < static_cast<unsigned>(a.H)) & (static_cast<unsigned>(ix) < static_cast<unsigned>(a.W));
            const uint8_t* src = ok ? xn + (static_cast<long long>(iy) * a.W + ix) * CI + chunk * 16 : a.pad16;
            __builtin_amdgcn_global_load_lds((GlobalPtr)(src), (LdsPtr)(halo + i * 1024), 16, 0, 0);
        }
    }

    // ---- the bracket rows of the channel table go to LDS: the epilogue then waits for no global load ---------------------
    v4i tab_piece = {0, 0, 0, 0};
    if (tid < BN) tab_piece = *reinterpret_cast<const v4i*>(a.ct.p + static_cast<long long>((tid / (BN / 4)) + 2) * a.ct.stride + tn * BN + (tid % (BN / 4)) * 4);

    // ---- weights: lane fetches row (lane >> 3) of each 8-row group, the chunk whose slot is (lane & 7) ---------------------
    const int lrow = lane >> 3;
    const int lchunk_even = (lane & 7) ^ (lrow >> 1);
    const int lchunk_odd = (lane & 7) ^ ((lrow >> 1) + 4);
    const int8_t* wrow = a.w + static_cast<long long>(tn * BN + wave * (BN / 4) + lrow) * a.K_pad;
    auto load_w = [&](int kt, int stage) {
        uint8_t* Bs = wst + stage * WSTAGE + wave * (BN / 4) * 128;
#pragma unroll
        for (int j = 0; j < RB; ++j)
        {
            const int8_t* src = wrow + static_cast<long long>(j * 8) * a.K_pad + kt * 128 + ((j & 1) ? lchunk_odd : lchunk_even) * 16;
            __builtin_amdgcn_global_load_lds((GlobalPtr)(src), (LdsPtr)(Bs + j * 8 * 128), 16, 0, 0);
        }
    };

    // ---- accumulators start at the zero-point correction -------------------------------------------------------------
    const int lane_c = 4 * (lane >> 5);
    const int cbase = tn * BN + wn * 32;
    v16i acc[TP];
    {
        v16i init;
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const v4i c4 = *reinterpret_cast<const v4i*>(a.corr + cbase + 8 * q + lane_c);
            init[4 * q + 0] = c4[0];
            init[4 * q + 1] = c4[1];
            init[4 * q + 2] = c4[2];
            init[4 * q + 3] = c4[3];
        }
#pragma unroll
        for (int tp = 0; tp < TP; ++tp) acc[tp] = init;
    }

    // ---- this lane's pixel of each fragment, as an index into the resident tile for tap (0, 0) ----------------------------
    const int frag_row = lane & 31;
    const int frag_half = lane >> 5;
    int pb[TP];
#pragma unroll
    for (int tp = 0; tp < TP; ++tp)
    {
        int t = (wm * TP + tp) * 32 + frag_row;
        t = t < mt ? t : 0;                                    // fragments past the tile compute on pixel 0 and store nothing
        const int oy = static_cast<int>(__umulhi(static_cast<uint32_t>(t), a.wo_magic));
        pb[tp] = oy * a.WP + (t - oy * a.Wo);
    }
    const int xm = static_cast<int>(a.xor_mask);
    const int ntaps = a.Kh * a.Kw;
    const int nk = a.K_pad / 128;

    auto compute = [&](int kt, int stage) {
        const uint8_t* Bs = wst + stage * WSTAGE;
        constexpr int SUB = CI >= 128 ? 4 : 2;                 // k-steps of 32 that share a tap
#pragma unroll
        for (int g = 0; g < 4 / SUB; ++g)
        {
            // tap of k-steps g * SUB .. g * SUB + SUB - 1 of this tile, and the first channel of the first of them
            const int kglob = kt * 128 + g * SUB * 32;
            int tap = kglob / CI;
            const int c0 = kglob - tap * CI;
            tap = min(tap, ntaps - 1);                         // beyond K (64 channels, odd tap count): zero weights
            const int ky = tap / a.Kw;
            const int shift = ky * a.WP + (tap - ky * a.Kw);
            int pc[TP], sw[TP];
#pragma unroll
            for (int tp = 0; tp < TP; ++tp)
            {
                const int p = pb[tp] + shift;
                pc[tp] = p * CI;
                sw[tp] = (p >> SH) & (NCH - 1);
            }
#pragma unroll
            for (int s = 0; s < SUB; ++s)
            {
                const int ks = g * SUB + s;
                const int chunk = (c0 >> 4) + 2 * s + frag_half;
                const v4i fw = *reinterpret_cast<const v4i*>(Bs + (wn * 32 + frag_row) * 128 + (((ks * 2 + frag_half) ^ ((frag_row >> 1) & 7)) * 16));
#pragma unroll
                for (int tp = 0; tp < TP; ++tp)
                {
                    v4i fa = *reinterpret_cast<const v4i*>(halo + pc[tp] + ((chunk ^ sw[tp]) << 4));
                    if (U8) fa ^= xm;
                    acc[tp] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw, fa, acc[tp], 0, 0, 0);
                }
            }
        }
    };

    // ---- pipeline: ST - 1 weight tiles requested ahead; the resident tile's loads are older than all of them -----------
#pragma unroll
    for (int s = 0; s < ST - 1; ++s)
        if (s < nk) load_w(s, s);
    if (tid < BN) *reinterpret_cast<v4i*>(tab_lds + tid * 4) = tab_piece;      // visible to all after the first barrier below
    int stage = 0;
    for (int kt = 0; kt < nk; ++kt)
    {
        const int younger = min(ST - 2, nk - 1 - kt);
        if (ST >= 4 && younger == 2) __builtin_amdgcn_s_waitcnt(VmcntImm(2 * RB));
        else if (ST >= 3 && younger == 1) __builtin_amdgcn_s_waitcnt(VmcntImm(RB));
        else __builtin_amdgcn_s_waitcnt(VmcntImm(0));
        __syncthreads();
        if (kt + ST - 1 < nk)
        {
            int ls = stage + ST - 1;
            if (ls >= ST) ls -= ST;
            load_w(kt + ST - 1, ls);
        }
        compute(kt, stage);
        if (++stage == ST) stage = 0;
    }
    __syncthreads();

    // ---- epilogue: requantize, stage the byte tile in LDS (over the resident tile and the weight stages), coalesced write-out --------------------
    uint8_t* Os = smem;
    {
        const int cl = wn * 32;
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const int cq = cl + 8 * q + lane_c;
            const float4 mp = *reinterpret_cast<const float4*>(tab_lds + 0 * BN + cq);
            const float4 bp = *reinterpret_cast<const float4*>(tab_lds + 1 * BN + cq);
            const float4 mm = *reinterpret_cast<const float4*>(tab_lds + 2 * BN + cq);
            const float4 bm = *reinterpret_cast<const float4*>(tab_lds + 3 * BN + cq);
#pragma unroll
            for (int tp = 0; tp < TP; ++tp)
            {
                const v16i& c = acc[tp];
                const uint32_t out = Requant4Dev(c[4 * q + 0], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3], mp, bp, mm, bm, a.ct, nullptr, tn * BN + cq, a.rq);
                const int pl = (wm * TP + tp) * 32 + (lane & 31);
                *reinterpret_cast<uint32_t*>(Os + pl * LDO + cl + 8 * q + lane_c) = out;
            }
        }
    }
    __syncthreads();
    constexpr int CHUNKS = BN / 16;
    constexpr int ROWS_PER_PASS = 256 / CHUNKS;
    const int oc = tid % CHUNKS;
    const int orow = tid / CHUNKS;
    const int c0 = tn * BN + oc * 16;
    uint8_t* yt = a.y + (static_cast<long long>(n) * a.Ho + y0) * a.Wo * a.Co;     // the tile's rows are contiguous in the output
    const OutPtr outp = MakeOutPtr(yt, static_cast<long long>(mt) * a.Co);
    if ((a.Co & 15) == 0)
    {
        if (c0 < a.Co)
        {
            for (int r = orow; r < mt; r += ROWS_PER_PASS)
                StoreOut16(outp, static_cast<long long>(r) * a.Co + c0, *reinterpret_cast<const v4i*>(Os + r * LDO + oc * 16));
        }
    }
    else
    {
        for (int r = orow; r < mt; r += ROWS_PER_PASS)
            for (int b = 0; b < 16; ++b)
            {
                const int c = c0 + b;
                if (c < a.Co) yt[static_cast<long long>(r) * a.Co + c] = Os[r * LDO + oc * 16 + b];
            }
    }
}

} // namespace mi355x
