// Implicit GEMM whose k-tiles travel from global memory straight into LDS (global_load_lds_dwordx4): no staging
// registers, no ds_write, and the loads of the next tiles stay in flight across the block barrier.
//
//   * For convolutions whose channel count is a multiple of 128: a k-tile is 128 bytes of ONE filter tap, so the walk over
//     (ky, kx, ci) is scalar and a lane's address is a fixed per-row pointer plus a scalar tap offset.
//   * A wave's load instruction moves 8 rows x 128 bytes; lane l delivers its 16 bytes to LDS slot l of that 1 KB, so
//     the LDS image of a tile is dense (row pitch 128 bytes = half of the 64 banks).  A ds_read_b128 serves 16 lanes
//     per cycle; an MFMA fragment read takes the same chunk of 16 consecutive rows there, which must therefore sit in
//     16 different 4-bank groups: chunk c of row r lives at slot c ^ ((r >> 1) & 7) (rows of equal parity share the
//     bank half and get 8 different slots).  Lanes pick the global chunk that belongs in their slot; readers apply
//     the same xor.
//   * uint8 activations become int8 by xor 0x80 on the fragment registers (template U8), weights are int8 already.
//   * ST stages of LDS (2 to 8); tile kt + ST - 1 is requested right after the barrier that retires tile kt - 1, so
//     ST - 1 tiles are on their way while one is multiplied: deep for the few-block problems whose k-loop would
//     otherwise run at one memory round trip per tile.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"

namespace mi355x
{

template <int BM, int BN, int ST>
constexpr int IgemmLdsSmemBytes()
{
    constexpr int stages = ST * (BM + BN) * 128;
    constexpr int out = BM * (BN + 16);
    return stages > out ? stages : out;
}

// s_waitcnt immediate that waits for all but the `n` youngest vector-memory operations and for nothing else
constexpr int VmcntImm(int n)
{
    return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8);
}

// WM x WN waves per block (4, 8 or 16), each with a (BM / WM) x (BN / WN) tile of the block tile.
// AW: the weights have a zero point; each pixel's activations are summed beside the products (see IgemmKernel).
// UNIT: the launch is a 1x1 stride-1 unpadded convolution or a FullyConnected layer (a.unit) whose tensors are below
// 2 GiB: output row m reads input row m, there is no padding and no tap walk, and every load address is a wave-uniform
// base (advanced by 128 bytes per k-tile) plus a 32-bit lane offset fixed for the kernel -- no vector arithmetic per load.
// The work of one block on output tile `tile` (row-block major: tile = tm * tiles_n + tn); `smem` is the block's
// IgemmLdsSmemBytes<BM, BN, ST>() bytes of LDS.  Ends with the tile's stores issued (not waited for) and LDS still in
// use by the write-out: a caller that runs another tile afterwards puts a block barrier in between.
// `after_loads()` is called by every thread once the tile's last global load has been issued (before the write-out's
// stores; a fused Addition with more than four pieces per thread still loads its other input afterwards): a persistent
// caller starts the memory operations of its own bookkeeping there, behind the tile's loads.
struct NoTileHook
{
    __device__ __forceinline__ void operator()() const {}
};

template <int BM, int BN, int WM, int WN, int ST, bool U8, bool AW = false, bool UNIT = false, typename Hook = NoTileHook>
__device__ __forceinline__ void IgemmLdsTile(const IgemmArgs& a, const int tile, uint8_t* const smem, Hook after_loads = Hook())
{
    static_assert(ST >= 2 && ST <= 8, "2 to 8 LDS stages");
    static_assert((ST - 2) * (BM + BN) / (8 * WM * WN) < 64, "outstanding loads must fit the vmcnt counter");
    constexpr int BK = 128;
    constexpr int NW = WM * WN;                 // waves
    constexpr int NT = 64 * NW;                 // threads
    constexpr int WTM = BM / WM, WTN = BN / WN; // wave tile
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tiles are multiples of 32");
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "every wave loads whole 8-row groups");
    constexpr int RA = BM / (8 * NW);           // load instructions per wave and k-tile: activations (8 rows each)
    constexpr int RB = BN / (8 * NW);           //                                         weights
    constexpr int TP = WTM / 32, TC = WTN / 32;
    constexpr int STAGE = (BM + BN) * BK;
    constexpr int LDO = BN + 16;
    typedef __attribute__((address_space(3))) void* LdsPtr;
    typedef const __attribute__((address_space(1))) void* GlobalPtr;

    const int tn = tile % a.tiles_n;
    const int tm = tile / a.tiles_n;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    // ---- what this lane fetches: row (lane >> 3) of each 8-row group; the chunk whose slot is (lane & 7).  Row r of
    // the tile is 8 * (group index) + lrow, and a wave's first row is a multiple of 16, so (r >> 1) & 7 is
    // (lrow >> 1) + 4 * (group parity).
    const int lrow = lane >> 3;
    const int lchunk_even = (lane & 7) ^ (lrow >> 1);            // groups j = 0, 2, ...
    const int lchunk_odd = (lane & 7) ^ ((lrow >> 1) + 4);       // groups j = 1, 3, ...
    const uint8_t* xrow[RA];
    int iy0[RA], ix0[RA];
    bool mvalid[RA];
#pragma unroll
    for (int j = 0; j < RA; ++j)
    {
        const int m = tm * BM + wave * (BM / NW) + j * 8 + lrow;
        mvalid[j] = m < a.M;
        const int mm = min(m, a.M - 1);          // rows past the end re-read the last row (never stored)
        int n, oy, ox;
        if (a.unit)
        {
            // 1x1, stride 1, no padding (and FullyConnected): output pixel m reads input pixel m, so the tensor is walked
            // as one row of M pixels and the divisions below are not needed
            n = 0; oy = 0; ox = mm;
        }
        else
        {
            ox = mm % a.Wo;
            const int t = mm / a.Wo;
            oy = t % a.Ho;
            n = t / a.Ho;
        }
        iy0[j] = oy * a.stride_y - a.pad_top;
        ix0[j] = ox * a.stride_x - a.pad_left;
        // the chunk this lane would fetch for tap (0, 0), channel 0 (outside the tensor when that tap is padding; such
        // an address is never dereferenced)
        xrow[j] = a.x + static_cast<long long>(n) * a.H * a.W * a.Ci + (static_cast<long long>(iy0[j]) * a.W + ix0[j]) * a.Ci +
                  ((j & 1) ? lchunk_odd : lchunk_even) * 16;
    }
    static_assert((BM / NW) % 16 == 0 && (BN / NW) % 16 == 0, "a wave's first row is a multiple of 16");
    const int8_t* wrow = a.w + static_cast<long long>(tn * BN + wave * (BN / NW) + lrow) * a.K_pad;
    int ci = 0, kx = 0, ky = 0;                  // tap walk, identical in every thread
    // UNIT: lane offsets from the tensors' first bytes (rows past the end re-read the last row; their results are not stored)
    uint32_t aoff[RA], boff[RB];
    if constexpr (UNIT)
    {
#pragma unroll
        for (int j = 0; j < RA; ++j)
        {
            const int m = tm * BM + wave * (BM / NW) + j * 8 + lrow;
            aoff[j] = static_cast<uint32_t>(min(m, a.M - 1)) * static_cast<uint32_t>(a.Ci) + ((j & 1) ? lchunk_odd : lchunk_even) * 16;
        }
#pragma unroll
        for (int j = 0; j < RB; ++j)
            boff[j] = static_cast<uint32_t>(tn * BN + wave * (BN / NW) + j * 8 + lrow) * static_cast<uint32_t>(a.K_pad) + ((j & 1) ? lchunk_odd : lchunk_even) * 16;
    }

    auto load_tile = [&](int kt, int stage) {
        uint8_t* As = smem + stage * STAGE + wave * (BM / NW) * BK;
        uint8_t* Bs = smem + stage * STAGE + BM * BK + wave * (BN / NW) * BK;
        if constexpr (UNIT)
        {
            const uint8_t* abase = a.x + kt * BK;
            const int8_t* bbase = a.w + kt * BK;
#pragma unroll
            for (int j = 0; j < RA; ++j) __builtin_amdgcn_global_load_lds((GlobalPtr)(abase + aoff[j]), (LdsPtr)(As + j * 8 * BK), 16, 0, 0);
#pragma unroll
            for (int j = 0; j < RB; ++j) __builtin_amdgcn_global_load_lds((GlobalPtr)(bbase + boff[j]), (LdsPtr)(Bs + j * 8 * BK), 16, 0, 0);
            return;
        }
        const int dy = ky * a.dil_y, dx = kx * a.dil_x;
        const long long tap_off = (static_cast<long long>(dy) * a.W + dx) * a.Ci + ci;
#pragma unroll
        for (int j = 0; j < RA; ++j)
        {
            const int iy = iy0[j] + dy;
            const int ix = ix0[j] + dx;
            const bool ok = mvalid[j] && static_cast<unsigned>(iy) < static_cast<unsigned>(a.H) && static_cast<unsigned>(ix) < static_cast<unsigned>(a.W);
            // padding and rows past the end fetch 16 prepared bytes instead: every lane always delivers its slot
            const uint8_t* src = ok ? xrow[j] + tap_off : a.pad16;
            __builtin_amdgcn_global_load_lds((GlobalPtr)(src), (LdsPtr)(As + j * 8 * BK), 16, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < RB; ++j)
        {
            const int8_t* src = wrow + static_cast<long long>(j * 8) * a.K_pad + kt * BK + ((j & 1) ? lchunk_odd : lchunk_even) * 16;
            __builtin_amdgcn_global_load_lds((GlobalPtr)(src), (LdsPtr)(Bs + j * 8 * BK), 16, 0, 0);
        }
        ci += BK;
        if (ci >= a.Ci)
        {
            ci = 0;
            if (++kx == a.Kw) { kx = 0; ++ky; }
        }
    };

    // ---- accumulators start at the zero-point correction ---------------------------------------------------------
    const int lane_c = 4 * (lane >> 5);
    const int cbase = tn * BN + wn * WTN;
    v16i acc[TC][TP];
#pragma unroll
    for (int tc = 0; tc < TC; ++tc)
    {
        v16i init;
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const v4i c4 = *reinterpret_cast<const v4i*>(a.corr + cbase + tc * 32 + 8 * q + lane_c);
            init[4 * q + 0] = c4[0];
            init[4 * q + 1] = c4[1];
            init[4 * q + 2] = c4[2];
            init[4 * q + 3] = c4[3];
        }
#pragma unroll
        for (int tp = 0; tp < TP; ++tp) acc[tc][tp] = init;
    }

    const int nk = a.K_pad / BK;
    const int frag_row = lane & 31;
    const int frag_half = lane >> 5;
    const int xm = static_cast<int>(a.xor_mask);
    int rowsum[TP];
#pragma unroll
    for (int tp = 0; tp < TP; ++tp) rowsum[tp] = 0;

    // Fragment reads run ahead of the MFMAs that use them: a block that has a CU to itself has one wave per SIMD, and
    // nothing else hides a ds_read's latency between dependent read -> MFMA pairs.  Small wave tiles fetch the whole
    // k-tile's fragments first (32 VGPRs per fragment column); larger ones keep one k-step in flight.
    constexpr int KS = BK / 32;
    constexpr bool ALL_AHEAD = TP * TC <= 2;
    auto compute = [&](int stage) {
        const uint8_t* As = smem + stage * STAGE;
        const uint8_t* Bs = As + BM * BK;
        auto read_a = [&](int ks, int tp) {
            // chunk ks*2 + half of row r sits at slot chunk ^ ((r >> 1) & 7); fragment rows start at multiples of 32
            const int slot = ((ks * 2 + frag_half) ^ ((frag_row >> 1) & 7)) * 16;
            v4i f = *reinterpret_cast<const v4i*>(As + (wm * WTM + tp * 32 + frag_row) * BK + slot);
            if (U8) f ^= xm;
            return f;
        };
        auto read_w = [&](int ks, int tc) {
            const int slot = ((ks * 2 + frag_half) ^ ((frag_row >> 1) & 7)) * 16;
            return *reinterpret_cast<const v4i*>(Bs + (wn * WTN + tc * 32 + frag_row) * BK + slot);
        };
        auto multiply = [&](const v4i (&fa)[TP], const v4i (&fw)[TC]) {
            if constexpr (AW)
            {
#pragma unroll
                for (int tp = 0; tp < TP; ++tp)
#pragma unroll
                    for (int i = 0; i < 4; ++i) rowsum[tp] = __builtin_amdgcn_sdot4(fa[tp][i], 0x01010101, rowsum[tp], false);
            }
#pragma unroll
            for (int tc = 0; tc < TC; ++tc)
#pragma unroll
                for (int tp = 0; tp < TP; ++tp)
                    acc[tc][tp] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[tc], fa[tp], acc[tc][tp], 0, 0, 0);
        };
        if constexpr (ALL_AHEAD)
        {
            v4i fa[KS][TP], fw[KS][TC];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
            {
#pragma unroll
                for (int tp = 0; tp < TP; ++tp) fa[ks][tp] = read_a(ks, tp);
#pragma unroll
                for (int tc = 0; tc < TC; ++tc) fw[ks][tc] = read_w(ks, tc);
            }
            __builtin_amdgcn_sched_barrier(0);      // the scheduler would otherwise sink every read to just before its MFMA
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) multiply(fa[ks], fw[ks]);
        }
        else
        {
            v4i fa[2][TP], fw[2][TC];
#pragma unroll
            for (int tp = 0; tp < TP; ++tp) fa[0][tp] = read_a(0, tp);
#pragma unroll
            for (int tc = 0; tc < TC; ++tc) fw[0][tc] = read_w(0, tc);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
            {
                if (ks + 1 < KS)
                {
#pragma unroll
                    for (int tp = 0; tp < TP; ++tp) fa[(ks + 1) & 1][tp] = read_a(ks + 1, tp);
#pragma unroll
                    for (int tc = 0; tc < TC; ++tc) fw[(ks + 1) & 1][tc] = read_w(ks + 1, tc);
                }
                __builtin_amdgcn_sched_barrier(0);  // keep the next k-step's reads ahead of this k-step's MFMAs
                multiply(fa[ks & 1], fw[ks & 1]);
            }
        }
    };

    // ---- pipeline: ST - 1 tiles requested ahead ---------------------------------------------------------------------
#pragma unroll
    for (int s = 0; s < ST - 1; ++s)
        if (s < nk) load_tile(s, s);
    int stage = 0;
    for (int kt = 0; kt < nk; ++kt)
    {
        // tile kt has landed when at most the requests of the younger tiles (up to ST - 2 of them) are outstanding
        const int younger = min(ST - 2, nk - 1 - kt);
        if (ST >= 8 && younger == 6) __builtin_amdgcn_s_waitcnt(VmcntImm(6 * (RA + RB)));
        else if (ST >= 7 && younger == 5) __builtin_amdgcn_s_waitcnt(VmcntImm(5 * (RA + RB)));
        else if (ST >= 6 && younger == 4) __builtin_amdgcn_s_waitcnt(VmcntImm(4 * (RA + RB)));
        else if (ST >= 5 && younger == 3) __builtin_amdgcn_s_waitcnt(VmcntImm(3 * (RA + RB)));
        else if (ST >= 4 && younger == 2) __builtin_amdgcn_s_waitcnt(VmcntImm(2 * (RA + RB)));
        else if (ST >= 3 && younger == 1) __builtin_amdgcn_s_waitcnt(VmcntImm(RA + RB));
        else __builtin_amdgcn_s_waitcnt(VmcntImm(0));
        __syncthreads();                         // every wave's part of tile kt is in LDS; tile kt - 1 is no longer read
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

    // ---- epilogue: requantize, pack 4 channels per dword, stage the byte tile in LDS, coalesced write-out -----------
    uint8_t* Os = smem;
    constexpr int CHUNKS = BN / 16;
    constexpr int ROWS_PER_PASS = NT / CHUNKS;
    constexpr int NP = (BM + ROWS_PER_PASS - 1) / ROWS_PER_PASS;   // 16-byte pieces a thread writes
    const int oc = tid % CHUNKS;
    const int orow = tid / CHUNKS;
    const int c0 = tn * BN + oc * 16;
    // The other input of an Addition that runs in this write-out: every piece a thread will need is requested here, before
    // the requantization, from clamped addresses (no load waits inside a divergent branch).  Tiles of more than four
    // pieces per thread request them after the requantization instead, when the accumulators' registers are free.
    constexpr bool EARLY = NP <= 4;
    const bool fuse = a.res != nullptr && (a.Co & 15) == 0;
    v4i other[NP] = {};
    auto load_other = [&]() {
#pragma unroll
        for (int i = 0; i < NP; ++i)
        {
            const int m = min(tm * BM + min(orow + i * ROWS_PER_PASS, BM - 1), a.M - 1);
            other[i] = *reinterpret_cast<const v4i*>(a.res + static_cast<long long>(m) * a.Co + min(c0, a.Co - 16));
        }
    };
    if (EARLY && fuse) load_other();
    if constexpr (AW)
    {
#pragma unroll
        for (int tp = 0; tp < TP; ++tp) rowsum[tp] = (rowsum[tp] + __shfl_xor(rowsum[tp], 32) - a.rowsum_bias) * a.zw_neg;
    }
#pragma unroll
    for (int tc = 0; tc < TC; ++tc)
    {
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const int cl = wn * WTN + tc * 32 + 8 * q + lane_c;
            const Fast4 f4 = LoadFast4(a.ct, tn * BN + cl);
#pragma unroll
            for (int tp = 0; tp < TP; ++tp)
            {
                const v16i& c = acc[tc][tp];
                const int rt = AW ? rowsum[tp] : 0;
                const uint32_t out = Requant4Dev(c[4 * q + 0] + rt, c[4 * q + 1] + rt, c[4 * q + 2] + rt, c[4 * q + 3] + rt, f4, a.ct, tn * BN + cl, a.rq);
                const int pl = wm * WTM + tp * 32 + (lane & 31);
                *reinterpret_cast<uint32_t*>(Os + pl * LDO + cl) = out;
            }
        }
    }
    __syncthreads();
    after_loads();
    if (!EARLY && fuse) load_other();
    const OutPtr outp = MakeOutPtr(a.y, static_cast<long long>(a.M) * a.Co);
    if ((a.Co & 15) == 0)
    {
        if (c0 < a.Co)
        {
#pragma unroll
            for (int i = 0; i < NP; ++i)
            {
                const int r = orow + i * ROWS_PER_PASS;
                const int m = tm * BM + r;
                if (r < BM && m < a.M)
                {
                    v4i ov = *reinterpret_cast<const v4i*>(Os + r * LDO + oc * 16);
                    if (fuse) ov = AddResidual16(ov, other[i], a.add);
                    StoreOut16(outp, static_cast<long long>(m) * a.Co + c0, ov);
                }
            }
        }
    }
    else
    {
        for (int r = orow; r < BM; r += ROWS_PER_PASS)
        {
            const int m = tm * BM + r;
            if (m >= a.M) continue;
            for (int b = 0; b < 16; ++b)
            {
                const int c = c0 + b;
                if (c < a.Co) a.y[static_cast<long long>(m) * a.Co + c] = Os[r * LDO + oc * 16 + b];
            }
        }
    }
}

// One tile per block; consecutive block ids are dealt round-robin to the 8 XCDs, each with an L2 of its own.
//   xcd_cols == 1: XCD x takes the contiguous range of tiles [x * per_xcd, (x + 1) * per_xcd) in row-block-major order: the
//   column tiles of a row block share an L2, an activation row is fetched by one XCD, every XCD fetches all weights.
//   xcd_cols == 2 (even tiles_n): XCD x takes column half x >> 2 and the (x & 3)-th quarter of the row blocks: a weight is
//   fetched by four XCDs instead of eight, an activation row by two instead of one -- less traffic where the weights
//   outweigh a quarter of the activations.  The grid is 8 * IgemmLdsBlocksPerXcd() blocks either way.
__host__ __device__ inline int IgemmLdsBlocksPerXcd(int tiles_m, int tiles_n, int xcd_cols)
{
    if (xcd_cols == 2) return ((tiles_m + 3) / 4) * (tiles_n / 2);
    return (tiles_m * tiles_n + 7) / 8;
}

template <int BM, int BN, int WM, int WN, int ST, bool U8, bool AW = false, bool UNIT = false>
__global__ __launch_bounds__(64 * WM * WN) void IgemmLdsKernel(IgemmArgs a)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];   // IgemmLdsSmemBytes<BM, BN, ST>()
    const int x = static_cast<int>(blockIdx.x & 7), i = static_cast<int>(blockIdx.x >> 3);
    int tile;
    if (a.xcd_cols == 2)
    {
        const int half = a.tiles_n >> 1, rows_per = (a.tiles_m + 3) >> 2;
        const int tm = (x & 3) * rows_per + i / half;
        if (i >= rows_per * half || tm >= a.tiles_m) return;
        tile = tm * a.tiles_n + (x >> 2) * half + i % half;
    }
    else
    {
        const int nblocks = a.tiles_m * a.tiles_n;
        const int per_xcd = (nblocks + 7) >> 3;
        tile = x * per_xcd + i;
        if (i >= per_xcd || tile >= nblocks) return;
    }
    IgemmLdsTile<BM, BN, WM, WN, ST, U8, AW, UNIT>(a, tile, smem);
}

} // namespace mi355x
