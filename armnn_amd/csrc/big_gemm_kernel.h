// Implicit GEMM for the large launches: one wave per SIMD, each with a wave tile of up to 128 x 128 outputs.
//
// What the counters of the smaller-tiled kernels showed, and what this kernel does about it:
//   * A CU's vector L1 keeps only about a hundred cache lines on their way from L2 at once, so at the L2's latency
//     (300 clocks on a hit, around a thousand on a miss) a CU receives 28 to 45 bytes per clock, whatever the layout in
//     memory.  The matrix cores consume 4096 (BM + BN) / (BM BN) bytes per clock at full rate: 64 for 128 x 128 tiles,
//     48 for 256 x 128, 32 for 256 x 256.  Hence the largest tile the register file allows.
//   * The int32 accumulators of a 128 x 128 wave tile are 256 registers: they live in the accumulation registers
//     (AGPRs), the 256 architectural registers hold fragments, addresses and the epilogue (this file is compiled
//     without the "MFMA results in VGPRs" switch the other kernels use).
//   * With one wave per SIMD nothing hides a wait, so the k-loop is software-pipelined by hand: fragments are double
//     buffered in registers (the reads of k-step i + 1 are issued between the MFMAs of k-step i), the one block barrier
//     per k-tile sits in the tile's last k-step behind a few of its MFMAs, and the requests for the k-tile ST tiles
//     ahead are issued right behind it.  The steady-state loop body is one basic block so that the instruction groups
//     below pin the interleaving.
//   * k-tiles travel from global memory straight into LDS (global_load_lds_dwordx4), 128 bytes per row so that every
//     request is one whole cache line; dense rows with the chunk order xor-swizzled as in IgemmLdsKernel.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"
#include "igemm_lds_kernel.h"

namespace mi355x
{

template <int BM, int BN, int ST>
constexpr int BigGemmSmemBytes()
{
    constexpr int stages = ST * (BM + BN) * 128;
    constexpr int out = BM * (BN + 16);
    return (stages > out ? stages : out) + 4 * BN * 4;       // + the block's slice of the per-channel table
}

// 2 x 2 waves, wave tile (BM / 2) x (BN / 2).  Needs Ci % 128 == 0 (a k-tile is 128 bytes of one filter tap) and
// Co_pad % BN == 0.  U8 / AW as in IgemmLdsKernel.
// UNIT: 1x1 kernel, stride 1, no padding (and FullyConnected): a row's k-tiles are consecutive in memory, so a request's
// address is a per-row constant plus a scalar.  Otherwise every row carries a bit mask of the filter taps that fall inside
// the image for it (Kh * Kw <= 32), and a tap outside fetches 16 prepared padding bytes.
template <int BM, int BN, int ST, bool U8, bool AW, bool UNIT>
__global__ __launch_bounds__(256) void BigGemmKernel(IgemmArgs a, int xcd_rows)
{
    static_assert(ST >= 2 && ST <= 4, "2 to 4 LDS stages");
    constexpr int BK = 128, KS = 4;
    constexpr int WTM = BM / 2, WTN = BN / 2, TP = WTM / 32, TC = WTN / 32;
    constexpr int NM = TP * TC, NDS = TP + TC;
    constexpr int STAGE = (BM + BN) * BK;
    constexpr int RA = BM / 32, RB = BN / 32;          // wave-loads (8 rows x 128 bytes) per wave and k-tile
    constexpr int LDO = BN + 16;
    static_assert(NM >= 2 * NDS / 2 && NM / 4 >= 1, "enough MFMAs per k-step to carry the fragment reads");
    typedef __attribute__((address_space(3))) void* LdsPtr;
    typedef const __attribute__((address_space(1))) void* GlobalPtr;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];   // BigGemmSmemBytes<BM, BN, ST>()

    // ---- tile of this block: each XCD gets a contiguous run of tiles, walked xcd_rows tile rows at a time so that the
    // blocks resident together share both their activation rows and their weight rows in that XCD's L2
    const int nblocks = a.tiles_m * a.tiles_n;
    const int per_xcd = (nblocks + 7) >> 3;
    const int tile = static_cast<int>(blockIdx.x & 7) * per_xcd + static_cast<int>(blockIdx.x >> 3);
    if (tile >= nblocks) return;
    int tm, tn;
    {
        const int band = xcd_rows * a.tiles_n;
        const int b = tile / band, r = tile - b * band;
        const int rows = min(xcd_rows, a.tiles_m - b * xcd_rows);
        tn = r / rows;
        tm = b * xcd_rows + (r - tn * rows);
    }

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // ---- what this lane fetches: row (lane >> 3) of each 8-row group, the chunk that belongs in slot (lane & 7)
    const int lrow = lane >> 3;
    const int lchunk_even = (lane & 7) ^ (lrow >> 1);
    const int lchunk_odd = (lane & 7) ^ ((lrow >> 1) + 4);
    long long xoff[RA];                          // byte offset from a.x of the chunk this lane fetches for tap (0, 0), channel 0
    uint32_t tapmask[RA];                        // bit ky * Kw + kx: that tap of this row lies inside the image
#pragma unroll
    for (int j = 0; j < RA; ++j)
    {
        const int m = tm * BM + wave * (BM / 4) + j * 8 + lrow;
        const bool mvalid = m < a.M;
        const int chunk = ((j & 1) ? lchunk_odd : lchunk_even) * 16;
        if constexpr (UNIT)
        {
            // rows past the end read the last row again (their outputs are never stored)
            xoff[j] = static_cast<long long>(mvalid ? m : a.M - 1) * a.Ci + chunk;
            tapmask[j] = 1u;
        }
        else
        {
            const int mm = mvalid ? m : 0;
            const int ox = mm % a.Wo;
            const int t = mm / a.Wo;
            const int oy = t % a.Ho;
            const int n = t / a.Ho;
            const int iy0 = oy * a.stride_y - a.pad_top;
            const int ix0 = ox * a.stride_x - a.pad_left;
            xoff[j] = static_cast<long long>(n) * a.H * a.W * a.Ci + (static_cast<long long>(iy0) * a.W + ix0) * a.Ci + chunk;
            uint32_t mask = 0u;
            for (int ty = 0; ty < a.Kh; ++ty)
                for (int tx = 0; tx < a.Kw; ++tx)
                {
                    const int iy = iy0 + ty * a.dil_y, ix = ix0 + tx * a.dil_x;
                    const bool ok = mvalid & (static_cast<unsigned>(iy) < static_cast<unsigned>(a.H)) & (static_cast<unsigned>(ix) < static_cast<unsigned>(a.W));
                    mask |= (ok ? 1u : 0u) << (ty * a.Kw + tx);
                }
            tapmask[j] = mask;
        }
    }
    const int8_t* wrow = a.w + static_cast<long long>(tn * BN + wave * (BN / 4) + lrow) * a.K_pad;
    const long long wstep = 8ll * a.K_pad;
    int ci = 0, kx = 0, ky = 0;                  // tap walk, identical in every thread
    const long long pad_rel = a.pad16 - a.x;     // a chunk outside the image (or past the last row) fetches 16 prepared bytes

    auto load_tile = [&](int kt, int stage) {
        uint8_t* As = smem + stage * STAGE + wave * (BM / 4) * BK;
        uint8_t* Bs = smem + stage * STAGE + BM * BK + wave * (BN / 4) * BK;
        if constexpr (UNIT)
        {
            const uint8_t* xk = a.x + kt * BK;
#pragma unroll
            for (int j = 0; j < RA; ++j)
                __builtin_amdgcn_global_load_lds((GlobalPtr)(xk + xoff[j]), (LdsPtr)(As + j * 8 * BK), 16, 0, 0);
        }
        else
        {
            const int dy = ky * a.dil_y, dx = kx * a.dil_x;
            const long long tap_off = (static_cast<long long>(dy) * a.W + dx) * a.Ci + ci;
            const uint32_t tapbit = 1u << (ky * a.Kw + kx);
#pragma unroll
            for (int j = 0; j < RA; ++j)
            {
                // a select, not a branch: nothing may split the loop body
                const long long off = (tapmask[j] & tapbit) != 0u ? xoff[j] + tap_off : pad_rel;
                __builtin_amdgcn_global_load_lds((GlobalPtr)(a.x + off), (LdsPtr)(As + j * 8 * BK), 16, 0, 0);
            }
            // next tap, without branches (scalar selects)
            ci += BK;
            const int wrap_c = ci >= a.Ci ? 1 : 0;
            ci = wrap_c ? 0 : ci;
            kx += wrap_c;
            const int wrap_x = kx == a.Kw ? 1 : 0;
            kx = wrap_x ? 0 : kx;
            ky += wrap_x;
        }
        const int8_t* wk = wrow + kt * BK;
#pragma unroll
        for (int j = 0; j < RB; ++j)
            __builtin_amdgcn_global_load_lds((GlobalPtr)(wk + j * wstep + ((j & 1) ? lchunk_odd : lchunk_even) * 16), (LdsPtr)(Bs + j * 8 * BK), 16, 0, 0);
    };

    // ---- accumulators start at the zero-point correction
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
    const int frag_row = lane & 31, frag_half = lane >> 5;
    const int fsw = (frag_row >> 1) & 7;
    int aoff[KS], woff[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
    {
        const int slot = ((ks * 2 + frag_half) ^ fsw) * 16;
        aoff[ks] = (wm * WTM + frag_row) * BK + slot;
        woff[ks] = BM * BK + (wn * WTN + frag_row) * BK + slot;
    }
    const int xm = static_cast<int>(a.xor_mask);
    int rowsum[TP];
#pragma unroll
    for (int tp = 0; tp < TP; ++tp) rowsum[tp] = 0;

    v4i fa[2][TP], fw[2][TC];
    auto read_frags = [&](int stage, int ks, int buf) {
        const uint8_t* S = smem + stage * STAGE;
#pragma unroll
        for (int tp = 0; tp < TP; ++tp) fa[buf][tp] = *reinterpret_cast<const v4i*>(S + aoff[ks] + tp * 32 * BK);
#pragma unroll
        for (int tc = 0; tc < TC; ++tc) fw[buf][tc] = *reinterpret_cast<const v4i*>(S + woff[ks] + tc * 32 * BK);
    };
    // uint8 activations become int8 on the fragment registers; weights with a zero point need each pixel's sum
    auto prepare = [&](int buf) {
        if constexpr (U8 || AW)
        {
#pragma unroll
            for (int tp = 0; tp < TP; ++tp)
            {
                if (U8) fa[buf][tp] ^= xm;
                if constexpr (AW)
                {
#pragma unroll
                    for (int i = 0; i < 4; ++i) rowsum[tp] = __builtin_amdgcn_sdot4(fa[buf][tp][i], 0x01010101, rowsum[tp], false);
                }
            }
        }
    };
    auto mfmas_range = [&](int buf, int lo, int hi) {
#pragma unroll
        for (int i = lo; i < hi; ++i)
        {
            const int tc = i / TP, tp = i % TP;
            acc[tc][tp] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[buf][tc], fa[buf][tp], acc[tc][tp], 0, 0, 0);
        }
    };
    // k-steps 0 .. KS - 2 of the tile in `stage`: the next k-step's fragments are read between this one's MFMAs
    auto inner_steps = [&](int stage) {
#pragma unroll
        for (int ks = 0; ks < KS - 1; ++ks)
        {
            const int cur = ks & 1;
            read_frags(stage, ks + 1, cur ^ 1);
            prepare(cur);
            mfmas_range(cur, 0, NM);
#pragma unroll
            for (int i = 0; i < NDS; ++i)
            {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
            }
            __builtin_amdgcn_sched_group_barrier(0x008, NM - NDS, 0);
        }
    };
    constexpr int LAST = (KS - 1) & 1;           // fragment buffer of a tile's last k-step
    constexpr int PRE = NM / 4;                  // MFMAs of the last k-step issued ahead of the barrier

    // ---- the block's slice of the per-channel table (rows 2 .. 5: the fast path's bracket, BN channels) goes to LDS behind
    // the stages: with one wave per SIMD nothing would hide the epilogue's table reads from global memory, one round trip
    // per channel quad.  The rare exact path reads its two rows from global memory.
    constexpr int TAB = (ST * STAGE > BM * LDO ? ST * STAGE : BM * LDO);
    float* tab_lds = reinterpret_cast<float*>(smem + TAB);
    {
        constexpr int N4 = 4 * BN / 4;                     // float4 pieces
        v4i piece[(N4 + 255) / 256];
#pragma unroll
        for (int i = 0; i < (N4 + 255) / 256; ++i)
        {
            const int e = i * 256 + tid;
            const int row = e / (BN / 4), col = e - row * (BN / 4);
            if (e < N4) piece[i] = *reinterpret_cast<const v4i*>(a.ct.p + static_cast<long long>(row + 2) * a.ct.stride + tn * BN + col * 4);
        }
        // ---- prologue: ST tiles requested behind the table reads (older requests complete first) ...
#pragma unroll
        for (int s = 0; s < ST; ++s)
            if (s < nk) load_tile(s, s);
#pragma unroll
        for (int i = 0; i < (N4 + 255) / 256; ++i)
        {
            const int e = i * 256 + tid;
            if (e < N4) *reinterpret_cast<v4i*>(tab_lds + e * 4) = piece[i];
        }
    }
    // ... and the first one waited for
    {
        const int younger = min(ST - 1, nk - 1);
        if (ST >= 4 && younger == 3) __builtin_amdgcn_s_waitcnt(VmcntImm(3 * (RA + RB)));
        else if (ST >= 3 && younger == 2) __builtin_amdgcn_s_waitcnt(VmcntImm(2 * (RA + RB)));
        else if (younger == 1) __builtin_amdgcn_s_waitcnt(VmcntImm(RA + RB));
        else __builtin_amdgcn_s_waitcnt(VmcntImm(0));
    }
    __syncthreads();
    read_frags(0, 0, 0);

    int stage = 0;
    int kt = 0;
    // ---- steady state: every iteration requests tile kt + ST and finds ST - 2 younger requests behind tile kt + 1
    for (; kt + ST < nk; ++kt)
    {
        int nstage = stage + 1;
        if (nstage == ST) nstage = 0;
        inner_steps(stage);
        __builtin_amdgcn_sched_barrier(0);
        prepare(LAST);
        mfmas_range(LAST, 0, PRE);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(VmcntImm((ST - 2) * (RA + RB)));
        __syncthreads();      // tile kt + 1 is in LDS for every wave; nobody reads tile kt any more
        __builtin_amdgcn_sched_barrier(0);
        read_frags(nstage, 0, LAST ^ 1);
        load_tile(kt + ST, stage);
        mfmas_range(LAST, PRE, NM);
        {
            constexpr int REST = NM - PRE;
            constexpr int NA_ = (NDS + 1) / 2;              // MFMAs that carry two fragment reads each
            constexpr int NB_ = REST - NA_;                 // MFMAs that carry the requests
            constexpr int VM = (RA + RB + NB_ - 1) / NB_;
#pragma unroll
            for (int i = 0; i < NA_; ++i)
            {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            }
#pragma unroll
            for (int i = 0; i < NB_; ++i)
            {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, VM, 0);   // global -> LDS requests
            }
        }
        stage = nstage;
    }
    // ---- tail: nothing left to request
    for (; kt < nk; ++kt)
    {
        int nstage = stage + 1;
        if (nstage == ST) nstage = 0;
        inner_steps(stage);
        prepare(LAST);
        if (kt + 1 < nk)
        {
            const int younger = nk - 2 - kt;      // 0 .. ST - 2
            if (ST >= 4 && younger == 2) __builtin_amdgcn_s_waitcnt(VmcntImm(2 * (RA + RB)));
            else if (ST >= 3 && younger == 1) __builtin_amdgcn_s_waitcnt(VmcntImm(RA + RB));
            else __builtin_amdgcn_s_waitcnt(VmcntImm(0));
            __syncthreads();
            read_frags(nstage, 0, LAST ^ 1);
        }
        mfmas_range(LAST, 0, NM);
        stage = nstage;
    }
    __syncthreads();

    // ---- epilogue: requantize, pack 4 channels per dword, stage the byte tile in LDS, coalesced write-out
    uint8_t* Os = smem;
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
            const float4 mp = *reinterpret_cast<const float4*>(tab_lds + 0 * BN + cl);
            const float4 bp = *reinterpret_cast<const float4*>(tab_lds + 1 * BN + cl);
            const float4 mm = *reinterpret_cast<const float4*>(tab_lds + 2 * BN + cl);
            const float4 bm = *reinterpret_cast<const float4*>(tab_lds + 3 * BN + cl);
#pragma unroll
            for (int tp = 0; tp < TP; ++tp)
            {
                const v16i& c = acc[tc][tp];
                const int rt = AW ? rowsum[tp] : 0;
                const uint32_t out = Requant4Dev(c[4 * q + 0] + rt, c[4 * q + 1] + rt, c[4 * q + 2] + rt, c[4 * q + 3] + rt, mp, bp, mm, bm, a.ct, nullptr, tn * BN + cl, a.rq);
                const int pl = wm * WTM + tp * 32 + (lane & 31);
                *reinterpret_cast<uint32_t*>(Os + pl * LDO + cl) = out;
            }
        }
    }
    __syncthreads();
    constexpr int CHUNKS = BN / 16;
    constexpr int ROWS_PER_PASS = 256 / CHUNKS;
    const int oc = tid % CHUNKS;
    const int orow = tid / CHUNKS;
    const int c0 = tn * BN + oc * 16;
    const OutPtr outp = MakeOutPtr(a.y, static_cast<long long>(a.M) * a.Co);
    if ((a.Co & 15) == 0)
    {
        if (c0 < a.Co)
        {
#pragma unroll 4
            for (int r = orow; r < BM; r += ROWS_PER_PASS)
            {
                const int m = tm * BM + r;
                if (m < a.M)
                    StoreOut16(outp, static_cast<long long>(m) * a.Co + c0, *reinterpret_cast<const v4i*>(Os + r * LDO + oc * 16));
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

} // namespace mi355x
