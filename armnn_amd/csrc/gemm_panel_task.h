// Work unit of a persistent launch for 1x1 stride-1 unpadded convolutions (a GEMM with K = input channels): ONE block
// computes 64 output rows over ALL output channels.
//   * The 64 x K activation panel goes to LDS once (K <= 512: at most 32 KB) and stays there; only the weights stream,
//     64 channels x 128 bytes per step, through a ring of ST slots (global_load_lds, no staging registers).  A 64 x 64
//     tile launched on its own re-reads the panel for every column tile: 64 KB through the CU's vector L1 per tile
//     against 36 KB here, and the L1 fill rate is what bounds these layers.
//   * The weight stream never drains inside the unit: the steps (column tile, k-tile) are walked as one sequence, so
//     while a column tile is requantized and stored the loads of the next one are already in flight.  Vector memory
//     operations of a wave complete in issue order on this architecture, loads and stores alike, so the wait for a ring slot
//     counts the stores issued since as well.
//   * No vector load sits inside the sequence: a load's result can only be awaited together with everything issued
//     before it, which would drain the weight stream at every column tile.  So the accumulators start at zero (the
//     zero-point correction is part of the bracket constants, rows 6 / 7 of the channel table) and the four bracket rows
//     of all output channels are staged in LDS before the first step.
//   * LDS images, swizzle, fragment reads and MFMA shape are those of IgemmLdsTile<64, 64, 2, 2>, and the requantization
//     bracket closes on the exact result or falls back to it: the bytes written are identical.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"
#include "igemm_lds_kernel.h"

namespace mi355x
{

// ncol: output channels rounded up to whole 64-wide column tiles
template <int ST, int NK>
constexpr int GemmPanelSmemBytes(int ncol)
{
    return NK * 64 * 128 + ST * 64 * 128 + 64 * (64 + 16) + 4 * ncol * 4;
}
constexpr int kGemmPanelMaxCols = 1024;

// a: arguments as for IgemmLdsTile with a.unit set (tiles_m / tiles_n for 64 x 64 tiles); tm: the row block.
// NK = K_pad / 128 (1 .. 4), ST - 1 <= NK.
template <int ST, int NK, bool U8>
__device__ __forceinline__ void GemmPanelTask(const IgemmArgs& a, const int tm, uint8_t* const smem)
{
    static_assert(ST >= 2 && ST - 1 <= NK, "the stores of one column tile must be older than the slot awaited ST - 1 steps later");
    constexpr int BK = 128, BM = 64, BN = 64, NW = 4;
    constexpr int RA = BM / (8 * NW), RB = BN / (8 * NW);     // 2 load instructions per wave and k-tile for each operand
    constexpr int LDO = BN + 16;
    constexpr int NT = 256;
    constexpr int CHUNKS = BN / 16, ROWS_PER_PASS = NT / CHUNKS, NP = BM / ROWS_PER_PASS;   // 4 stores of 16 bytes per thread and column tile
    typedef __attribute__((address_space(3))) void* LdsPtr;
    typedef const __attribute__((address_space(1))) void* GlobalPtr;
    uint8_t* const panel = smem;                              // [NK][64 rows][128 B]
    uint8_t* const ring = smem + NK * BM * BK;                // [ST][64 channels][128 B]
    uint8_t* const Os = ring + ST * BN * BK;                  // [64][LDO] output bytes of one column tile
    float* const tab = reinterpret_cast<float*>(Os + BM * LDO); // [4][ncol]: m+, b+ with corr folded in, m-, b- with corr folded in

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane >> 3;
    const int lchunk_even = (lane & 7) ^ (lrow >> 1);
    const int lchunk_odd = (lane & 7) ^ ((lrow >> 1) + 4);
    uint32_t aoff[RA], boff[RB];
#pragma unroll
    for (int j = 0; j < RA; ++j)
    {
        const int m = tm * BM + wave * (BM / NW) + j * 8 + lrow;
        aoff[j] = static_cast<uint32_t>(min(m, a.M - 1)) * static_cast<uint32_t>(a.Ci) + ((j & 1) ? lchunk_odd : lchunk_even) * 16;
    }
#pragma unroll
    for (int j = 0; j < RB; ++j)
        boff[j] = static_cast<uint32_t>(wave * (BN / NW) + j * 8 + lrow) * static_cast<uint32_t>(a.K_pad) + ((j & 1) ? lchunk_odd : lchunk_even) * 16;

    const int tiles_n = a.tiles_n;
    const int steps = tiles_n * NK;
    const int ncol = tiles_n * BN;                             // <= the table's row stride (channels are padded to 128)
    // the bracket rows of every output channel: requested first, written to LDS once the panel and the first weight tiles
    // have been requested behind them
    constexpr int TABV = 4 * kGemmPanelMaxCols / 4 / NT;       // float4 pieces per thread at most
    float4 tv[TABV];
#pragma unroll
    for (int i = 0; i < TABV; ++i)
    {
        const int e = min(tid + i * NT, ncol - 1);             // float4 index within [4][ncol / 4], clamped
        const int row = e / (ncol / 4), col4 = e - row * (ncol / 4);
        const int src_row = row == 0 ? 2 : row == 1 ? 6 : row == 2 ? 4 : 7;
        tv[i] = *reinterpret_cast<const float4*>(a.ct.p + src_row * a.ct.stride + col4 * 4);
    }
    // weights of step s = (column tile s / NK, k-tile s % NK) into ring slot `slot`
    auto load_b = [&](int s, int slot) {
        const int tn = s / NK, kt = s - tn * NK;
        const int8_t* bbase = a.w + static_cast<long long>(tn) * BN * a.K_pad + kt * BK;
        uint8_t* Bs = ring + slot * BN * BK + wave * (BN / NW) * BK;
#pragma unroll
        for (int j = 0; j < RB; ++j) __builtin_amdgcn_global_load_lds((GlobalPtr)(bbase + boff[j]), (LdsPtr)(Bs + j * 8 * BK), 16, 0, 0);
    };
    // ---- the panel, then the first ST - 1 weight tiles ------------------------------------------------------------------
#pragma unroll
    for (int kt = 0; kt < NK; ++kt)
    {
        uint8_t* As = panel + kt * BM * BK + wave * (BM / NW) * BK;
#pragma unroll
        for (int j = 0; j < RA; ++j) __builtin_amdgcn_global_load_lds((GlobalPtr)(a.x + kt * BK + aoff[j]), (LdsPtr)(As + j * 8 * BK), 16, 0, 0);
    }
#pragma unroll
    for (int s = 0; s < ST - 1; ++s)
        if (s < steps) load_b(s, s);

#pragma unroll
    for (int i = 0; i < TABV; ++i)
        if (tid + i * NT < ncol) *reinterpret_cast<float4*>(tab + (tid + i * NT) * 4) = tv[i];
    // (the first step's barrier orders these writes before the first write-out reads them)

    const int lane_c = 4 * (lane >> 5);
    const int frag_row = lane & 31;
    const int frag_half = lane >> 5;
    const int xm = static_cast<int>(a.xor_mask);
    const int oc = tid % CHUNKS;
    const int orow = tid / CHUNKS;
    const OutPtr outp = MakeOutPtr(a.y, static_cast<long long>(a.M) * a.Co);

    int slot = 0;
    for (int tn = 0; tn < tiles_n; ++tn)
    {
        v16i acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int kt = 0; kt < NK; ++kt)
        {
            const int s = tn * NK + kt;
            // Slot of step s has landed when at most the operations issued after its loads are outstanding: the loads of the
            // up to ST - 2 younger steps and, during the first ST - 1 steps of a column tile, the NP stores of the tile before
            // (issued after the loads of step s).
            const int younger = min(ST - 2, steps - 1 - s);
            const bool stores_between = tn > 0 && kt < ST - 1;
            // (the counts are small compile-time sets; vmcnt immediates must be constants)
            if (stores_between)
            {
                if (younger >= 2) __builtin_amdgcn_s_waitcnt(VmcntImm(2 * RB + NP));
                else if (younger == 1) __builtin_amdgcn_s_waitcnt(VmcntImm(RB + NP));
                else __builtin_amdgcn_s_waitcnt(VmcntImm(NP));
            }
            else
            {
                if (younger >= 2) __builtin_amdgcn_s_waitcnt(VmcntImm(2 * RB));
                else if (younger == 1) __builtin_amdgcn_s_waitcnt(VmcntImm(RB));
                else __builtin_amdgcn_s_waitcnt(VmcntImm(0));
            }
            __syncthreads();                     // every wave's part of step s is in LDS; the slot of step s - 1 is no longer read
            if (s + ST - 1 < steps)
            {
                int ls = slot + ST - 1;
                if (ls >= ST) ls -= ST;
                load_b(s + ST - 1, ls);
            }
            const uint8_t* As = panel + kt * BM * BK;
            const uint8_t* Bs = ring + slot * BN * BK;
            v4i fa[4], fw[4];
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
            {
                const int sl = ((ks * 2 + frag_half) ^ ((frag_row >> 1) & 7)) * 16;
                fa[ks] = *reinterpret_cast<const v4i*>(As + (wm * 32 + frag_row) * BK + sl);
                if (U8) fa[ks] ^= xm;
                fw[ks] = *reinterpret_cast<const v4i*>(Bs + (wn * 32 + frag_row) * BK + sl);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[ks], fa[ks], acc, 0, 0, 0);
            if (++slot == ST) slot = 0;
        }
        // ---- write-out of column tile tn (the next tiles' weights are on their way meanwhile) ------------------------------
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const int cl = wn * 32 + 8 * q + lane_c;
            const int c = tn * BN + cl;
            const float4 mp = *reinterpret_cast<const float4*>(tab + c);
            const float4 bp = *reinterpret_cast<const float4*>(tab + ncol + c);
            const float4 mm = *reinterpret_cast<const float4*>(tab + 2 * ncol + c);
            const float4 bm = *reinterpret_cast<const float4*>(tab + 3 * ncol + c);
            // the rare exact path reads rows 0 / 1 and the correction from global memory (and waits for everything in flight)
            const uint32_t out = Requant4Dev(acc[4 * q + 0], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3], mp, bp, mm, bm, a.ct, a.corr, c, a.rq);
            const int pl = wm * 32 + (lane & 31);
            *reinterpret_cast<uint32_t*>(Os + pl * LDO + cl) = out;
        }
        __syncthreads();
        // Every wave issues exactly NP store instructions per column tile (the slot accounting above counts them): rows past
        // the end of the tensor store the last row's bytes to the last row once more, the same bytes its owner writes;
        // channel chunks past the end are masked lanes of an instruction the wave issues anyway (chunk 0 always exists).
        const int c0 = tn * BN + oc * 16;
#pragma unroll
        for (int i = 0; i < NP; ++i)
        {
            const int m = min(tm * BM + orow + i * ROWS_PER_PASS, a.M - 1);
            const int r = m - tm * BM;
            const v4i ov = *reinterpret_cast<const v4i*>(Os + r * LDO + oc * 16);
            if (c0 < a.Co) StoreOut16(outp, static_cast<long long>(m) * a.Co + c0, ov);
        }
    }
}

} // namespace mi355x
