// The 64 x 64-tile direct-to-LDS implicit GEMM with K split over the waves of a block, for launches of at most about one
// block per CU and a long K (late ResNet layers at small batch, FullyConnected with a few hundred rows).
//
// Such a block has a CU to itself, and with four waves every SIMD holds ONE wave: the k-loop then runs at that wave's
// instruction issue rate -- about 120 instructions per k-tile (address arithmetic of the gather, tap walk, waits, eight
// fragment reads, four MFMAs), each waiting for its predecessor, 600 to 900 clocks per tile whatever the number of
// stages in flight, the tile shape or the number of blocks.  Here a block has KG groups of four waves; group g walks
// k-tiles g, g + KG, ... with LDS stages of its own, so a SIMD interleaves KG instruction streams.  After the loop the
// groups' int32 partial tiles meet in LDS (no memory outside the block is involved, so the result does not depend on
// timing), group 0 adds them in a fixed order and runs the usual epilogue.  Integer sums: the bytes are those of
// IgemmLdsKernel.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"
#include "igemm_lds_kernel.h"

namespace mi355x
{

template <int KG, int ST>
constexpr int IgemmKSplitSmemBytes()
{
    constexpr int stages = KG * ST * 128 * 128;
    constexpr int partials = 8192 + (KG - 1) * 4 * 4096;
    return stages > partials ? stages : partials;
}

template <int KG, int ST, bool U8>
__global__ __launch_bounds__(256 * KG) void IgemmKSplitKernel(IgemmArgs a)
{
    static_assert(KG == 2 || KG == 4, "2 or 4 k-groups");
    static_assert(ST == 2 || ST == 3, "2 or 3 LDS stages per group");
    constexpr int BM = 64, BN = 64, BK = 128;
    constexpr int NT = 256 * KG;
    constexpr int RA = 2, RB = 2;                // load instructions per wave and k-tile (8 rows each)
    constexpr int STAGE = (BM + BN) * BK;
    constexpr int LDO = BN + 16;
    constexpr int POFF = 8192;                   // partial tiles start behind the output staging area
    static_assert(BM * LDO <= POFF, "output staging fits in front of the partial tiles");
    typedef __attribute__((address_space(3))) void* LdsPtr;
    typedef const __attribute__((address_space(1))) void* GlobalPtr;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];   // IgemmKSplitSmemBytes<KG, ST>()

    const int nblocks = a.tiles_m * a.tiles_n;
    const int per_xcd = (nblocks + 7) >> 3;
    const int tile = static_cast<int>(blockIdx.x & 7) * per_xcd + static_cast<int>(blockIdx.x >> 3);
    if (tile >= nblocks) return;
    const int tn = tile % a.tiles_n;
    const int tm = tile / a.tiles_n;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int grp = tid >> 8;                    // k-group
    const int wave = (tid >> 6) & 3;             // wave within the group
    const int wm = wave >> 1, wn = wave & 1;
    uint8_t* gsmem = smem + grp * (ST * STAGE);

    // ---- what this lane fetches (the layout of IgemmLdsKernel) --------------------------------------------------------
    const int lrow = lane >> 3;
    const int lchunk_even = (lane & 7) ^ (lrow >> 1);
    const int lchunk_odd = (lane & 7) ^ ((lrow >> 1) + 4);
    const uint8_t* xrow[RA];
    int iy0[RA], ix0[RA];
    bool mvalid[RA];
#pragma unroll
    for (int j = 0; j < RA; ++j)
    {
        const int m = tm * BM + wave * 16 + j * 8 + lrow;
        mvalid[j] = m < a.M;
        const int mm = mvalid[j] ? m : 0;
        int n, oy, ox;
        if (a.unit)
        {
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
        xrow[j] = a.x + static_cast<long long>(n) * a.H * a.W * a.Ci + (static_cast<long long>(iy0[j]) * a.W + ix0[j]) * a.Ci +
                  ((j & 1) ? lchunk_odd : lchunk_even) * 16;
    }
    const int8_t* wrow = a.w + static_cast<long long>(tn * BN + wave * 16 + lrow) * a.K_pad;
    int ci = 0, kx = 0, ky = 0;                  // tap walk, identical in every thread of a group
    auto advance = [&](int tiles) {
        for (int i = 0; i < tiles; ++i)
        {
            ci += BK;
            if (ci >= a.Ci)
            {
                ci = 0;
                if (++kx == a.Kw) { kx = 0; ++ky; }
            }
        }
    };
    advance(grp);                                // this group's first k-tile is tile `grp`

    auto load_tile = [&](int kt, int stage) {
        uint8_t* As = gsmem + stage * STAGE + wave * 16 * BK;
        uint8_t* Bs = gsmem + stage * STAGE + BM * BK + wave * 16 * BK;
        const int dy = ky * a.dil_y, dx = kx * a.dil_x;
        const long long tap_off = (static_cast<long long>(dy) * a.W + dx) * a.Ci + ci;
#pragma unroll
        for (int j = 0; j < RA; ++j)
        {
            const int iy = iy0[j] + dy;
            const int ix = ix0[j] + dx;
            const bool ok = mvalid[j] && static_cast<unsigned>(iy) < static_cast<unsigned>(a.H) && static_cast<unsigned>(ix) < static_cast<unsigned>(a.W);
            const uint8_t* src = ok ? xrow[j] + tap_off : a.pad16;
            __builtin_amdgcn_global_load_lds((GlobalPtr)(src), (LdsPtr)(As + j * 8 * BK), 16, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < RB; ++j)
        {
            const int8_t* src = wrow + static_cast<long long>(j * 8) * a.K_pad + kt * BK + ((j & 1) ? lchunk_odd : lchunk_even) * 16;
            __builtin_amdgcn_global_load_lds((GlobalPtr)(src), (LdsPtr)(Bs + j * 8 * BK), 16, 0, 0);
        }
        advance(KG);
    };

    // ---- accumulators: group 0 starts at the zero-point correction, the others at zero ------------------------------------
    const int lane_c = 4 * (lane >> 5);
    const int cbase = tn * BN + wn * 32;
    v16i acc;
#pragma unroll
    for (int q = 0; q < 4; ++q)
    {
        v4i c4 = {0, 0, 0, 0};
        if (grp == 0) c4 = *reinterpret_cast<const v4i*>(a.corr + cbase + 8 * q + lane_c);
        acc[4 * q + 0] = c4[0]; acc[4 * q + 1] = c4[1]; acc[4 * q + 2] = c4[2]; acc[4 * q + 3] = c4[3];
    }

    const int nk = a.K_pad / BK;
    const int nkg = grp < nk ? (nk - grp + KG - 1) / KG : 0;     // k-tiles of this group
    const int iters = (nk + KG - 1) / KG;                        // the same for every group: barriers are block-wide
    const int frag_row = lane & 31;
    const int frag_half = lane >> 5;
    const int xm = static_cast<int>(a.xor_mask);

    auto compute = [&](int stage) {
        const uint8_t* As = gsmem + stage * STAGE;
        const uint8_t* Bs = As + BM * BK;
        v4i fa[4], fw[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
        {
            const int slot = ((ks * 2 + frag_half) ^ ((frag_row >> 1) & 7)) * 16;
            fa[ks] = *reinterpret_cast<const v4i*>(As + (wm * 32 + frag_row) * BK + slot);
            if (U8) fa[ks] ^= xm;
            fw[ks] = *reinterpret_cast<const v4i*>(Bs + (wn * 32 + frag_row) * BK + slot);
        }
        __builtin_amdgcn_sched_barrier(0);       // all fragment reads first, then the MFMAs
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[ks], fa[ks], acc, 0, 0, 0);
    };

#pragma unroll
    for (int s = 0; s < ST - 1; ++s)
        if (s < nkg) load_tile(grp + s * KG, s);
    int stage = 0;
    for (int it = 0; it < iters; ++it)
    {
        if (it < nkg)
        {
            // this group's tile `it` has landed when at most its younger tiles' requests are outstanding
            const int younger = min(ST - 2, nkg - 1 - it);
            if (ST >= 3 && younger == 1) __builtin_amdgcn_s_waitcnt(VmcntImm(RA + RB));
            else __builtin_amdgcn_s_waitcnt(VmcntImm(0));
        }
        __syncthreads();
        if (it + ST - 1 < nkg)
        {
            int ls = stage + ST - 1;
            if (ls >= ST) ls -= ST;
            load_tile(grp + (it + ST - 1) * KG, ls);
        }
        if (it < nkg) compute(stage);
        if (++stage == ST) stage = 0;
    }
    __syncthreads();

    // ---- the groups' partial tiles meet in LDS; group 0 adds them in the order 1, 2, ... -------------------------------------
    v4i* part = reinterpret_cast<v4i*>(smem + POFF);
    if (grp > 0)
    {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            part[(((grp - 1) * 4 + wave) * 4 + q) * 64 + lane] = v4i{acc[4 * q + 0], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
    }
    __syncthreads();
    uint8_t* Os = smem;
    if (grp == 0)
    {
#pragma unroll
        for (int g = 1; g < KG; ++g)
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const v4i p4 = part[(((g - 1) * 4 + wave) * 4 + q) * 64 + lane];
                acc[4 * q + 0] += p4[0]; acc[4 * q + 1] += p4[1]; acc[4 * q + 2] += p4[2]; acc[4 * q + 3] += p4[3];
            }
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const int cl = wn * 32 + 8 * q + lane_c;
            const Fast4 f4 = LoadFast4(a.ct, tn * BN + cl);
            const uint32_t out = Requant4Dev(acc[4 * q + 0], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3], f4, a.ct, tn * BN + cl, a.rq);
            const int pl = wm * 32 + (lane & 31);
            *reinterpret_cast<uint32_t*>(Os + pl * LDO + cl) = out;
        }
    }
    __syncthreads();
    constexpr int CHUNKS = BN / 16;
    constexpr int ROWS_PER_PASS = NT / CHUNKS;
    const int oc = tid % CHUNKS;
    const int orow = tid / CHUNKS;
    const int c0 = tn * BN + oc * 16;
    const OutPtr outp = MakeOutPtr(a.y, static_cast<long long>(a.M) * a.Co);
    if ((a.Co & 15) == 0)
    {
        if (c0 < a.Co)
        {
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
