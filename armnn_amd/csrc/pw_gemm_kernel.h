// Pointwise (1x1, stride 1, unpadded) Convolution2d and FullyConnected as a weight-stationary GEMM on MFMA.
//
//   out[m][n] = requant( sum_k A[m][k] * W[n][k] ),  A = activations [M][K] (NHWC rows are pixels), W = [N][K].
//
//   A block keeps its BN x K weight slab in LDS for its whole life and walks over 32-row tiles of A.  Each wave owns
//   whole tiles: it reads its MFMA "B" fragments (lane = pixel row, 16 contiguous K bytes) straight from global
//   memory into registers -- NHWC makes them contiguous -- NB-1 register chunks ahead of the MFMAs, so there is no
//   LDS staging of activations, no block barrier after the prologue, and many 16-byte loads in flight per lane.
//   The epilogue requantizes 4 channels at a time, stages the 32 x BN byte tile in the wave's private LDS area and
//   writes it with 16-byte row-contiguous stores.
//
//   Zero points: uint8 activations are xor-ed with 0x80 in registers; acc = sum x' w, and the per-channel constant
//   corr[n] = -zx' * sum_k w[n][k] is folded into the requantization constants (rows 5/6 of the channel table) on
//   the fast path and added to the accumulator on the exact path.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"

namespace mi355x
{

struct PwArgs
{
    const uint8_t* x;
    const int8_t*  w;        // [>= n_slabs*BN][w_stride], rows zero padded
    ChanTab        ct;       // rows 0,1 exact; rows 2,5,6: fm, fb + corr*fm, threshold for the corr-folded form
    const int32_t* corr;
    uint8_t*       y;
    int M, K, N;
    int w_stride;
    int n_slabs, gm;         // grid = n_slabs * gm blocks; block (slab, g) takes tile groups g, g+gm, ...
    uint32_t xor_mask;
    int zw_neg;              // AW: minus the zero point of the stored int8 weights
    const uint8_t* res;      // the other input of an Addition fused into the write-out ([M][N]), or null
    AddFuse add;
    Requant rq;
};

template <int BN>
constexpr int PwSmemBytes(int K)
{
    return BN * (K + 16) + 4 * 32 * (BN + 16) + 4 * BN * 4;
}

// KS = MFMA k-steps (of 32) per register chunk, K % (32 * KS) == 0;  NB = register chunks per wave (NB-1 in flight).
// AW: the weights have a zero point zw'; a lane sums the activation bytes it feeds to the MFMAs (v_dot4 with ones), the two
// lanes holding the halves of a row's k-slices add up, and -zw' times that sum joins the row's accumulators.
template <int BN, int KS, int NB, bool AW = false>
__global__ __launch_bounds__(256) void PwGemmKernel(PwArgs a)
{
    constexpr int TC = BN / 32;
    constexpr int LDO = BN + 16;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int LDW = a.K + 16;
    uint8_t* slab = smem;
    float* cst = reinterpret_cast<float*>(smem + BN * LDW);                 // [4][BN]: the corr-folded bracket m+, bc+, m-, bc-
    uint8_t* ostage_all = smem + BN * LDW + 4 * BN * 4;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    // Consecutive block ids land on different XCDs (8 per device, each with its own L2).  All slabs of one group of
    // activation rows are given to the same XCD, so those rows cross the fabric once and are then served from that
    // XCD's L2; the (small) weight slabs are what gets replicated.
    const int xcd = blockIdx.x & 7;
    const int local = blockIdx.x >> 3;
    const int slab_id = local % a.n_slabs;
    const int g = (local / a.n_slabs) * 8 + xcd;
    const int n0 = slab_id * BN;

    uint8_t* ostage = ostage_all + wave * 32 * LDO;
    const int n_tiles = (a.M + 31) >> 5;
    const OutPtr outp = MakeOutPtr(a.y, static_cast<long long>(a.M) * a.N);
    const int nch = a.K / (32 * KS);
    const int frag_row = lane & 31;
    const int frag_k = (lane >> 5) * 16;
    const int xm = static_cast<int>(a.xor_mask);
    const int tile_step = a.gm * 4;
    const int tile0 = g * 4 + wave;              // first tile of this wave

    v16i acc[TC];
    int rowsum = 0;

    auto load_chunk = [&](v4i (&buf)[KS], int t, int ch) {
        // rows past the end re-read the last row (their results are never stored): no load depends on a branch
        const int row = min(t * 32 + frag_row, a.M - 1);
        const uint8_t* p = a.x + static_cast<long long>(row) * a.K + ch * (32 * KS) + frag_k;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) buf[ks] = *reinterpret_cast<const v4i*>(p + ks * 32);
    };

    // FIRST: the chunk opens a tile; its first MFMA takes a zero C operand instead of cleared registers
    auto compute_chunk = [&](v4i (&buf)[KS], int ch, auto first) {
        constexpr bool FIRST = decltype(first)::value;
        const uint8_t* wbase = slab + frag_row * LDW + ch * (32 * KS) + frag_k;
        const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
        {
            const v4i av = buf[ks] ^ xm;
            if constexpr (AW)
            {
                if (FIRST && ks == 0) rowsum = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) rowsum = __builtin_amdgcn_sdot4(av[i], 0x01010101, rowsum, false);
            }
#pragma unroll
            for (int tc = 0; tc < TC; ++tc)
            {
                const v4i wv = *reinterpret_cast<const v4i*>(wbase + tc * 32 * LDW + ks * 32);
                acc[tc] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wv, av, (FIRST && ks == 0) ? zero : acc[tc], 0, 0, 0);
            }
        }
    };

    auto epilogue = [&](int t) {
        const int lane_c = 4 * (lane >> 5);
        constexpr int CH = BN / 16;                 // 16-byte chunks per row
        constexpr int NJ = 32 * CH / 64;
        // The Addition's other input: all of a tile's pieces are requested here, ahead of the requantization whose
        // arithmetic they then travel behind, from clamped addresses (so none sits in a divergent branch and waits there).
        const bool fuse = (a.N & 15) == 0 && a.res != nullptr;
        v4i other[NJ] = {};
        if (fuse)
        {
#pragma unroll
            for (int i = 0; i < NJ; ++i)
            {
                const int j = lane + 64 * i;
                const int row = min(t * 32 + j / CH, a.M - 1);
                const int c0 = min(n0 + (j % CH) * 16, a.N - 16);
                other[i] = *reinterpret_cast<const v4i*>(a.res + static_cast<long long>(row) * a.N + c0);
            }
        }
        int rt = 0;
        if constexpr (AW) rt = (rowsum + __shfl_xor(rowsum, 32)) * a.zw_neg;
#pragma unroll
        for (int tc = 0; tc < TC; ++tc)
        {
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const int cl = tc * 32 + 8 * q + lane_c;
                const float4 mp = *reinterpret_cast<const float4*>(cst + cl);
                const float4 bp = *reinterpret_cast<const float4*>(cst + BN + cl);
                const float4 mm = *reinterpret_cast<const float4*>(cst + 2 * BN + cl);
                const float4 bm = *reinterpret_cast<const float4*>(cst + 3 * BN + cl);
                const uint32_t out = Requant4Dev(acc[tc][4 * q + 0] + rt, acc[tc][4 * q + 1] + rt, acc[tc][4 * q + 2] + rt, acc[tc][4 * q + 3] + rt,
                                                 mp, bp, mm, bm, a.ct, a.corr, n0 + cl, a.rq);
                *reinterpret_cast<uint32_t*>(ostage + frag_row * LDO + cl) = out;
            }
        }
        // the wave reads back what its own lanes wrote: LDS operations of one wave complete in order; the fences keep
        // the compiler from moving the reads above the writes (different lanes, so no dependency it can see)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (fuse)
        {
#pragma unroll
            for (int i = 0; i < NJ; ++i)
            {
                const int j = lane + 64 * i;
                const int r = j / CH, cc = j % CH;
                const int row = t * 32 + r;
                const int c0 = n0 + cc * 16;
                if (row < a.M && c0 < a.N)
                    StoreOut16(outp, static_cast<long long>(row) * a.N + c0,
                               AddResidual16(*reinterpret_cast<const v4i*>(ostage + r * LDO + cc * 16), other[i], a.add));
            }
        }
        else if ((a.N & 15) == 0)
        {
#pragma unroll
            for (int j = lane; j < 32 * CH; j += 64)
            {
                const int r = j / CH, cc = j % CH;
                const int row = t * 32 + r;
                const int c0 = n0 + cc * 16;
                if (row < a.M && c0 < a.N)
                    StoreOut16(outp, static_cast<long long>(row) * a.N + c0, *reinterpret_cast<const v4i*>(ostage + r * LDO + cc * 16));
            }
        }
        else
        {
            for (int j = lane; j < 32 * BN; j += 64)
            {
                const int r = j / BN, c = j % BN;
                const int row = t * 32 + r;
                if (row < a.M && n0 + c < a.N) a.y[static_cast<long long>(row) * a.N + n0 + c] = ostage[r * LDO + c];
            }
        }
        // and the next tile's staging writes must stay behind these reads
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

    // ---- software pipeline over (tile, chunk): NB-1 chunks are in flight while one feeds the MFMAs --------------
    // The first activation loads are issued before the weight slab is fetched, so both latencies overlap.
    v4i buf[NB][KS];
    int t_cur = tile0, c_cur = 0;                // chunk being computed
    int t_nxt = tile0, c_nxt = 0;                // next chunk to load
    auto advance = [&](int& t, int& c) {
        if (++c == nch) { c = 0; t += tile_step; }
    };
#pragma unroll
    for (int j = 0; j < NB - 1; ++j)
    {
        if (t_nxt < n_tiles) { load_chunk(buf[j], t_nxt, c_nxt); advance(t_nxt, c_nxt); }
    }

    // ---- prologue: weight slab and epilogue constants into LDS (loads batched per column of chunks) ---------
    {
        const int chunks = a.K >> 4;
        const int8_t* src = a.w + static_cast<long long>(n0 + (tid >> 4)) * a.w_stride;
        for (int c = tid & 15; c < chunks; c += 16)
        {
            v4i t[BN / 16];
#pragma unroll
            for (int i = 0; i < BN / 16; ++i) t[i] = *reinterpret_cast<const v4i*>(src + static_cast<long long>(16 * i) * a.w_stride + c * 16);
#pragma unroll
            for (int i = 0; i < BN / 16; ++i) *reinterpret_cast<v4i*>(slab + ((tid >> 4) + 16 * i) * LDW + c * 16) = t[i];
        }
        for (int i = tid; i < 4 * BN; i += 256)
        {
            // the corr-folded bracket: m+, bc+, m-, bc-
            const int row = i / BN, c = i - row * BN;
            const int src_row = row == 0 ? 2 : row == 1 ? 6 : row == 2 ? 4 : 7;
            cst[i] = a.ct.p[src_row * a.ct.stride + n0 + c];
        }
    }
    __syncthreads();
    if (tile0 >= n_tiles) return;

    // One loop iteration = one chunk.  The buffer index is wave-uniform; dispatching on it keeps every register
    // index static while the epilogue appears only once in the code.
    static_assert(NB == 2 || NB == 4, "2 or 4 register chunks");
    int j = 0;
    while (t_cur < n_tiles)
    {
        const bool more = t_nxt < n_tiles;
        auto step = [&](auto jc) {
            constexpr int J = decltype(jc)::value;
            if (more) load_chunk(buf[(J + NB - 1) % NB], t_nxt, c_nxt);
            if (c_cur == 0) compute_chunk(buf[J], 0, std::true_type{});
            else compute_chunk(buf[J], c_cur, std::false_type{});
        };
        if (j == 0) step(std::integral_constant<int, 0>{});
        else if (j == 1) step(std::integral_constant<int, 1>{});
        else if constexpr (NB == 4)
        {
            if (j == 2) step(std::integral_constant<int, 2>{});
            else step(std::integral_constant<int, 3>{});
        }
        if (more) advance(t_nxt, c_nxt);
        j = (j + 1 == NB) ? 0 : j + 1;
        if (c_cur == nch - 1) epilogue(t_cur);
        advance(t_cur, c_cur);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// FullyConnected / pointwise layers with at most 4 GEMM rows (batch-1 inference): a matrix-vector product bound by
// streaming the weights once from HBM.  A wave owns 4 output channels at a time; its 64 lanes split K in 16-byte
// chunks (one coalesced 1 KB load per weight row and step), multiply with v_dot4 and reduce across the wave.
struct GemvArgs
{
    const uint8_t* x;        // [M][K]
    const int8_t*  w;        // [>= N rounded up to 4][w_stride], rows zero padded
    ChanTab        ct;
    const int32_t* corr;
    uint8_t*       y;        // [M][N]
    int M, K, N, w_stride;
    uint32_t xor_mask;
    int zw_neg;              // minus the zero point of the stored int8 weights; when not 0 every row's activations are summed
                             // as well and zw_neg times that sum joins the row's accumulators
    Requant rq;
};

template <int MR>
__global__ __launch_bounds__(256) void GemvKernel(GemvArgs a)
{
    constexpr int R = 4;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n0 = (static_cast<int>(blockIdx.x) * 4 + wave) * R;
    if (n0 >= a.N) return;
    const int xm = static_cast<int>(a.xor_mask);
    int acc[R][MR], xs[MR];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[r][m] = 0;
#pragma unroll
    for (int m = 0; m < MR; ++m) xs[m] = 0;
    const int chunks = a.K >> 4;
    const int8_t* wrow = a.w + static_cast<long long>(n0) * a.w_stride;
#pragma unroll 4
    for (int j = lane; j < chunks; j += 64)
    {
        v4i xv[MR];
#pragma unroll
        for (int m = 0; m < MR; ++m) xv[m] = *reinterpret_cast<const v4i*>(a.x + static_cast<long long>(m) * a.K + j * 16) ^ xm;
        if (a.zw_neg != 0)       // uniform
        {
#pragma unroll
            for (int m = 0; m < MR; ++m)
#pragma unroll
                for (int d = 0; d < 4; ++d) xs[m] = __builtin_amdgcn_sdot4(xv[m][d], 0x01010101, xs[m], false);
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
        {
            const v4i wv = *reinterpret_cast<const v4i*>(wrow + static_cast<long long>(r) * a.w_stride + j * 16);
#pragma unroll
            for (int m = 0; m < MR; ++m)
#pragma unroll
                for (int d = 0; d < 4; ++d) acc[r][m] = __builtin_amdgcn_sdot4(xv[m][d], wv[d], acc[r][m], false);
        }
    }
    if (a.zw_neg != 0)
    {
#pragma unroll
        for (int m = 0; m < MR; ++m)
        {
            xs[m] *= a.zw_neg;           // joins every channel's sum below, lane by lane
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r][m] += xs[m];
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m)
        {
            int v = acc[r][m];
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
            if (lane == 0 && n0 + r < a.N)
                a.y[static_cast<long long>(m) * a.N + n0 + r] = static_cast<uint8_t>(Requant1FoldedDev(v, a.ct, a.corr, n0 + r, a.rq));
        }
}

// ---------------------------------------------------------------------------------------------------------------
// A few dozen rows (the classifier of a network at its batch size): too many for the vector kernel above, too few to
// fill LDS-tiled blocks.  A block owns 32 rows x 32 channels; its four waves split K (wave w takes the 32-byte
// k-steps w, w+4, ...), each issues the loads of UN steps at once and feeds them to v_mfma_i32_32x32x32_i8, and the
// four partial tiles meet in LDS, where wave g requantizes accumulator group g.  K must be a multiple of 16.
// As a device function of a 256-thread block (tile at rows m0.., channels n0..; `part`: 4 x 16 x 64 ints of LDS, `rowpart`:
// 4 x 64; a barrier must separate two calls).  THROUGH: outputs are written through L2 as they are stored, for a caller
// that hands them to other blocks of the same launch (a.y + a.M * a.N below 4 GiB from a.y).
template <int UN, bool THROUGH>
__device__ __forceinline__ void SmallMGemmTile(const GemvArgs& a, int n0, int m0, int (*part)[16][64], int (*rowpart)[64])
{
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int frag_row = lane & 31;
    const int frag_k = (lane >> 5) * 16;
    const int xm = static_cast<int>(a.xor_mask);
    const int steps = (a.K + 31) >> 5;
    // rows past the end re-read the last row (never stored); a lane's 16 bytes past K re-read the row's last 16 bytes
    // against weights that are zero there: no load depends on a branch
    const uint8_t* xp = a.x + static_cast<long long>(min(m0 + frag_row, a.M - 1)) * a.K;
    const int8_t* wp = a.w + static_cast<long long>(n0 + frag_row) * a.w_stride + frag_k;
    v16i acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    int xs = 0;
    for (int s0 = wave; s0 < steps; s0 += 4 * UN)
    {
        v4i xv[UN], wv[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u)
        {
            const int s = min(s0 + 4 * u, steps - 1);
            xv[u] = *reinterpret_cast<const v4i*>(xp + min(s * 32 + frag_k, a.K - 16));
            wv[u] = *reinterpret_cast<const v4i*>(wp + s * 32);
        }
#pragma unroll
        for (int u = 0; u < UN; ++u)
        {
            const v4i zero = {0, 0, 0, 0};
            const v4i wu = (s0 + 4 * u < steps) ? wv[u] : zero;      // steps past the end (clamped above) add nothing
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wu, xv[u] ^ xm, acc, 0, 0, 0);
            // the row's sum counts a lane's 16 bytes only where they are bytes of the row that no other step covers
            if (a.zw_neg != 0 && s0 + 4 * u < steps && (s0 + 4 * u) * 32 + frag_k + 16 <= a.K)
            {
                const v4i xb = xv[u] ^ xm;
#pragma unroll
                for (int d = 0; d < 4; ++d) xs = __builtin_amdgcn_sdot4(xb[d], 0x01010101, xs, false);
            }
        }
    }
    rowpart[wave][lane] = xs;
#pragma unroll
    for (int i = 0; i < 16; ++i) part[wave][i][lane] = acc[i];
    __syncthreads();
    int v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        v[i] = part[0][4 * wave + i][lane] + part[1][4 * wave + i][lane] + part[2][4 * wave + i][lane] + part[3][4 * wave + i][lane];
    if (a.zw_neg != 0)
    {
        // the four waves split the k-steps and the two lanes of a row the halves of each step
        int total = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) total += rowpart[w][frag_row] + rowpart[w][frag_row + 32];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] += total * a.zw_neg;
    }
    // accumulator group g of the 32x32 tile: channels 8 g + 4 (lane / 32) + 0..3 of row lane % 32
    const int c = n0 + 8 * wave + 4 * (lane >> 5);
    const int row = m0 + frag_row;
    const float4 mp = *reinterpret_cast<const float4*>(a.ct.p + 2 * a.ct.stride + c);
    const float4 bp = *reinterpret_cast<const float4*>(a.ct.p + 6 * a.ct.stride + c);
    const float4 mm = *reinterpret_cast<const float4*>(a.ct.p + 4 * a.ct.stride + c);
    const float4 bm = *reinterpret_cast<const float4*>(a.ct.p + 7 * a.ct.stride + c);
    const uint32_t out = Requant4Dev(v[0], v[1], v[2], v[3], mp, bp, mm, bm, a.ct, a.corr, c, a.rq);
    if constexpr (THROUGH)
    {
        // Bytes written through one by one are slow, and rows of N bytes start anywhere: the tile meets in LDS (in `part`,
        // once every wave has read its sums) and leaves as the dwords of the output's own 4-byte grid, with single bytes
        // only where a dword is shared with a neighbouring tile or row.  a.y must be 4-byte aligned.
        __syncthreads();
        uint8_t* stage = reinterpret_cast<uint8_t*>(part);
        *reinterpret_cast<uint32_t*>(stage + frag_row * 32 + (c - n0)) = out;
        __syncthreads();
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.M * a.N, 0x00020000);
        const int r = threadIdx.x >> 3, seg = threadIdx.x & 7;
        if (m0 + r < a.M)
        {
            const int len = min(32, a.N - n0);
            const int first = (m0 + r) * a.N + n0;            // byte offset of the row's piece
#pragma unroll
            for (int e = 0; e < 2; ++e)
            {
                if (e == 1 && seg != 0) break;
                const int word = (first >> 2) + (e == 0 ? seg : 8);
                const int lo = word * 4 - first;               // position of the dword's first byte within the piece: -3 .. 32
                if (lo >= 0 && lo + 4 <= len)
                {
                    const uint8_t* sb = stage + r * 32 + lo;
                    const uint32_t v = static_cast<uint32_t>(sb[0]) | (static_cast<uint32_t>(sb[1]) << 8) | (static_cast<uint32_t>(sb[2]) << 16) |
                                       (static_cast<uint32_t>(sb[3]) << 24);
                    __builtin_amdgcn_raw_buffer_store_b32(v, rsrc, word * 4, 0, kStoreAuxSc1);
                }
                else
                {
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        if (lo + k >= 0 && lo + k < len) __builtin_amdgcn_raw_buffer_store_b8(stage[r * 32 + lo + k], rsrc, word * 4 + k, 0, kStoreAuxSc1);
                }
            }
        }
    }
    else if (row < a.M)
    {
        uint8_t* dst = a.y + static_cast<long long>(row) * a.N + c;
        if ((a.N & 3) == 0 && c + 3 < a.N) *reinterpret_cast<uint32_t*>(dst) = out;
        else
        {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (c + i < a.N) dst[i] = static_cast<uint8_t>(out >> (8 * i));
        }
    }
}

template <int UN>
__global__ __launch_bounds__(256) void SmallMGemmKernel(GemvArgs a)
{
    __shared__ int part[4][16][64];
    __shared__ int rowpart[4][64];
    SmallMGemmTile<UN, false>(a, static_cast<int>(blockIdx.x) * 32, static_cast<int>(blockIdx.y) * 32, part, rowpart);
}

} // namespace mi355x
