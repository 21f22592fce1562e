// Device kernels for quantized Convolution2d / DepthwiseConvolution2d / FullyConnected on gfx950.
//
//   ConvDirectKernel      one thread per output element; every configuration the library accepts.
//   DepthwiseC4Kernel     depthwise, multiplier 1, channels % 4 == 0: one thread per (pixel, 4 channels).
//   IgemmKernel<BM,BN,..> implicit GEMM on v_mfma_i32_32x32x32_i8, NHWC tiles staged in LDS, exact int32
//                         accumulation, fused requantize/clamp epilogue, output tile staged in LDS and stored
//                         with 16-byte coalesced writes.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "device_math.h"

namespace mi355x
{

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

struct ConvGeom
{
    int H, W, Ci, Ho, Wo, Co;
    int Kh, Kw;
    int pad_top, pad_left, stride_x, stride_y, dil_x, dil_y;
    int depth_mult;     // depthwise only
    int zx, zw;         // zero points of input and weights (in their own domain)
    int in_u8, w_u8;
};

// ---------------------------------------------------------------------------------------------------------
// Direct kernel.  Weights are laid out [Kh][Kw][Ci][Co] (conv) or [Kh][Kw][Co] (depthwise) so that
// neighbouring threads (neighbouring output channels) read neighbouring bytes.
// ---------------------------------------------------------------------------------------------------------
template <bool DEPTHWISE>
__global__ __launch_bounds__(256) void ConvDirectKernel(ConvGeom g, Requant rq, const uint8_t* __restrict__ x,
                                                        const uint8_t* __restrict__ w, ChanTab ct,
                                                        uint8_t* __restrict__ y, long long total)
{
    const long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    // one 64-bit division to split off the batch index, 32-bit arithmetic below it
    const unsigned per_image = static_cast<unsigned>(g.Ho) * g.Wo * g.Co;
    const long long n = idx / per_image;
    unsigned rem = static_cast<unsigned>(idx - n * per_image);
    const int co = static_cast<int>(rem % g.Co);
    rem /= g.Co;
    const int ox = static_cast<int>(rem % g.Wo);
    const int oy = static_cast<int>(rem / g.Wo);

    const uint8_t* xn = x + n * g.H * g.W * g.Ci;
    int acc = 0;
    for (int ky = 0; ky < g.Kh; ++ky)
    {
        const int iy = oy * g.stride_y + ky * g.dil_y - g.pad_top;
        if (iy < 0 || iy >= g.H) continue;
        for (int kx = 0; kx < g.Kw; ++kx)
        {
            const int ix = ox * g.stride_x + kx * g.dil_x - g.pad_left;
            if (ix < 0 || ix >= g.W) continue;
            const uint8_t* xp = xn + (static_cast<long long>(iy) * g.W + ix) * g.Ci;
            if (DEPTHWISE)
            {
                const int ci = co / g.depth_mult;
                const int xv = g.in_u8 ? static_cast<int>(xp[ci]) : static_cast<int>(static_cast<int8_t>(xp[ci]));
                const uint8_t wb = w[(ky * g.Kw + kx) * g.Co + co];
                const int wv = g.w_u8 ? static_cast<int>(wb) : static_cast<int>(static_cast<int8_t>(wb));
                acc += (xv - g.zx) * (wv - g.zw);
            }
            else
            {
                const uint8_t* wp = w + static_cast<long long>(ky * g.Kw + kx) * g.Ci * g.Co + co;
                for (int ci = 0; ci < g.Ci; ++ci)
                {
                    const int xv = g.in_u8 ? static_cast<int>(xp[ci]) : static_cast<int>(static_cast<int8_t>(xp[ci]));
                    const uint8_t wb = wp[static_cast<long long>(ci) * g.Co];
                    const int wv = g.w_u8 ? static_cast<int>(wb) : static_cast<int>(static_cast<int8_t>(wb));
                    acc += (xv - g.zx) * (wv - g.zw);
                }
            }
        }
    }
    y[idx] = static_cast<uint8_t>(Requant1Dev(acc, ct, co, rq));
}

// ---------------------------------------------------------------------------------------------------------
// Depthwise, multiplier 1, C % 4 == 0.  Weights stay in the reference layout [Kh][Kw][C].
// ---------------------------------------------------------------------------------------------------------
template <bool IN_U8, bool W_U8>
__device__ __forceinline__ void DwMac4(uint32_t xw, uint32_t ww, int zx, int zw, int acc[4])
{
#pragma unroll
    for (int b = 0; b < 4; ++b)
    {
        const int xv = IN_U8 ? static_cast<int>((xw >> (8 * b)) & 0xffu)
                             : static_cast<int>(static_cast<int8_t>((xw >> (8 * b)) & 0xffu));
        const int wv = W_U8 ? static_cast<int>((ww >> (8 * b)) & 0xffu)
                            : static_cast<int>(static_cast<int8_t>((ww >> (8 * b)) & 0xffu));
        acc[b] += (xv - zx) * (wv - zw);
    }
}

template <bool IN_U8, bool W_U8>
__global__ __launch_bounds__(256) void DepthwiseC4Kernel(ConvGeom g, Requant rq, const uint8_t* __restrict__ x,
                                                         const uint8_t* __restrict__ w, ChanTab ct,
                                                         uint8_t* __restrict__ y, long long total_c4)
{
    const long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total_c4) return;
    const unsigned C4 = static_cast<unsigned>(g.Co) >> 2;
    const unsigned per_image = static_cast<unsigned>(g.Ho) * g.Wo * C4;
    const long long n = idx / per_image;
    unsigned rem = static_cast<unsigned>(idx - n * per_image);
    const int c = static_cast<int>(rem % C4) * 4;
    rem /= C4;
    const int ox = static_cast<int>(rem % g.Wo);
    const int oy = static_cast<int>(rem / g.Wo);

    const uint8_t* xn = x + n * g.H * g.W * g.Ci + c;
    int acc[4] = {0, 0, 0, 0};
    for (int ky = 0; ky < g.Kh; ++ky)
    {
        const int iy = oy * g.stride_y + ky * g.dil_y - g.pad_top;
        if (iy < 0 || iy >= g.H) continue;
        for (int kx = 0; kx < g.Kw; ++kx)
        {
            const int ix = ox * g.stride_x + kx * g.dil_x - g.pad_left;
            if (ix < 0 || ix >= g.W) continue;
            const uint32_t xw = *reinterpret_cast<const uint32_t*>(xn + (static_cast<long long>(iy) * g.W + ix) * g.Ci);
            const uint32_t ww = *reinterpret_cast<const uint32_t*>(w + (ky * g.Kw + kx) * g.Co + c);
            DwMac4<IN_U8, W_U8>(xw, ww, g.zx, g.zw, acc);
        }
    }
    const Fast4 f4 = LoadFast4(ct, c);
    *reinterpret_cast<uint32_t*>(y + idx * 4) = Requant4Dev(acc[0], acc[1], acc[2], acc[3], f4, ct, c, rq);
}

// ---------------------------------------------------------------------------------------------------------
// Implicit GEMM on MFMA.
//
//   GEMM view: rows m = (n, oy, ox) output pixels, columns = output channels, K = (ky, kx, ci) with ci
//   fastest -- which is the memory order of both the NHWC input (per tap) and the [Co][Kh][Kw][Ci] weights, so
//   both operands are read in 16-byte pieces that are contiguous in K.  Requires Ci % 16 == 0.
//
//   Inputs are brought to signed int8 on the fly (uint8: x ^ 0x80, i.e. x - 128, zero point shifted likewise);
//   padding taps are filled with the (shifted) zero point, so acc = sum x'w - zx' * sum_k w, and the second
//   term is a per-channel constant that initialises the accumulators (`corr`).
//
//   Weights with a zero point (template AW): w' = w - zw' with the stored int8 w, so
//   sum (x' - zx')(w - zw') = sum x'w + corr[c] - zw' * S[m],  S[m] = sum_k x'[m][k] over the whole padded K row
//   (bytes outside the image are zx', which corr accounts for; those beyond K, zx' as well, are taken off again as the
//   constant `rowsum_bias`).  S[m] is summed with v_dot4 from the
//   activation fragments a lane reads for the MFMA anyway -- the two lanes that hold the halves of a pixel's k-slice
//   add up at the end -- and enters the accumulators just before they are requantized.
//
//   Block = 256 threads = 4 waves arranged WM x WN; each wave owns (BM/WM) x (BN/WN) outputs as 32x32 MFMA
//   tiles.  The MFMA "A" operand is the weight fragment (row = channel) and "B" the activation fragment
//   (column = pixel), so a lane ends up with 4 consecutive channels of one pixel per accumulator quad: the
//   epilogue packs them into one dword, stages the BM x BN byte tile in LDS, and the block writes it out
//   in 16-byte row-contiguous stores.
// ---------------------------------------------------------------------------------------------------------
struct IgemmArgs
{
    const uint8_t* x;
    const uint8_t* pad16;   // 16 bytes of (padding value ^ input xor): what a chunk outside the image loads
    const int8_t*  w;       // [Co_pad][K_pad], zero padded
    ChanTab        ct;      // per-channel requantization constants, rows of Co_pad floats
    const int32_t* corr;    // [Co_pad]
    uint8_t*       y;
    int M;                  // batch * Ho * Wo
    int H, W, Ci, Ho, Wo, Co;
    int Kh, Kw;
    int pad_top, pad_left, stride_x, stride_y, dil_x, dil_y;
    int K_pad;
    int unit;               // 1x1 kernel, stride 1, no padding: H = 1, W = M describe the input as one row of pixels
    int tiles_m, tiles_n;
    int xcd_cols = 1;       // direct-to-LDS kernel: XCD groups over the output channels (1: every XCD takes a range of row blocks over all
                            // column tiles and so reads every weight; 2: XCDs 0-3 take the lower half of the column tiles, 4-7 the
                            // upper half, each over a quarter of the row blocks: half the weights per XCD, every activation row twice)
    uint32_t xor_mask;      // 0x80808080 for uint8 input, else 0
    uint32_t pad_word;      // shifted input zero point replicated in 4 bytes
    int zw_neg;             // minus the zero point of the stored int8 weights (0: symmetric)
    int rowsum_bias;        // (K_pad - K) * zx': what the bytes beyond K add to a row sum
    Requant rq;
    const uint8_t* res = nullptr;   // direct-to-LDS kernel: the other input of an Addition fused into the write-out ([M][Co]), or null
    AddFuse add;
};

// K is walked in tiles of BK bytes per GEMM row.  BK = 128 makes every row chunk a whole 128-byte cache line: with 64-byte
// chunks half of each line fetched from L2 is thrown away, and the L2-to-CU path (not MFMA, not HBM) becomes the limit.
// LDS rows are BK + 16 bytes apart (80 or 144), which keeps the ds_read_b128 fragment reads free of bank conflicts.
template <int BM, int BN, int BK>
constexpr int IgemmSmemBytes()
{
    constexpr int stage = (BM + BN) * (BK + 16);
    constexpr int out = BM * (BN + 16);
    return 2 * stage > out ? 2 * stage : out;
}

// D = register slots for k-tiles on their way from global memory to LDS: the loads of tile kt + D - 1 are issued while
// tile kt is multiplied, so D - 1 tiles are in flight and an iteration no longer has to last a whole memory round trip.
// UT ("uniform tap"): Ci is a multiple of BK, so a k-tile never straddles two filter taps.  The walk over (ky, kx, ci) is
// then the same for every thread (scalar registers), and a thread's address is a fixed per-row pointer plus a scalar
// tap offset: no per-load multiplications.
template <int BM, int BN, int WM, int WN, int D, int BK, bool UT, bool AW = false>
__global__ __launch_bounds__(256) void IgemmKernel(IgemmArgs a)
{
    static_assert(WM * WN == 4, "4 waves per block");
    static_assert(D >= 2 && D <= 4, "2 to 4 register slots");
    static_assert(BM % 64 == 0 && BN % 64 == 0, "tile sizes are multiples of 64");
    static_assert(BK == 64 || BK == 128, "k-tiles of 64 or 128 bytes");
    constexpr int LDK = BK + 16;
    constexpr int CPR = BK / 16;                // 16-byte chunks per row of a k-tile
    constexpr int RP = 256 / CPR;               // rows covered by one pass of the block's threads
    constexpr int RA = BM / RP;                 // activation rows loaded per thread per k-tile
    constexpr int RB = BN / RP;                 // weight rows loaded per thread per k-tile
    constexpr int WTM = BM / WM;                // wave tile (pixels)
    constexpr int WTN = BN / WN;                // wave tile (channels)
    constexpr int TP = WTM / 32;                // 32-pixel sub-tiles per wave
    constexpr int TC = WTN / 32;                // 32-channel sub-tiles per wave
    constexpr int STAGE = (BM + BN) * LDK;
    constexpr int LDO = BN + 16;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];   // IgemmSmemBytes<BM, BN, BK>()

    // XCD-aware tile order: consecutive block ids land on different XCDs, so give each XCD a contiguous run
    // of tiles (tiles that share activation rows then share that XCD's L2).
    const int nblocks = a.tiles_m * a.tiles_n;
    const int per_xcd = (nblocks + 7) >> 3;
    const int tile = static_cast<int>(blockIdx.x & 7) * per_xcd + static_cast<int>(blockIdx.x >> 3);
    if (tile >= nblocks) return;
    const int tn = tile % a.tiles_n;
    const int tm = tile / a.tiles_n;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN;
    const int wn = wave % WN;

    // ---- global -> LDS load assignment: 16-byte chunk `lc` of row `lr (+64 j)` -------------------------
    const int lc = tid % CPR;
    const int lr = tid / CPR;

    const uint8_t* xrow[RA];
    int iy0[RA], ix0[RA];
    bool mvalid[RA];
#pragma unroll
    for (int j = 0; j < RA; ++j)
    {
        const int m = tm * BM + lr + RP * j;
        mvalid[j] = m < a.M;
        const int mm = mvalid[j] ? m : 0;
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
        xrow[j] = a.x + static_cast<long long>(n) * a.H * a.W * a.Ci;
        // UT: the chunk this thread would load for tap (0, 0), channel 0 (outside the tensor when the tap is padding;
        // such an address is never dereferenced)
        if constexpr (UT) xrow[j] += (static_cast<long long>(iy0[j]) * a.W + ix0[j]) * a.Ci + lc * 16;
    }
    // position of this thread's chunk inside K: (ky, kx, ci), advanced by BK every k-tile
    int ci, kx, ky;
    if constexpr (UT) { ci = 0; kx = 0; ky = 0; }       // of the k-tile: identical in every thread
    else
    {
        const int k0 = lc * 16;
        const int tap = k0 / a.Ci;
        ci = k0 - tap * a.Ci;
        ky = tap / a.Kw;
        kx = tap - ky * a.Kw;
    }
    const int8_t* wrow = a.w + static_cast<long long>(tn * BN + lr) * a.K_pad + lc * 16;

    v4i ra[D][RA], rb[D][RB];
    const int xm = static_cast<int>(a.xor_mask);

    auto load_tile = [&](int kt, auto slot) {
        constexpr int SL = decltype(slot)::value;
        const bool kvalid = ky < a.Kh;
        const int dy = ky * a.dil_y, dx = kx * a.dil_x;
        const long long tap_off = (static_cast<long long>(dy) * a.W + dx) * a.Ci + ci;      // UT: scalar
#pragma unroll
        for (int j = 0; j < RA; ++j)
        {
            const int iy = iy0[j] + dy;
            const int ix = ix0[j] + dx;
            const bool ok = mvalid[j] && kvalid && static_cast<unsigned>(iy) < static_cast<unsigned>(a.H) &&
                            static_cast<unsigned>(ix) < static_cast<unsigned>(a.W);
            // A chunk outside the image loads 16 prepared padding bytes instead: every load is unconditional and its
            // value is used as it is, so the compiler has no branch to put it in (a load inside a divergent branch is
            // waited for on the spot, which would serialise the prefetch).
            const uint8_t* in = UT ? xrow[j] + tap_off : xrow[j] + ((static_cast<long long>(iy) * a.W + ix) * a.Ci + ci);
            const uint8_t* src = ok ? in : a.pad16;
            ra[SL][j] = *reinterpret_cast<const v4i*>(src);   // the xor waits until the value goes to LDS
        }
#pragma unroll
        for (int j = 0; j < RB; ++j)
        {
            rb[SL][j] = *reinterpret_cast<const v4i*>(wrow + static_cast<long long>(RP * j) * a.K_pad + kt * BK);
        }
        // advance (ky, kx, ci) by one k-tile
        ci += BK;
        while (ci >= a.Ci)
        {
            ci -= a.Ci;
            if (++kx == a.Kw) { kx = 0; ++ky; }
        }
    };

    auto store_tile = [&](int buf, auto slot) {
        constexpr int SL = decltype(slot)::value;
        uint8_t* As = smem + buf * STAGE;
        uint8_t* Bs = As + BM * LDK;
#pragma unroll
        for (int j = 0; j < RA; ++j) *reinterpret_cast<v4i*>(As + (lr + RP * j) * LDK + lc * 16) = ra[SL][j] ^ xm;
#pragma unroll
        for (int j = 0; j < RB; ++j) *reinterpret_cast<v4i*>(Bs + (lr + RP * j) * LDK + lc * 16) = rb[SL][j];
    };

    // ---- accumulators, initialised with the zero-point correction -------------------------------------
    // lane owns pixel (lane & 31) of each pixel sub-tile and channels 8*(v/4) + 4*(lane/32) + v%4 of each
    // channel sub-tile.
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
    const int frag_k = (lane >> 5) * 16;
    using std::integral_constant;
    int rowsum[TP];
#pragma unroll
    for (int tp = 0; tp < TP; ++tp) rowsum[tp] = 0;

    auto compute = [&](int buf) {
        const uint8_t* As = smem + buf * STAGE;
        const uint8_t* Bs = As + BM * LDK;
#pragma unroll
        for (int ks = 0; ks < BK / 32; ++ks)
        {
            v4i fa[TP], fw[TC];
#pragma unroll
            for (int tp = 0; tp < TP; ++tp)
                fa[tp] = *reinterpret_cast<const v4i*>(As + (wm * WTM + tp * 32 + frag_row) * LDK + ks * 32 + frag_k);
#pragma unroll
            for (int tc = 0; tc < TC; ++tc)
                fw[tc] = *reinterpret_cast<const v4i*>(Bs + (wn * WTN + tc * 32 + frag_row) * LDK + ks * 32 + frag_k);
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
        }
    };

    // prologue: tiles 0 .. D-2 go on their way, tile 0 lands in LDS
    load_tile(0, integral_constant<int, 0>{});
    if constexpr (D > 2) { if (1 < nk) load_tile(1, integral_constant<int, 1>{}); }
    if constexpr (D > 3) { if (2 < nk) load_tile(2, integral_constant<int, 2>{}); }
    store_tile(0, integral_constant<int, 0>{});
    __syncthreads();

    // iteration kt (kt % D == J): issue tile kt+D-1 into the slot tile kt-1 left, multiply tile kt, move tile kt+1
    // from its slot to the other LDS buffer
    auto step = [&](int kt, auto jc) {
        constexpr int J = decltype(jc)::value;
        if (kt + D - 1 < nk) load_tile(kt + D - 1, integral_constant<int, (J + D - 1) % D>{});
        compute(kt & 1);
        if (kt + 1 < nk) store_tile((kt + 1) & 1, integral_constant<int, (J + 1) % D>{});
        __syncthreads();
    };
    for (int kt = 0; kt < nk; kt += D)
    {
        step(kt, integral_constant<int, 0>{});
        if (kt + 1 < nk) step(kt + 1, integral_constant<int, 1>{});
        if constexpr (D > 2) { if (kt + 2 < nk) step(kt + 2, integral_constant<int, 2>{}); }
        if constexpr (D > 3) { if (kt + 3 < nk) step(kt + 3, integral_constant<int, 3>{}); }
    }

    // ---- epilogue: requantize, pack 4 channels per dword, stage the byte tile in LDS ---------------------
    uint8_t* Os = smem;   // all reads of the stage buffers are behind the loop's final barrier
    if constexpr (AW)
    {
        // lanes l and l ^ 32 hold the two halves of every k-slice of pixel (l & 31)
#pragma unroll
        for (int tp = 0; tp < TP; ++tp) rowsum[tp] = (rowsum[tp] + __shfl_xor(rowsum[tp], 32) - a.rowsum_bias) * a.zw_neg;
    }
#pragma unroll
    for (int tc = 0; tc < TC; ++tc)
    {
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const int cl = wn * WTN + tc * 32 + 8 * q + lane_c;           // channel within the block tile
            const Fast4 f4 = LoadFast4(a.ct, tn * BN + cl);
#pragma unroll
            for (int tp = 0; tp < TP; ++tp)
            {
                const v16i& c = acc[tc][tp];
                const int rt = AW ? rowsum[tp] : 0;
                const uint32_t out = Requant4Dev(c[4 * q + 0] + rt, c[4 * q + 1] + rt, c[4 * q + 2] + rt, c[4 * q + 3] + rt, f4, a.ct, tn * BN + cl, a.rq);
                const int pl = wm * WTM + tp * 32 + (lane & 31);          // pixel within the block tile
                *reinterpret_cast<uint32_t*>(Os + pl * LDO + cl) = out;
            }
        }
    }
    __syncthreads();

    // ---- coalesced write-out ----------------------------------------------------------------------------
    constexpr int CHUNKS = BN / 16;             // 16-byte chunks per tile row
    constexpr int ROWS_PER_PASS = 256 / CHUNKS;
    const int oc = tid % CHUNKS;
    const int orow = tid / CHUNKS;
    const int c0 = tn * BN + oc * 16;
    const OutPtr outp = MakeOutPtr(a.y, static_cast<long long>(a.M) * a.Co);
    if ((a.Co & 15) == 0)
    {
        if (c0 < a.Co)
        {
#pragma unroll
            for (int r = orow; r < BM; r += ROWS_PER_PASS)
            {
                const int m = tm * BM + r;
                if (m < a.M)
                {
                    const v4i v = *reinterpret_cast<const v4i*>(Os + r * LDO + oc * 16);
                    StoreOut16(outp, static_cast<long long>(m) * a.Co + c0, v);
                }
            }
        }
    }
    else
    {
        // ragged channel count (e.g. 1001 classes): rows are not 16-byte aligned, store byte by byte
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
