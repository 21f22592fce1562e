// VALU kernels built on v_dot4_i32_i8 with LDS-staged halo tiles:
//
//   Depthwise3x3Kernel<S,R> DepthwiseConvolution2d 3x3, multiplier 1, stride S in {1,2}, channels % 16 == 0, R output rows per thread.
//                           (A block takes 32 channels; the last block of a tensor with 16 more stages padding for the missing
//                           half, computes on it and stores nothing for it.  The packed weights, corr and the channel table are
//                           padded to whole blocks.)
//   SmallCiConvKernel<..>   Convolution2d with <= 4 input channels (network stems): too little K per tap for MFMA.
//
// Both bring the input to signed int8 while staging (uint8: x ^ 0x80) and fill out-of-image positions with the
// shifted zero point, so that   sum (x - zx) w  =  sum x' w  -  zx' * sum_taps w ;   the second term is a
// per-channel constant (`corr`) that initialises the accumulators.  The depthwise kernel takes as "w" the difference
// d = w - zw between a weight and the weights' zero point; where some d does not fit int8 (it lies in -255 .. 254) it is
// the sum of two int8 halves, each in a packed array of its own (template W2), and costs a second v_dot4.  The stem
// kernels do the same, the MFMA variant with a second set of weight fragments and a second run of MFMAs over the same patches.
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
    const uint8_t*  pad16;    // 16 bytes of (padding value ^ input xor)
    const uint32_t* wpack;    // [C][4] dwords; dword r (r < 3) = bytes { w[r][0][c], w[r][1][c], w[r][2][c], 0 }
    const uint32_t* wpack2;   // W2: the second halves, same layout
    ChanTab         ct;
    const int32_t*  corr;     // [C]  -zx' * sum of the 9 taps
    uint8_t*        y;
    int N, H, W, C, Ho, Wo;
    int pad_top, pad_left;
    int tiles_x, tiles_y, cblocks;
    int total_blocks, xcd_chunk;   // work items, and ceil(work items / 8): the grid is 8 * xcd_chunk blocks
    uint32_t xor_mask, pad_word;
    uint32_t rcp_cblocks, rcp_tiles_x, rcp_tiles_y;   // matrix-core kernel: ceil(2^32 / d) of the three divisors (unused where d = 1)
    Requant rq;
};

// Consecutive block ids are dealt round-robin to the 8 XCDs, each with its own L2.  Giving XCD x the contiguous range
// [x * chunk, (x + 1) * chunk) of work items makes blocks that run together on one XCD neighbours in the work order,
// so the channel blocks of one pixel tile -- which read different 32-byte parts of the same cache lines -- share an L2.
__device__ __forceinline__ int XcdContiguousWorkItem(int block, int chunk)
{
    return (block & 7) * chunk + (block >> 3);
}

// Block: 8 R output rows x (4 groups of P pixels) x 32 channels; thread = (4 channels, P pixels of R consecutive rows).
// A thread reads 6 consecutive input pixels per input row (one dword = 4 channels each), transposes them with
// v_perm_b32 into per-channel dwords of 4 consecutive pixels, and each such dword feeds
//   stride 1: two outputs  (weights {w0,w1,w2,0} and {0,w0,w1,w2})
//   stride 2: one output   (weights {w0,w1,w2,0})
// through one v_dot4 per channel and output row that the input row belongs to.  With R = 2 the rows two outputs share
// are read and transposed once, and the per-thread set-up (staging, constants, addresses) is spread over twice the
// outputs; R = 1 keeps more blocks in flight for small feature maps.
//
// CB = 64 (channel counts that are odd multiples of 64): 64 channels of a tile of 4 R rows x 4 P pixels, 16 lanes per
// pixel; with 64 channels in all a tile row is then one contiguous run of memory.
// CB = 128 (channel counts that are multiples of 128): a block takes 128 channels of a tile of 4 R rows x 2 P pixels, 32
// lanes per pixel.  Every pixel it loads or stores is then one whole 128-byte line instead of a quarter of one; the
// smaller tile costs more halo (1.56 x instead of 1.27 x at stride 1).  The stores are ordinary ones: dwords written
// through L2 one by one (buffer stores with sc1) made a MobileNetV1 step 1.2 % slower.
template <int S, int R, int CB>
struct Dw3x3Tile
{
    static constexpr int LPC = CB / 4;                  // lanes per pixel
    static constexpr int XG = CB == 128 ? 2 : 4;        // thread columns
    static constexpr int TH = (256 / (LPC * XG)) * R;   // 8 R (CB = 32) or 4 R output rows per tile
    static constexpr int P = S == 1 ? 4 : 2;            // outputs per thread and row
    static constexpr int TW = P * XG;                   // outputs per tile row
    static constexpr int HR = TH * S + 2;               // halo rows held in LDS
    static constexpr int HC = TW * S + 2;               // halo columns
    // bytes per pixel in LDS.  CB = 32: 48 spreads the dword reads of a wave's eight pixels over the banks; CB = 64: 80 does
    // the same for the four pixels (P S pixels apart) a wave reads; CB = 128: the 32 lanes of a pixel read 128 contiguous bytes
    static constexpr int PITCH = CB == 32 ? 48 : CB == 64 ? 80 : 128;
    static constexpr int SMEM = HR * HC * PITCH;
};

// The work of one block (256 threads) on work item `b` (channel block fastest, then tile column, tile row, image); `tile`
// is the block's Dw3x3Tile<S, R, CB>::SMEM bytes of LDS.  THROUGH: the output dwords are written through L2 as they are
// issued (buffer stores with sc1; tensors below 4 GiB), for callers that hand the output to other blocks of the same launch.
struct NoBlockHook
{
    __device__ __forceinline__ void operator()() const {}
};

// `after_loads()` is called by every thread once the block's last global load has been issued (before its stores).
template <int S, int R, bool W2, int CB, bool THROUGH, typename Hook = NoBlockHook>
__device__ __forceinline__ void Depthwise3x3Block(const Dw3x3Args& a, int b, uint8_t* const tile, Hook after_loads = Hook())
{
    static_assert(CB == 32 || CB == 64 || CB == 128, "32, 64 or 128 channels per block");
    using G = Dw3x3Tile<S, R, CB>;
    constexpr int LPC = G::LPC, XG = G::XG, TH = G::TH, P = G::P, TW = G::TW, HR = G::HR, HC = G::HC, PITCH = G::PITCH;
    constexpr int CPP = CB / 16;                 // 16-byte staging chunks per pixel
    constexpr int IR = (R - 1) * S + 3;          // input rows a thread walks

    const int cb = b % a.cblocks; b /= a.cblocks;
    const int tx = b % a.tiles_x; b /= a.tiles_x;
    const int ty = b % a.tiles_y;
    const int n = b / a.tiles_y;
    const int tid = threadIdx.x;

    // ---- stage the halo tile: 16-byte chunks, two per pixel ------------------------------------------------
    const int iy_org = ty * TH * S - a.pad_top;
    const int ix_org = tx * TW * S - a.pad_left;
    const uint8_t* xn = a.x + static_cast<long long>(n) * a.H * a.W * a.C + cb * CB;
    const int xm = static_cast<int>(a.xor_mask);
    // all of a thread's staging loads are issued before the first is used; a chunk outside the image reads 16 prepared
    // bytes that become the padding value under the xor, so no load sits in a divergent branch
    constexpr int NST = (HR * HC * CPP + 255) / 256;
    v4i st[NST];
#pragma unroll
    for (int k = 0; k < NST; ++k)
    {
        const int i = min(tid + k * 256, HR * HC * CPP - 1);
        const int part = i % CPP;
        const int pix = i / CPP;
        const int col = pix % HC;
        const int row = pix / HC;
        const int iy = iy_org + row, ix = ix_org + col;
        const bool ok = static_cast<unsigned>(iy) < static_cast<unsigned>(a.H) && static_cast<unsigned>(ix) < static_cast<unsigned>(a.W) &&
                        cb * CB + part * 16 < a.C;
        const uint8_t* src = ok ? xn + (static_cast<long long>(iy) * a.W + ix) * a.C + part * 16 : a.pad16;
        st[k] = *reinterpret_cast<const v4i*>(src);
    }
#pragma unroll
    for (int k = 0; k < NST; ++k)
    {
        const int i = tid + k * 256;
        if (i < HR * HC * CPP) *reinterpret_cast<v4i*>(tile + (i / CPP) * PITCH + (i % CPP) * 16) = st[k] ^ xm;
    }

    // ---- per-thread constants ---------------------------------------------------------------------------------
    const int c4 = tid % LPC;
    const int xg = (tid / LPC) % XG;
    const int row = (tid / (LPC * XG)) * R;      // first of this thread's output rows within the tile
    const int c = cb * CB + c4 * 4;
    uint32_t wA[3][4], wB[3][4];
#pragma unroll
    for (int ch = 0; ch < 4; ++ch)
    {
        const uint4 w4 = *reinterpret_cast<const uint4*>(a.wpack + (c + ch) * 4);
        wA[0][ch] = w4.x; wA[1][ch] = w4.y; wA[2][ch] = w4.z;
        if constexpr (W2)
        {
            const uint4 v4 = *reinterpret_cast<const uint4*>(a.wpack2 + (c + ch) * 4);
            wB[0][ch] = v4.x; wB[1][ch] = v4.y; wB[2][ch] = v4.z;
        }
        else
        {
            wB[0][ch] = wB[1][ch] = wB[2][ch] = 0u;
        }
    }
    const v4i corr4 = *reinterpret_cast<const v4i*>(a.corr + c);
    int acc[R][P][4];
#pragma unroll
    for (int o = 0; o < R; ++o)
#pragma unroll
        for (int j = 0; j < P; ++j)
#pragma unroll
            for (int ch = 0; ch < 4; ++ch) acc[o][j][ch] = corr4[ch];

    __syncthreads();

#pragma unroll
    for (int ir = 0; ir < IR; ++ir)
    {
        const uint8_t* base = tile + ((row * S + ir) * HC + xg * P * S) * PITCH + c4 * 4;
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
            // input row ir is filter row r = ir - o * S of output row o
#pragma unroll
            for (int o = 0; o < R; ++o)
            {
                const int r = ir - o * S;
                if (r < 0 || r > 2) continue;
#pragma unroll
                for (int ch = 0; ch < 4; ++ch)
                {
                    if (S == 1)
                    {
                        acc[o][2 * g][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), static_cast<int>(wA[r][ch]), acc[o][2 * g][ch], false);
                        acc[o][2 * g + 1][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), static_cast<int>(wA[r][ch] << 8), acc[o][2 * g + 1][ch], false);
                        if constexpr (W2)
                        {
                            acc[o][2 * g][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), static_cast<int>(wB[r][ch]), acc[o][2 * g][ch], false);
                            acc[o][2 * g + 1][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), static_cast<int>(wB[r][ch] << 8), acc[o][2 * g + 1][ch], false);
                        }
                    }
                    else
                    {
                        acc[o][g][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), static_cast<int>(wA[r][ch]), acc[o][g][ch], false);
                        if constexpr (W2) acc[o][g][ch] = __builtin_amdgcn_sdot4(static_cast<int>(chv[ch]), static_cast<int>(wB[r][ch]), acc[o][g][ch], false);
                    }
                }
            }
        }
    }

    // ---- epilogue ------------------------------------------------------------------------------------------------
    const Fast4 f4 = LoadFast4(a.ct, c);
    after_loads();
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t yrsrc = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, -1, 0x00020000);
#pragma unroll
    for (int o = 0; o < R; ++o)
    {
        const int oy = ty * TH + row + o;
        if (oy >= a.Ho) break;
        uint8_t* yrow = a.y + (static_cast<long long>(n) * a.Ho + oy) * a.Wo * a.C + c;
#pragma unroll
        for (int j = 0; j < P; ++j)
        {
            const int ox = tx * TW + xg * P + j;
            if (ox < a.Wo && c < a.C)
            {
                const uint32_t q = Requant4Dev(acc[o][j][0], acc[o][j][1], acc[o][j][2], acc[o][j][3], f4, a.ct, c, a.rq);
                if constexpr (THROUGH)
                    __builtin_amdgcn_raw_buffer_store_b32(q, yrsrc, static_cast<int>(yrow - a.y) + ox * a.C, 0, kStoreAuxSc1);
                else
                    // an ordinary store: the pieces of a line are merged in L2 (written through one by one they are slower)
                    *reinterpret_cast<uint32_t*>(yrow + static_cast<long long>(ox) * a.C) = q;
            }
        }
    }
}

template <int S, int R, bool W2 = false, int CB = 32>
__global__ __launch_bounds__(256) void Depthwise3x3Kernel(Dw3x3Args a)
{
    __shared__ __attribute__((aligned(16))) uint8_t tile[Dw3x3Tile<S, R, CB>::SMEM];
    const int b = XcdContiguousWorkItem(blockIdx.x, a.xcd_chunk);
    if ((static_cast<int>(blockIdx.x) >> 3) >= a.xcd_chunk || b >= a.total_blocks) return;
    Depthwise3x3Block<S, R, W2, CB, false>(a, b, tile);
}

// ---------------------------------------------------------------------------------------------------------------
// Constant address space: a wave-uniform load through such a pointer is a scalar load, whatever stores the kernel
// makes elsewhere.  Only memory that no kernel writes while this one runs (plan constants) may be read this way.
#define MI355X_CONST_AS __attribute__((address_space(4)))

template <typename T>
__device__ __forceinline__ const T MI355X_CONST_AS* AsConstant(const T* p)
{
    return (const T MI355X_CONST_AS*)p;
}

struct SmallCiArgs
{
    const uint8_t*  x;
    const uint32_t* wpack;    // [Co][KH][RD] dwords: row r of filter co as consecutive (kx, ci) bytes, zero padded
    const uint32_t* wpack2;   // W2: the second halves, same layout
    ChanTab         ct;       // rows 2, 5, 6 on the fast path (accumulators start at zero), rows 0, 1 on the exact path
    const int32_t*  corr;     // [Co]
    uint8_t*        y;
    int N, H, W, Ci, Ho, Wo, Co;
    int Kw, stride, pad_top, pad_left;
    int tiles_x, tiles_y;
    int lp;                   // LDS row pitch in bytes (multiple of 4)
    uint32_t ndw_recip;       // ceil(2^32 / (lp / 4))
    uint32_t xor_mask, pad_byte;
    int vec16;                // output rows allow 16-byte stores (y 16-byte aligned, Co % 16 == 0)
    const uint8_t* pad16;     // 16 bytes of (padding value ^ input xor)
    int vec_stage;            // every halo row starts 16-byte aligned and image rows are whole 16-byte chunks: stage with
                              // 16-byte loads (lp is then a multiple of 16)
    uint32_t nch_recip;       // ceil(2^32 / (lp / 16))
    const int8_t* w_mfma;     // MFMA variant: [Co rounded up to 32][kp] bytes, a filter's rows as RD dwords each, zero padded
    const int8_t* w_mfma2;    // W2: the second halves, same layout
    int kp;                   // bytes per weight row of w_mfma (multiple of 32)
    Requant rq;
};

// Block: 32 x 16 output pixels; thread = two horizontally adjacent pixels, all output channels.
//   Staging: each halo row is copied as ALIGNED dwords (rows start at arbitrary byte addresses when Ci is 3, so the
//   LDS row keeps the global misalignment and readers add it back); only dwords that straddle an image edge are
//   assembled byte by byte, and positions outside the image hold the shifted zero point.
//   Compute: a thread reads its KH rows of Kw*Ci contiguous bytes as aligned dwords + v_alignbyte, then walks the
//   output channels; weights and requantization constants are wave-uniform scalar loads, so a v_dot4 takes its
//   weight operand from an SGPR.  16 channels of a pixel leave as one 16-byte store.
// Geometry of the small-Ci kernels' block tile: 32 x 16 output pixels and its input halo in LDS.
template <int KH, int TH_ = 16>
struct SmallCiTile
{
    static constexpr int TW = 32, TH = TH_;
    static constexpr int HRMAX = (TH - 1) * 2 + KH;
    static constexpr int LPMAX = 288;                        // >= 3 + (TW-1)*2*4 + 4*6 rounded up, + 8
    static constexpr int DWORDS = HRMAX * LPMAX / 4;
};

// Copies the halo of output tile (tx, ty) of image n into `tile` (LDS row pitch a.lp bytes).
//   Each halo row is copied as ALIGNED dwords (rows start at arbitrary byte addresses when Ci is 3, so the LDS row keeps
//   the global misalignment and readers add it back: row r starts at byte (A_r & 3) of its LDS row, A_r being the row's
//   byte offset from the aligned image base); only dwords that straddle an image edge are assembled byte by byte, and
//   positions outside the image hold the shifted zero point.  Returns through the references what readers need.
template <int KH, int TH_ = 16>
__device__ __forceinline__ void StageSmallCiHalo(const SmallCiArgs& a, uint32_t* tile, int tx, int ty, int n, int tid,
                                                 int& iy_org, int& ix_org, int& mis)
{
    constexpr int TW = SmallCiTile<KH, TH_>::TW, TH = SmallCiTile<KH, TH_>::TH;
    constexpr int HRMAX = SmallCiTile<KH, TH_>::HRMAX, LPMAX = SmallCiTile<KH, TH_>::LPMAX;
    const int S = a.stride;
    const int HR = (TH - 1) * S + KH;
    const int NDW = a.lp >> 2;
    iy_org = ty * TH * S - a.pad_top;
    ix_org = tx * TW * S - a.pad_left;
    const uint8_t* xn = a.x + static_cast<long long>(n) * a.H * a.W * a.Ci;
    mis = static_cast<int>(reinterpret_cast<uintptr_t>(xn) & 3);
    const uint8_t* xal = xn - mis;                           // 4-byte aligned
    const uint32_t xm = a.xor_mask & 0xffu;
    const uint32_t xm4 = xm * 0x01010101u;
    const uint32_t pad4 = (a.pad_byte & 0xffu) * 0x01010101u;
    if (a.vec_stage)          // block-uniform
    {
        // Aligned geometry: a 16-byte chunk lies wholly inside the image or wholly outside it; a chunk outside loads 16
        // prepared bytes that become the padding value under the xor, so every load is unconditional and in flight at once.
        constexpr int MAXV = (HRMAX * (LPMAX / 16) + 255) / 256;
        const int nch = a.lp >> 4;
        const int total = HR * nch;
        const int row_bytes = a.W * a.Ci;
        const int col0 = ix_org * a.Ci;
        v4i sv[MAXV];
#pragma unroll
        for (int k = 0; k < MAXV; ++k)
        {
            const int i = min(tid + k * 256, total - 1);
            const int row = static_cast<int>(__umulhi(static_cast<uint32_t>(i), a.nch_recip));
            const int c = i - row * nch;
            const int iy = iy_org + row;
            const bool ok = static_cast<unsigned>(iy) < static_cast<unsigned>(a.H) && col0 + 16 * c + 16 <= row_bytes;
            const uint8_t* src = ok ? xn + static_cast<long long>(iy) * row_bytes + col0 + 16 * c : a.pad16;
            sv[k] = *reinterpret_cast<const v4i*>(src);
        }
#pragma unroll
        for (int k = 0; k < MAXV; ++k)
        {
            const int i = tid + k * 256;
            if (i < total) *reinterpret_cast<v4i*>(tile + i * 4) = sv[k] ^ static_cast<int>(xm4);
        }
        return;
    }
    // columns of the halo that lie inside the image, as byte offsets from the halo's first column
    const int vb0 = max(0, -ix_org) * a.Ci;
    const int vb1 = min((TW - 1) * S + a.Kw, a.W - ix_org) * a.Ci;
    // Two passes so that all of a thread's global loads are in flight together: pass 1 issues the aligned dword
    // loads, pass 2 assembles the few dwords that straddle an image edge and writes everything to LDS.
    constexpr int MAXIT = (HRMAX * (LPMAX / 4) + 255) / 256;
    const int total = HR * NDW;
    const int nit = (total + 255) >> 8;                      // passes this tile really needs (block-uniform)
    uint32_t sv[MAXIT];
    int slo[MAXIT];                                          // dword offset from xal; bit 0: straddles an image edge
    // loads are unconditional (a dword that is not wholly inside the image reads a harmless in-tensor address and
    // is discarded), so that none of them waits for another
    const long long safe = reinterpret_cast<const uint8_t*>((reinterpret_cast<uintptr_t>(a.x) + 3) & ~static_cast<uintptr_t>(3)) - xal;
#pragma unroll
    for (int k = 0; k < MAXIT; ++k)
    {
        if (k < nit)
        {
            const int i = min(tid + k * 256, total - 1);
            const int row = static_cast<int>(__umulhi(static_cast<uint32_t>(i), a.ndw_recip));
            const int j = i - row * NDW;
            const int iy = iy_org + row;
            const int A = (iy * a.W + ix_org) * a.Ci + mis;  // halo row start as a byte offset from xal (may be < 0)
            const int lo = (A & ~3) + 4 * j;
            const int vbeg = A + vb0, vend = A + vb1;
            const bool row_ok = static_cast<unsigned>(iy) < static_cast<unsigned>(a.H);
            const bool inside = row_ok && lo >= vbeg && lo + 4 <= vend;
            const bool edge = row_ok && !inside && lo + 4 > vbeg && lo < vend;
            const uint32_t ld = *reinterpret_cast<const uint32_t*>(xal + (inside ? static_cast<long long>(lo) : safe));
            sv[k] = inside ? (ld ^ xm4) : pad4;
            slo[k] = lo | (edge ? 1 : 0);
        }
    }
#pragma unroll
    for (int k = 0; k < MAXIT; ++k)
    {
        const int i = tid + k * 256;
        if (k < nit && i < total)
        {
            uint32_t v = sv[k];
            if (slo[k] & 1)
            {
                // rare: rebuild the dword byte by byte against this row's valid range
                const int lo = slo[k] & ~3;
                const int row = static_cast<int>(__umulhi(static_cast<uint32_t>(i), a.ndw_recip));
                const int A = ((iy_org + row) * a.W + ix_org) * a.Ci + mis;
                const int vbeg = A + vb0, vend = A + vb1;
                v = 0;
#pragma unroll
                for (int q = 0; q < 4; ++q)
                {
                    const int o = lo + q;
                    uint32_t byte = a.pad_byte & 0xffu;
                    if (o >= vbeg && o < vend) byte = static_cast<uint32_t>(xal[o]) ^ xm;
                    v |= byte << (8 * q);
                }
            }
            tile[i] = v;
        }
    }
}

template <int KH, int RD, bool W2 = false>
__global__ __launch_bounds__(256) void SmallCiConvKernel(SmallCiArgs a)
{
    constexpr int P = 2, TW = 16 * P, TH = 16;
    __shared__ __attribute__((aligned(16))) uint32_t tile[SmallCiTile<KH>::DWORDS];

    int b = blockIdx.x;
    const int tx = b % a.tiles_x; b /= a.tiles_x;
    const int ty = b % a.tiles_y;
    const int n = b / a.tiles_y;
    const int tid = threadIdx.x;
    const int S = a.stride;
    int iy_org, ix_org, mis;
    StageSmallCiHalo<KH>(a, tile, tx, ty, n, tid, iy_org, ix_org, mis);
    __syncthreads();

    const int lx = tid & 15, ly = tid >> 4;
    uint32_t xr[P][KH][RD];
#pragma unroll
    for (int r = 0; r < KH; ++r)
    {
        const int row = ly * S + r;
        const int sh_row = ((((iy_org + row) * a.W + ix_org) * a.Ci + mis) & 3);
#pragma unroll
        for (int p = 0; p < P; ++p)
        {
            const int off = row * a.lp + sh_row + (lx * P + p) * S * a.Ci;
            const uint32_t* q = tile + (off >> 2);
            const int sh = off & 3;
            uint32_t d[RD + 1];
#pragma unroll
            for (int i = 0; i <= RD; ++i) d[i] = q[i];
#pragma unroll
            for (int i = 0; i < RD; ++i) xr[p][r][i] = __builtin_amdgcn_alignbyte(d[i + 1], d[i], sh);
        }
    }

    const int oy = ty * TH + ly, ox0 = tx * TW + lx * P;
    if (oy >= a.Ho || ox0 >= a.Wo) return;
    const bool second = ox0 + 1 < a.Wo;
    uint8_t* yp = a.y + ((static_cast<long long>(n) * a.Ho + oy) * a.Wo + ox0) * a.Co;
    const uint32_t MI355X_CONST_AS* wc = AsConstant(a.wpack);
    const uint32_t MI355X_CONST_AS* wc2 = AsConstant(W2 ? a.wpack2 : a.wpack);
    const float MI355X_CONST_AS* tab = AsConstant(a.ct.p);
    const int ts = a.ct.stride;
    for (int co = 0; co < a.Co; co += 16)
    {
        const int groups = min(4, (a.Co - co) >> 2);
        uint32_t o[P][4];
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4)
        {
            if (g4 >= groups) continue;
            const int c = co + 4 * g4;
            int acc[P][4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                const uint32_t MI355X_CONST_AS* w = wc + (c + u) * (KH * RD);
#pragma unroll
                for (int p = 0; p < P; ++p) acc[p][u] = 0;
#pragma unroll
                for (int r = 0; r < KH; ++r)
#pragma unroll
                    for (int i = 0; i < RD; ++i)
                    {
                        const int wv = static_cast<int>(w[r * RD + i]);
#pragma unroll
                        for (int p = 0; p < P; ++p) acc[p][u] = __builtin_amdgcn_sdot4(static_cast<int>(xr[p][r][i]), wv, acc[p][u], false);
                        if constexpr (W2)
                        {
                            const int wv2 = static_cast<int>(wc2[(c + u) * (KH * RD) + r * RD + i]);
#pragma unroll
                            for (int p = 0; p < P; ++p) acc[p][u] = __builtin_amdgcn_sdot4(static_cast<int>(xr[p][r][i]), wv2, acc[p][u], false);
                        }
                    }
            }
            const float4 mp = {tab[2 * ts + c], tab[2 * ts + c + 1], tab[2 * ts + c + 2], tab[2 * ts + c + 3]};
            const float4 bp = {tab[6 * ts + c], tab[6 * ts + c + 1], tab[6 * ts + c + 2], tab[6 * ts + c + 3]};
            const float4 mm = {tab[4 * ts + c], tab[4 * ts + c + 1], tab[4 * ts + c + 2], tab[4 * ts + c + 3]};
            const float4 bm = {tab[7 * ts + c], tab[7 * ts + c + 1], tab[7 * ts + c + 2], tab[7 * ts + c + 3]};
#pragma unroll
            for (int p = 0; p < P; ++p)
                o[p][g4] = Requant4Dev(acc[p][0], acc[p][1], acc[p][2], acc[p][3], mp, bp, mm, bm, a.ct, a.corr, c, a.rq);
        }
        if (groups == 4 && a.vec16)
        {
            *reinterpret_cast<uint4*>(yp + co) = uint4{o[0][0], o[0][1], o[0][2], o[0][3]};
            if (second) *reinterpret_cast<uint4*>(yp + a.Co + co) = uint4{o[1][0], o[1][1], o[1][2], o[1][3]};
        }
        else
        {
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4)
            {
                if (g4 >= groups) continue;
                *reinterpret_cast<uint32_t*>(yp + co + 4 * g4) = o[0][g4];
                if (second) *reinterpret_cast<uint32_t*>(yp + a.Co + co + 4 * g4) = o[1][g4];
            }
        }
    }
}

// The same layers on the matrix cores.  A filter row of Kw*Ci bytes, padded to RD dwords, is how the dot4 kernel already
// holds a pixel's inputs in registers; laid end to end, the KH rows are a K vector of KH*RD*4 bytes (zero weights under
// the padding), and 32 pixels x 32 output channels become ceil(KH*RD/8) MFMA steps instead of 32*KH*RD dot products per
// pixel.  Both lanes of a pixel (lane, lane + 32) gather the pixel's rows from the LDS halo and keep the half of each
// 32-byte k-step that the MFMA B operand assigns them.  A wave takes 4 of the tile's 16 rows; NT = output channels / 32.
template <int KH, int RD, int NT, int TH, bool W2 = false>
__global__ __launch_bounds__(256) void SmallCiMfmaKernel(SmallCiArgs a)
{
    constexpr int TW = 32;
    constexpr int RPW = TH / 4;                   // tile rows per wave
    constexpr int NDWP = KH * RD;                 // patch dwords per pixel
    constexpr int KST = (NDWP + 7) / 8;           // MFMA k-steps of 32 bytes
    __shared__ __attribute__((aligned(16))) uint32_t tile[SmallCiTile<KH, TH>::DWORDS];
    __shared__ __attribute__((aligned(16))) float cst[4][NT * 32];      // the corr-folded bracket: m+, bc+, m-, bc-

    int b = blockIdx.x;
    const int tx = b % a.tiles_x; b /= a.tiles_x;
    const int ty = b % a.tiles_y;
    const int n = b / a.tiles_y;
    const int tid = threadIdx.x;
    const int S = a.stride;
    int iy_org, ix_org, mis;
    StageSmallCiHalo<KH, TH>(a, tile, tx, ty, n, tid, iy_org, ix_org, mis);
    for (int i = tid; i < 4 * NT * 32; i += 256)
    {
        const int row = i / (NT * 32), c = i - row * (NT * 32);
        cst[row][c] = a.ct.p[(row == 0 ? 2 : row == 1 ? 6 : row == 2 ? 4 : 7) * a.ct.stride + c];
    }

    const int lane = tid & 63, wave = tid >> 6;
    const int px = lane & 31, half = lane >> 5;
    // weight fragments of every channel tile and k-step stay in registers
    v4i wfrag[NT][KST];
#pragma unroll
    for (int ct = 0; ct < NT; ++ct)
#pragma unroll
        for (int t = 0; t < KST; ++t)
            wfrag[ct][t] = *reinterpret_cast<const v4i*>(a.w_mfma + static_cast<long long>(ct * 32 + px) * a.kp + t * 32 + half * 16);
    v4i wfrag2[W2 ? NT : 1][W2 ? KST : 1];
    if constexpr (W2)
    {
#pragma unroll
        for (int ct = 0; ct < NT; ++ct)
#pragma unroll
            for (int t = 0; t < KST; ++t)
                wfrag2[ct][t] = *reinterpret_cast<const v4i*>(a.w_mfma2 + static_cast<long long>(ct * 32 + px) * a.kp + t * 32 + half * 16);
    }
    __syncthreads();

    const int ox = tx * TW + px;
#pragma unroll 1
    for (int rr = 0; rr < RPW; ++rr)
    {
        const int ly = wave * RPW + rr;
        const int oy = ty * TH + ly;
        if (oy >= a.Ho) break;                    // wave-uniform
        uint32_t flat[KST * 8];
#pragma unroll
        for (int i = NDWP; i < KST * 8; ++i) flat[i] = 0u;
#pragma unroll
        for (int r = 0; r < KH; ++r)
        {
            const int row = ly * S + r;
            const int sh_row = ((((iy_org + row) * a.W + ix_org) * a.Ci + mis) & 3);
            const int off = row * a.lp + sh_row + px * S * a.Ci;
            const uint32_t* q = tile + (off >> 2);
            const int sh = off & 3;
            uint32_t d[RD + 1];
#pragma unroll
            for (int i = 0; i <= RD; ++i) d[i] = q[i];
#pragma unroll
            for (int i = 0; i < RD; ++i) flat[r * RD + i] = __builtin_amdgcn_alignbyte(d[i + 1], d[i], sh);
        }
        v4i bfrag[KST];
#pragma unroll
        for (int t = 0; t < KST; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) bfrag[t][j] = static_cast<int>(half ? flat[8 * t + 4 + j] : flat[8 * t + j]);

        uint8_t* yp = a.y + ((static_cast<long long>(n) * a.Ho + oy) * a.Wo + ox) * a.Co;
        const OutPtr outp = MakeOutPtr(a.y, static_cast<long long>(a.N) * a.Ho * a.Wo * a.Co);
#pragma unroll
        for (int ct = 0; ct < NT; ++ct)
        {
            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            v16i acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wfrag[ct][0], bfrag[0], zero, 0, 0, 0);
#pragma unroll
            for (int t = 1; t < KST; ++t) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wfrag[ct][t], bfrag[t], acc, 0, 0, 0);
            if constexpr (W2)
            {
#pragma unroll
                for (int t = 0; t < KST; ++t) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wfrag2[ct][t], bfrag[t], acc, 0, 0, 0);
            }
            uint32_t o[4];
#pragma unroll
            for (int qd = 0; qd < 4; ++qd)
            {
                const int cl = ct * 32 + 8 * qd + 4 * half;
                const float4 mp = *reinterpret_cast<const float4*>(&cst[0][cl]);
                const float4 bp = *reinterpret_cast<const float4*>(&cst[1][cl]);
                const float4 mm = *reinterpret_cast<const float4*>(&cst[2][cl]);
                const float4 bm = *reinterpret_cast<const float4*>(&cst[3][cl]);
                o[qd] = Requant4Dev(acc[4 * qd + 0], acc[4 * qd + 1], acc[4 * qd + 2], acc[4 * qd + 3], mp, bp, mm, bm, a.ct, a.corr, cl, a.rq);
            }
            // lane and lane + 32 hold interleaved 4-channel groups of one pixel; trading two dwords gives each of them
            // 16 contiguous channels (the low lane 0..15, the high lane 16..31) and one 16-byte store
            const uint32_t r0 = __shfl_xor(half ? o[0] : o[2], 32);
            const uint32_t r1 = __shfl_xor(half ? o[1] : o[3], 32);
            const uint4 v = half ? uint4{r0, o[2], r1, o[3]} : uint4{o[0], r0, o[1], r1};
            if (ox < a.Wo)
            {
                if (a.vec16) StoreOut16(outp, (yp - a.y) + ct * 32 + 16 * half, StoreVec4{static_cast<int>(v.x), static_cast<int>(v.y), static_cast<int>(v.z), static_cast<int>(v.w)});
                else
                {
                    uint32_t* dst = reinterpret_cast<uint32_t*>(yp + ct * 32 + 16 * half);
                    dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
                }
            }
        }
    }
}

} // namespace mi355x
