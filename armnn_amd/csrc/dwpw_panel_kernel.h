// Depthwise 3x3 (stride 1 or 2) + the pointwise 1x1 convolution that consumes it as ONE kernel, for 256 or 512 channels between
// them: a block of eight waves owns an 8 x 8 pixel tile of one image over ALL channels, and a CU holds one block.
//
//   The intermediate tensor never leaves the CU, and it is produced in exactly the pieces the GEMM consumes: the
//   depthwise layer's channel block kt (128 channels) of the 64 pixels IS k-tile kt of the GEMM's activation operand.
//   The kernel alternates, once per k-tile, between
//     a depthwise phase   the eight waves run the matrix-core arithmetic of DepthwiseMfmaKernel on channel block kt (wave =
//                         16 channels, four groups of 16 pixels: three v_mfma_i32_16x16x64_i8 per group over diagonal weight
//                         operands; a third of the VALU work of the v_dot4 formulation, which bounded this phase),
//                         requantize with the depthwise layer's own constants and write the codes -- the bytes the
//                         separate layer would have stored, shifted to int8 where they are uint8 -- into k-tile kt of the
//                         activation panel in LDS (the xor-swizzled image the MFMA fragment reads expect), and
//     a GEMM phase        all eight waves multiply k-tile kt into accumulators for ALL output channels: wave (wm, wq) keeps
//                         the 32 pixel rows wm x 64 NQ channels wq of the output in 32 NQ registers for the whole kernel.
//   What keeps the phases short is that nothing in them waits for memory: the weights of k-tile kt (64 KB for 512 output
//   channels) and the input halo of channel block kt + 1 are requested at the start of depthwise phase kt -- the halo and
//   the phase's constants first, the weights behind them, because a wave's vector memory operations complete in issue order
//   -- and are first touched after it.  One wait and one barrier per phase.
//   The write-out requantizes from a copy of the pointwise layer's bracket rows in LDS (accumulators start at zero: the
//   zero-point correction is part of rows 6 / 7), stages the 64 x Co output bytes over the weight ring and stores whole
//   rows of Co bytes per pixel.
//   Both layers' arithmetic is untouched -- exact int32 sums, the same requantization routine with the same constants -- so
//   the bytes are those of the two layers run one after the other.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"
#include "dw_stem_kernels.h"
#include "igemm_lds_kernel.h"

namespace mi355x
{

struct DwPwPanelArgs
{
    // depthwise 3x3, multiplier 1, C % 128 == 0
    const uint8_t*  x;
    const uint8_t*  pad16;      // 16 bytes that become the depthwise padding value under dw_xor
    const uint32_t* wpack;      // [C][4] dwords, rows of the 3x3 filter per channel (Dw3x3Args::wpack)
    ChanTab         dw_ct;
    const int32_t*  dw_corr;
    int N, H, W, C, Ho, Wo;
    int pad_top, pad_left;
    int tiles_x, tiles_y;
    int total_tiles, xcd_chunk;
    uint32_t dw_xor;
    Requant dw_rq;
    // pointwise 1x1: K = C, Co = 256 NQ
    const int8_t*  w;           // [Co_pad][K_pad], K_pad == C
    int            K_pad;
    ChanTab        pw_ct;
    const int32_t* pw_corr;
    uint8_t*       y;
    int            Co;
    uint32_t       mid_xor;     // 0x80808080 when the tensor between the layers is uint8: the panel holds the int8-shifted codes
    Requant        pw_rq;
#ifdef MI355X_DWPW_STAMPS
    unsigned long long* stamps; // [blocks][16] shader-clock stamps of wave 0
#endif
};

template <int KT, int NQ, int S = 1>
struct DwPwPanelGeom
{
    static constexpr int NCOL = 256 * NQ;             // output channels
    static constexpr int NT = 4 * NQ;                 // 64-channel weight tiles per k-tile
    static constexpr int HR = 7 * S + 3, HC = 7 * S + 3;   // halo of an 8 x 8 tile of outputs: 10 x 10 or 17 x 17 input pixels
    static constexpr int NCHUNK = HR * HC * 8;        // 16-byte pieces of a halo (128 channels per pixel)
    static constexpr int HPITCH = 144;                // bytes per halo pixel in LDS: 128 + 16, so that the 16-byte reads of 8
                                                      // neighbouring pixels fall on different bank quads (stride 1)
    static constexpr int HROWP = S == 1 ? 1664 : HC * HPITCH;   // bytes per halo row; at stride 1 >= 10 pixels and 128 mod 256, so that
                                                      // the reads of the pixel group's second row take the quads the first row's leave free
    static constexpr int HALO = HR * HROWP;
    static constexpr int LDO = NCOL + 16;
    static constexpr int PANEL = KT * 64 * 128;
    static constexpr int TAB = 4 * NCOL * 4;
    static constexpr int RING = NT * 64 * 128;
    static constexpr int OUT = 64 * LDO;
    static constexpr int WORK = HALO + RING > OUT ? HALO + RING : OUT;   // halo buffer + weight ring; the output staging reuses them
    static constexpr int SMEM = PANEL + TAB + WORK;
};

// KT = C / 128 (2 or 4), NQ = Co / 256 (1 or 2), S = depthwise stride.  512 threads.
template <int KT, int NQ, int S = 1>
__global__ __launch_bounds__(512) void DwPwPanelKernel(DwPwPanelArgs a)
{
    using G = DwPwPanelGeom<KT, NQ, S>;
    constexpr int NCHUNK = G::NCHUNK, NHS = (G::NCHUNK + 511) / 512;     // halo pieces, and pieces per thread
    constexpr int NCOL = G::NCOL, NT = G::NT, HC = G::HC, HALO = G::HALO, LDO = G::LDO, HPITCH = G::HPITCH, HROWP = G::HROWP;
    constexpr int NTHR = 512;
    typedef __attribute__((address_space(3))) void* LdsPtr;
    typedef const __attribute__((address_space(1))) void* GlobalPtr;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* const panel = smem;                                           // [KT][64 pixels][128 B]
    float* const tab = reinterpret_cast<float*>(smem + G::PANEL);          // [4][NCOL]: m+, b+ (corr folded in), m-, b- (corr folded in)
    uint8_t* const halo = smem + G::PANEL + G::TAB;                        // [10 rows of HROWP bytes][10 pixels of HPITCH bytes]
    uint8_t* const ring = halo + HALO;                                 // [NT][64 channels][128 B]
    uint8_t* const Os = halo;                                              // [64][LDO], after the last GEMM phase

    int b = XcdContiguousWorkItem(blockIdx.x, a.xcd_chunk);
    if ((static_cast<int>(blockIdx.x) >> 3) >= a.xcd_chunk || b >= a.total_tiles) return;
    const int tx = b % a.tiles_x; b /= a.tiles_x;
    const int ty = b % a.tiles_y;
    const int n = b / a.tiles_y;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
#ifdef MI355X_DWPW_STAMPS
    int stamp_i = 0;
#define DWPW_STAMP() do { if (tid == 0 && a.stamps) a.stamps[static_cast<size_t>(blockIdx.x) * 16 + stamp_i++] = clock64(); } while (0)
#else
#define DWPW_STAMP() do { } while (0)
#endif
    DWPW_STAMP();

    // ---- depthwise roles: wave = 16 channels of the current 128-channel block; lane (j, g): pixel j of a group of 16 (two
    // tile rows) and tap slot g as an MFMA operand, channel quad g of pixel j as a result
    const int dj = lane & 15, dg = lane >> 4;
    const int drj = dj >> 3, dcj = dj & 7;
    int dtap[3], dwrow[3], dwshift[3];
#pragma unroll
    for (int m = 0; m < 3; ++m)
    {
        const int t = 4 * m + dg;
        const int tc = min(t, 8);                      // slots past the ninth tap read the ninth; their weights are zero
        dtap[m] = (drj * S + tc / 3) * HROWP + (dcj * S + tc % 3) * HPITCH + wave * 16;
        dwrow[m] = tc / 3;
        dwshift[m] = t < 9 ? 8 * (tc % 3) : 24;        // shift 24: the zero byte of a packed filter row
    }
    // ---- staging of a halo: NCHUNK pieces of 16 bytes, NHS per thread at most; only the channel block moves from phase to phase
    const int iy_org = ty * 8 * S - a.pad_top;
    const int ix_org = tx * 8 * S - a.pad_left;
    const uint8_t* const xn = a.x + static_cast<long long>(n) * a.H * a.W * a.C;
    const int dxm = static_cast<int>(a.dw_xor);
    int hoff[NHS], hlds[NHS];                              // offset within the image (-1: outside, reads the padding), place in LDS (-1: none)
#pragma unroll
    for (int k = 0; k < NHS; ++k)
    {
        const int i = min(tid + k * NTHR, NCHUNK - 1);
        const int part = i & 7, pix = i >> 3;
        const int col = pix % HC, hrow = pix / HC;
        const int iy = iy_org + hrow, ix = ix_org + col;
        const bool ok = static_cast<unsigned>(iy) < static_cast<unsigned>(a.H) && static_cast<unsigned>(ix) < static_cast<unsigned>(a.W);
        hoff[k] = ok ? (iy * a.W + ix) * a.C + part * 16 : -1;
        hlds[k] = tid + k * NTHR < NCHUNK ? hrow * HROWP + col * HPITCH + part * 16 : -1;
    }
    auto load_halo = [&](int kt, v4i (&h)[NHS]) {
#pragma unroll
        for (int k = 0; k < NHS; ++k) h[k] = *reinterpret_cast<const v4i*>(hoff[k] >= 0 ? xn + hoff[k] + kt * 128 : a.pad16);
    };
    auto store_halo = [&](const v4i (&h)[NHS]) {
#pragma unroll
        for (int k = 0; k < NHS; ++k)
            if (hlds[k] >= 0) *reinterpret_cast<v4i*>(halo + hlds[k]) = h[k] ^ dxm;
    };

    // ---- GEMM roles: wave (wm, wq) owns pixel rows [32 wm, 32 wm + 32) x output channels [64 NQ wq, 64 NQ (wq + 1)) ----------
    const int wm = wave & 1, wq = wave >> 1;
    const int frag_row = lane & 31, frag_half = lane >> 5;
    const int lane_c = 4 * (lane >> 5);
    // weights of k-tile kt: tile tn (64 channels x 128 B) into ring slot tn; wave w fetches rows [8w, 8w + 8) of every tile,
    // lane l the chunk that belongs in slot (l & 7) of row 8w + (l >> 3)  (chunk c of row r sits at slot c ^ ((r >> 1) & 7))
    const int lrow = lane >> 3;
    const int wrow = 8 * wave + lrow;
    const uint32_t boff = static_cast<uint32_t>(wrow) * static_cast<uint32_t>(a.K_pad) + (((lane & 7) ^ ((wrow >> 1) & 7)) * 16);
    auto load_weights = [&](int kt) {
#pragma unroll
        for (int tn = 0; tn < NT; ++tn)
            __builtin_amdgcn_global_load_lds((GlobalPtr)(a.w + static_cast<long long>(tn) * 64 * a.K_pad + kt * 128 + boff),
                                             (LdsPtr)(ring + tn * 8192 + wave * 1024), 16, 0, 0);
    };

    // ---- prologue: the pointwise layer's bracket rows and the first halo --------------------------------------------------
    {
        constexpr int TABV = NCOL / NTHR + (NCOL % NTHR ? 1 : 0);          // float4 pieces per thread ([4][NCOL / 4] in all)
        float4 tv[TABV];
#pragma unroll
        for (int i = 0; i < TABV; ++i)
        {
            const int e = min(tid + i * NTHR, NCOL - 1);
            const int r = e / (NCOL / 4), col4 = e - r * (NCOL / 4);
            const int src_row = r == 0 ? 2 : r == 1 ? 6 : r == 2 ? 4 : 7;
            tv[i] = *reinterpret_cast<const float4*>(a.pw_ct.p + src_row * a.pw_ct.stride + col4 * 4);
        }
        v4i h0[NHS];
        load_halo(0, h0);
#pragma unroll
        for (int i = 0; i < TABV; ++i)
            if (tid + i * NTHR < NCOL) *reinterpret_cast<float4*>(tab + (tid + i * NTHR) * 4) = tv[i];
        store_halo(h0);
    }
    __syncthreads();
    DWPW_STAMP();

    v16i acc[NQ][2];
#pragma unroll
    for (int t = 0; t < NQ; ++t)
#pragma unroll
        for (int s = 0; s < 2; ++s) acc[t][s] = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
    {
        // ---- requests of this phase, in the order they will be needed: constants, next halo, weights ----------------------
        const int c0 = kt * 128 + wave * 16;
        const uint4 w4 = *reinterpret_cast<const uint4*>(a.wpack + (c0 + dj) * 4);
        const int cq = c0 + 4 * dg;                        // the four channels this lane requantizes
        const v4i corr4 = *reinterpret_cast<const v4i*>(a.dw_corr + cq);
        const Fast4 f4 = LoadFast4(a.dw_ct, cq);
        v4i hn[NHS];
        if (kt + 1 < KT) load_halo(kt + 1, hn);
        load_weights(kt);

        // ---- depthwise phase: channel block kt of the 8 x 8 tile --------------------------------------------------------
        // weight operands: byte dj of the lane's 16 is w[tap][c0 + dj], the others are zero
        v4i wa[3];
        {
            const int dw = dj >> 2, sh = 8 * (dj & 3);
#pragma unroll
            for (int m = 0; m < 3; ++m)
            {
                const uint32_t ra = dwrow[m] == 0 ? w4.x : dwrow[m] == 1 ? w4.y : w4.z;
                const int ba = static_cast<int>(((ra >> dwshift[m]) & 0xffu) << sh);
                wa[m] = v4i{dw == 0 ? ba : 0, dw == 1 ? ba : 0, dw == 2 ? ba : 0, dw == 3 ? ba : 0};
            }
        }
        const uint8_t* hb = halo;
#pragma unroll
        for (int u = 0; u < 4; ++u)
        {
            const v4i b0 = *reinterpret_cast<const v4i*>(hb + dtap[0] + u * 2 * S * HROWP);
            const v4i b1 = *reinterpret_cast<const v4i*>(hb + dtap[1] + u * 2 * S * HROWP);
            const v4i b2 = *reinterpret_cast<const v4i*>(hb + dtap[2] + u * 2 * S * HROWP);
            v4i dacc = corr4;
            dacc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa[0], b0, dacc, 0, 0, 0);
            dacc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa[1], b1, dacc, 0, 0, 0);
            dacc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa[2], b2, dacc, 0, 0, 0);
            // the codes of pixel r = 16 u + dj, channels cq .. cq + 3: chunk `wave` of panel row r, at its swizzled slot
            const uint32_t q = Requant4Dev(dacc[0], dacc[1], dacc[2], dacc[3], f4, a.dw_ct, cq, a.dw_rq) ^ a.mid_xor;
            const int r = 16 * u + dj;
            *reinterpret_cast<uint32_t*>(panel + kt * 8192 + r * 128 + ((wave ^ ((r >> 1) & 7)) * 16) + dg * 4) = q;
        }
        DWPW_STAMP();
        __builtin_amdgcn_s_waitcnt(VmcntImm(0));          // this wave's share of the weights (and of the next halo) has landed
        __syncthreads();                                   // k-tile kt of the panel and all weight tiles are in LDS; the halo has been read
        if (kt + 1 < KT) store_halo(hn);                   // (the barrier behind the GEMM phase orders it before the next phase's reads)
        DWPW_STAMP();

        // ---- GEMM phase: k-tile kt into every accumulator ------------------------------------------------------------------
        const uint8_t* As = panel + kt * 8192;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
        {
            const int sl = ((ks * 2 + frag_half) ^ ((frag_row >> 1) & 7)) * 16;
            const v4i fa = *reinterpret_cast<const v4i*>(As + (wm * 32 + frag_row) * 128 + sl);
#pragma unroll
            for (int t = 0; t < NQ; ++t)
            {
                const uint8_t* Bs = ring + (wq * NQ + t) * 8192;
#pragma unroll
                for (int s = 0; s < 2; ++s)
                {
                    const v4i fw = *reinterpret_cast<const v4i*>(Bs + (s * 32 + frag_row) * 128 + sl);
                    acc[t][s] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw, fa, acc[t][s], 0, 0, 0);
                }
            }
        }
        __syncthreads();                                   // the ring may be refilled; the next halo is in LDS
        DWPW_STAMP();
    }

    // ---- write-out ---------------------------------------------------------------------------------------------------------
#pragma unroll
    for (int t = 0; t < NQ; ++t)
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const int cl = (wq * NQ + t) * 64 + s * 32 + 8 * q + lane_c;
                const float4 mp = *reinterpret_cast<const float4*>(tab + cl);
                const float4 bp = *reinterpret_cast<const float4*>(tab + NCOL + cl);
                const float4 mm = *reinterpret_cast<const float4*>(tab + 2 * NCOL + cl);
                const float4 bm = *reinterpret_cast<const float4*>(tab + 3 * NCOL + cl);
                const v16i& v = acc[t][s];
                const uint32_t out = Requant4Dev(v[4 * q + 0], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3], mp, bp, mm, bm, a.pw_ct, a.pw_corr, cl, a.pw_rq);
                *reinterpret_cast<uint32_t*>(Os + (wm * 32 + frag_row) * LDO + cl) = out;
            }
    __syncthreads();
    DWPW_STAMP();
    const OutPtr outp = MakeOutPtr(a.y, static_cast<long long>(a.N) * a.Ho * a.Wo * a.Co);
    constexpr int CHUNKS = NCOL / 16;                      // 16-byte pieces per pixel
    constexpr int NP = 64 * CHUNKS / NTHR;
#pragma unroll
    for (int i = 0; i < NP; ++i)
    {
        const int idx = tid + i * NTHR;
        const int r = idx / CHUNKS, chunk = idx - r * CHUNKS;
        const int oy = ty * 8 + (r >> 3), ox = tx * 8 + (r & 7);
        if (oy < a.Ho && ox < a.Wo && chunk * 16 < a.Co)
        {
            const v4i ov = *reinterpret_cast<const v4i*>(Os + r * LDO + chunk * 16);
            StoreOut16(outp, ((static_cast<long long>(n) * a.Ho + oy) * a.Wo + ox) * a.Co + chunk * 16, ov);
        }
    }
#ifdef MI355X_DWPW_STAMPS
    __builtin_amdgcn_s_waitcnt(0);
    DWPW_STAMP();
#endif
#undef DWPW_STAMP
}

} // namespace mi355x
