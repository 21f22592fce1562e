// Depthwise 3x3 (stride 1 or 2) + the pointwise 1x1 convolution that consumes it as ONE kernel, for the wide, shallow
// layers at the front of a MobileNet: 32, 64 or 128 channels between the layers, 64, 128 or 256 output channels.
//
// Run apart, these layers are bound by memory: the tensor between them is written once and read once (112 x 112 x 32 at 64
// images: 26 MB each way, next to 26 MB in and 51 MB out).  Here it never leaves the CU.
//   * A block of four (or eight) waves is persistent: it keeps the pointwise weights (at most 256 x 128 bytes) and the pointwise
//     layer's requantization rows in LDS for its whole life and walks items -- TH x TW output pixels of one image over ALL
//     channels -- with the next item's input halo in flight (in registers) while the current one is computed.  Two barriers
//     per item: halo staged / panel complete.
//   * Depthwise phase: the matrix-core arithmetic of DepthwiseMfmaKernel (16 channels x 16 pixels x 4 taps per
//     v_mfma_i32_16x16x64_i8 over diagonal weight operands kept in registers), requantized with the depthwise layer's own
//     constants; the codes -- the bytes the separate layer would have stored, shifted to int8 where they are uint8 -- go
//     to an LDS panel [pixel][channel].
//   * Pointwise phase: v_mfma_i32_32x32x32_i8 over the panel and the resident weights; accumulators start at zero (the
//     zero-point correction is part of rows 6 / 7 of the channel table), the requantized dwords pass through a wave-private
//     LDS area and leave as 16 bytes per lane.
//   * Loads and stores of a wave complete in issue order and share one counter: an item's stores are issued at the start of
//     the next iteration, ahead of that iteration's loads, so the wait for those loads covers nothing younger.
//   * Stores go through a buffer descriptor of the item's image: a pixel right of the image gets an offset past the
//     descriptor's size, a row below the image runs past it by itself, and the hardware drops those stores.
// Both layers' arithmetic is untouched -- exact int32 sums, the same requantization routine with the same constants -- so
// the bytes are those of the two layers run one after the other.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"
#include "dw_mfma_kernel.h"

namespace mi355x
{

struct DwPwStreamArgs
{
    // depthwise 3x3, multiplier 1
    const uint8_t*  x;
    const uint8_t*  pad16;      // 16 bytes that become the depthwise padding value under dw_xor
    const uint32_t* wpack;      // [C][4] dwords, rows of the 3x3 filter per channel (Dw3x3Args::wpack)
    ChanTab         dw_ct;
    const int32_t*  dw_corr;
    int N, H, W, Ho, Wo;
    int pad_top, pad_left;
    int tiles_x, tiles_y;
    int total_items, xcd_chunk;
    uint32_t rcp_tiles_x, rcp_tiles_y;
    uint32_t dw_xor;
    Requant dw_rq;
    // pointwise 1x1
    const int8_t*  w;           // [Co_pad][w_stride]
    int            w_stride;
    ChanTab        pw_ct;
    const int32_t* pw_corr;
    uint8_t*       y;
    uint32_t       mid_xor;     // 0x80808080 when the tensor between the layers is uint8: the panel holds the int8-shifted codes
    Requant        pw_rq;
};

// S: depthwise stride; C: channels between the layers; NO: output channels; TH x TW: output pixels per item; NWAVES: 4 or
// 8 waves per block (8 where the weights and the halo leave room for one block per CU only)
template <int S, int C, int NO, int TH, int TW, int NWAVES = 4>
struct DwPwStreamGeom
{
    static_assert(C == 32 || C == 64 || C == 128 || C == 256, "channels between the layers");
    static_assert(NO == 64 || NO == 128 || NO == 256, "output channels");
    static_assert(TW == 8 || TW == 16, "a group of 16 pixels is one or two whole tile rows");
    static constexpr int NW = NWAVES, NT = 64 * NW;
    static constexpr int NCG = C / 16;
    static constexpr int P = TH * TW;                     // pixels per item
    static_assert(P % 64 == 0, "whole 32-pixel MFMA tiles, two per wave at least");
    static constexpr int NPG = P / 16;
    static constexpr int CGW = NCG > NW ? NCG / NW : 1;  // channel groups per wave
    static constexpr int WPC = NCG < NW ? NW / NCG : 1;  // waves sharing a channel group (they split the pixel groups)
    static constexpr int UNITS = NPG / WPC;               // pixel groups per wave and channel group
    static_assert(NPG % WPC == 0, "pixel groups split evenly");
    static constexpr int HR = (TH - 1) * S + 3;
    static constexpr int HC = (TW - 1) * S + 3;
    static constexpr int PITCH = C + 16;
    static constexpr int ROWP_RAW = HC * PITCH;
    static constexpr int ROWP = (TW == 8 && S == 1) ? ((ROWP_RAW + 127) / 256 * 256 + 128) : ROWP_RAW;
    static constexpr int HALO = HR * ROWP;                // the halo buffer
    static constexpr int KP = C + 16;                     // bytes per panel row and per weight row in LDS
    static constexpr int PANEL = P * KP;
    static constexpr int WTS = NO * KP;
    static constexpr int TAB = 4 * NO * 4;
    static constexpr int MT = P / 32, NTL = NO / 32;      // 32 x 32 MFMA tiles of an item's output
    static constexpr bool BYN = NTL >= NW;                // a wave owns output channels (all pixels) or pixels (all channels)
    static constexpr int MTW = BYN ? MT : MT / NW;
    static constexpr int NTW = BYN ? NTL / NW : NTL;
    static_assert(MTW == 2, "a wave's output area is 64 pixels deep");
    static constexpr int SC = NTW * 32;                   // channels a wave writes per pixel
    static constexpr int LDO = SC + 16;
    static constexpr int OUT = NW * 64 * LDO;
    static constexpr int QUADS = 64 * (SC / 16) / 64;     // 16-byte stores per lane and item
    static constexpr int SMEM = HALO + PANEL + WTS + TAB + OUT;
    // Blocks per CU that LDS allows; the register budget follows it (a few spilled registers cost less than the third block
    // gains: 112 x 112 x 32 -> 64 at 64 images 29.5 us with two blocks, 24.4 with three).
    static constexpr int BLOCKS = 160 * 1024 / SMEM >= 3 ? 3 : 160 * 1024 / SMEM >= 2 ? 2 : 1;
    static constexpr int WAVES_PER_SIMD = BLOCKS * NW / 4;
};

template <int S, int C, int NO, int TH, int TW, int NWAVES = 4>
__global__ __launch_bounds__(64 * NWAVES)
__attribute__((amdgpu_waves_per_eu(DwPwStreamGeom<S, C, NO, TH, TW, NWAVES>::WAVES_PER_SIMD, DwPwStreamGeom<S, C, NO, TH, TW, NWAVES>::WAVES_PER_SIMD)))
void DwPwStreamKernel(DwPwStreamArgs a)
{
    using G = DwPwStreamGeom<S, C, NO, TH, TW, NWAVES>;
    constexpr int NW = G::NW;
    constexpr int NT = G::NT, NCG = G::NCG, HR = G::HR, HC = G::HC, PITCH = G::PITCH, ROWP = G::ROWP, HALO = G::HALO;
    constexpr int CGW = G::CGW, WPC = G::WPC, UNITS = G::UNITS, KP = G::KP, MTW = G::MTW, NTW = G::NTW, LDO = G::LDO, QUADS = G::QUADS;
    constexpr int RPG = 16 / TW;
    constexpr int CPP = C / 16;
    constexpr int NCH = HR * HC * CPP;
    constexpr int NST = (NCH + NT - 1) / NT;
    extern __shared__ __attribute__((aligned(16))) uint8_t dwpw_stream_lds[];
    uint8_t* const lds = dwpw_stream_lds;
    constexpr int PANEL0 = HALO, WTS0 = PANEL0 + G::PANEL, TAB0 = WTS0 + G::WTS, OUT0 = TAB0 + G::TAB;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int xcd = blockIdx.x & 7;
    const int step = static_cast<int>(gridDim.x >> 3);
    const int item_end = min((xcd + 1) * a.xcd_chunk, a.total_items);
    int item = xcd * a.xcd_chunk + static_cast<int>(blockIdx.x >> 3);
    if (item >= item_end) return;

    // ---- resident constants of the pointwise layer -------------------------------------------------------------------------
    for (int i = tid; i < NO * CPP; i += NT)
    {
        const int row = i / CPP, part = i % CPP;
        *reinterpret_cast<v4i*>(lds + WTS0 + row * KP + part * 16) = *reinterpret_cast<const v4i*>(a.w + static_cast<long long>(row) * a.w_stride + part * 16);
    }
    for (int i = tid; i < NO; i += NT)                  // [4][NO / 4] float4: m+, b+ (corr folded in), m-, b- (corr folded in)
    {
        const int r = i / (NO / 4), col4 = i % (NO / 4);
        const int src_row = r == 0 ? 2 : r == 1 ? 6 : r == 2 ? 4 : 7;
        *reinterpret_cast<float4*>(lds + TAB0 + i * 16) = *reinterpret_cast<const float4*>(a.pw_ct.p + src_row * a.pw_ct.stride + col4 * 4);
    }

    // ---- staging of the input halo (as in DepthwiseMfmaKernel, all C channels) -------------------------------------------
    const int dxm = static_cast<int>(a.dw_xor);
    const int in_image = a.H * a.W * C;
    int st_lds[NST], st_row[NST], st_col[NST], st_off[NST];
#pragma unroll
    for (int k = 0; k < NST; ++k)
    {
        const int i = min(tid + k * NT, NCH - 1);
        const int part = i % CPP;
        const int pix = i / CPP;
        st_col[k] = pix % HC;
        st_row[k] = pix / HC;
        st_lds[k] = st_row[k] * ROWP + st_col[k] * PITCH + part * 16;
        st_off[k] = (st_row[k] * a.W + st_col[k]) * C + part * 16;
        if (tid + k * NT >= NCH) st_lds[k] = -1;
    }
    v4i st[NST];
    struct Where { int tx, ty, n; };
    auto decode = [&](int b) {
        Where w;
        int q = DivByInvariant(b, a.tiles_x, a.rcp_tiles_x);
        w.tx = b - q * a.tiles_x; b = q;
        q = DivByInvariant(b, a.tiles_y, a.rcp_tiles_y);
        w.ty = b - q * a.tiles_y; w.n = q;
        return w;
    };
    auto issue = [&](int b) {
        const Where w = decode(b);
        const int iy_org = w.ty * TH * S - a.pad_top;
        const int ix_org = w.tx * TW * S - a.pad_left;
        const uint8_t* xn = a.x + static_cast<long long>(w.n) * in_image;
        const int org = (iy_org * a.W + ix_org) * C;
#pragma unroll
        for (int k = 0; k < NST; ++k)
        {
            const bool ok = static_cast<unsigned>(iy_org + st_row[k]) < static_cast<unsigned>(a.H) &&
                            static_cast<unsigned>(ix_org + st_col[k]) < static_cast<unsigned>(a.W);
            const uint8_t* src = ok ? xn + (org + st_off[k]) : a.pad16;
            st[k] = *reinterpret_cast<const v4i*>(src);
        }
    };
    auto commit = [&](int halo) {
#pragma unroll
        for (int k = 0; k < NST; ++k)
            if (st_lds[k] >= 0) *reinterpret_cast<v4i*>(lds + halo + st_lds[k]) = st[k] ^ dxm;
    };

    // ---- depthwise roles: lane (j, g): pixel j of a group of 16 and tap slot g as an operand, channel quad g as a result --
    const int j = lane & 15, g = lane >> 4;
    const int rj = j / TW, cj = j % TW;
    const int cg0 = NCG > NW ? wave * CGW : wave % NCG;
    const int pg0 = NCG > NW ? 0 : wave / NCG;
    int lds_tap[3];
    v4i wa[CGW][3], corr4[CGW];
    Fast4 f4[CGW];
    {
        int wrow[3], wshift[3];
#pragma unroll
        for (int m = 0; m < 3; ++m)
        {
            const int t = 4 * m + g;
            const int tc = min(t, 8);                      // slots past the ninth tap read the ninth; their weights are zero
            lds_tap[m] = ((pg0 * RPG + rj) * S + tc / 3) * ROWP + (cj * S + tc % 3) * PITCH + cg0 * 16;
            wrow[m] = tc / 3;
            wshift[m] = t < 9 ? 8 * (tc % 3) : 24;         // shift 24: the zero byte of a packed filter row
        }
#pragma unroll
        for (int i = 0; i < CGW; ++i)
        {
            const int c0 = (cg0 + i) * 16;
            const uint4 w4 = *reinterpret_cast<const uint4*>(a.wpack + (c0 + j) * 4);
            const int dw = j >> 2, sh = 8 * (j & 3);
#pragma unroll
            for (int m = 0; m < 3; ++m)
            {
                const uint32_t ra = wrow[m] == 0 ? w4.x : wrow[m] == 1 ? w4.y : w4.z;
                const int ba = static_cast<int>(((ra >> wshift[m]) & 0xffu) << sh);
                wa[i][m] = v4i{dw == 0 ? ba : 0, dw == 1 ? ba : 0, dw == 2 ? ba : 0, dw == 3 ? ba : 0};
            }
            corr4[i] = *reinterpret_cast<const v4i*>(a.dw_corr + c0 + 4 * g);
            f4[i] = LoadFast4(a.dw_ct, c0 + 4 * g);
        }
    }
    // the codes of pixel (pg0 + u WPC) 16 + j, channels (cg0 + i) 16 + 4 g ..: one dword of the panel
    const int panel_write = PANEL0 + (pg0 * 16 + j) * KP + cg0 * 16 + 4 * g;

    // ---- pointwise roles: wave owns 32 x 32 tiles [m0, m0 + MTW) x [n0, n0 + NTW) of the item's P x NO output -------------
    const int m0 = G::BYN ? 0 : wave * MTW;
    const int n0 = G::BYN ? wave * NTW : 0;
    const int frag_row = lane & 31, frag_half = lane >> 5;
    const int a_frag = PANEL0 + (m0 * 32 + frag_row) * KP + frag_half * 16;
    const int b_frag = WTS0 + (n0 * 32 + frag_row) * KP + frag_half * 16;
    // the wave's output area [64 pixels][LDO]; lane writes dwords at (pixel frag_row of tile mt, channels 8 q + 4 frag_half of tile nt)
    const int out_area = OUT0 + wave * 64 * LDO;
    const int out_write = out_area + frag_row * LDO + 4 * frag_half;
    // 16-byte pieces of that area: piece id = k 64 + lane -> (pixel id / PPP, part id % PPP).  64 / PPP pixels per store
    // instruction are whole tile rows, so a lane keeps its column and part; only the row moves with k.
    constexpr int PPP = G::SC / 16;
    constexpr int RPS = 64 / PPP / TW;                     // tile rows per store instruction
    static_assert((64 / PPP) % TW == 0, "whole tile rows per store instruction");
    const int sr0 = lane / PPP, part0 = lane % PPP;
    const int y_col = (m0 * 32 + sr0) % TW;
    const int out_read = out_area + sr0 * LDO + part0 * 16;
    const int y_lane = (((m0 * 32 + sr0) / TW) * a.Wo + y_col) * NO + n0 * 32 + part0 * 16;
    const int y_step = RPS * a.Wo * NO;
    const int image_bytes = a.Ho * a.Wo * NO;

    int out_base = 0, out_n = -1, out_cols = 0;
    auto store_outputs = [&]() {
        const __amdgpu_buffer_rsrc_t yrsrc = __builtin_amdgcn_make_buffer_rsrc(a.y + static_cast<long long>(out_n) * image_bytes, 0, image_bytes, 0x00020000);
#pragma unroll
        for (int k = 0; k < QUADS; ++k)
        {
            const v4i v = *reinterpret_cast<const v4i*>(lds + out_read + k * (64 / PPP) * LDO);
            const int yo = y_col < out_cols ? out_base + y_lane + k * y_step : static_cast<int>(0x80000000u);
            __builtin_amdgcn_raw_buffer_store_b128(v, yrsrc, yo, 0, 0);
        }
    };
    auto depthwise = [&](int halo) {
#pragma unroll
        for (int i = 0; i < CGW; ++i)
#pragma unroll
            for (int u = 0; u < UNITS; ++u)
            {
                const int lo = halo + i * 16 + u * (WPC * RPG * S * ROWP);
                const v4i b0 = *reinterpret_cast<const v4i*>(lds + lds_tap[0] + lo);
                const v4i b1 = *reinterpret_cast<const v4i*>(lds + lds_tap[1] + lo);
                const v4i b2 = *reinterpret_cast<const v4i*>(lds + lds_tap[2] + lo);
                v4i acc = corr4[i];
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa[i][0], b0, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa[i][1], b1, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa[i][2], b2, acc, 0, 0, 0);
                const uint32_t q = Requant4Dev(acc[0], acc[1], acc[2], acc[3], f4[i], a.dw_ct, (cg0 + i) * 16 + 4 * g, a.dw_rq) ^ a.mid_xor;
                *reinterpret_cast<uint32_t*>(lds + panel_write + i * 16 + u * (WPC * 16 * KP)) = q;
            }
    };
    auto pointwise = [&](int b) {
        const Where w = decode(b);
        out_base = ((w.ty * TH) * a.Wo + w.tx * TW) * NO;
        out_cols = a.Wo - w.tx * TW;
        out_n = w.n;
        v16i acc[MTW][NTW];
#pragma unroll
        for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) acc[mt][nt] = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < C / 32; ++ks)
        {
            v4i fa[MTW], fw[NTW];
#pragma unroll
            for (int mt = 0; mt < MTW; ++mt) fa[mt] = *reinterpret_cast<const v4i*>(lds + a_frag + mt * 32 * KP + ks * 32);
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) fw[nt] = *reinterpret_cast<const v4i*>(lds + b_frag + nt * 32 * KP + ks * 32);
#pragma unroll
            for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[nt], fa[mt], acc[mt][nt], 0, 0, 0);
        }
        const float* tab = reinterpret_cast<const float*>(lds + TAB0);
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const int cl = (n0 + nt) * 32 + 8 * q + 4 * frag_half;
                const float4 mp = *reinterpret_cast<const float4*>(tab + cl);
                const float4 bp = *reinterpret_cast<const float4*>(tab + NO + cl);
                const float4 mm = *reinterpret_cast<const float4*>(tab + 2 * NO + cl);
                const float4 bm = *reinterpret_cast<const float4*>(tab + 3 * NO + cl);
#pragma unroll
                for (int mt = 0; mt < MTW; ++mt)
                {
                    const v16i& v = acc[mt][nt];
                    const uint32_t out = Requant4Dev(v[4 * q + 0], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3], mp, bp, mm, bm, a.pw_ct, a.pw_corr, cl, a.pw_rq);
                    *reinterpret_cast<uint32_t*>(lds + out_write + mt * 32 * LDO + nt * 32 + 8 * q) = out;
                }
            }
    };

    issue(item);
    while (true)
    {
        // (one halo buffer: its readers, the depthwise phase of the item before, all passed that item's second barrier)
        commit(0);
        // all waves are done with the item before (its panel has been multiplied) and this item's halo is in LDS; on the first
        // pass the barrier also orders the resident weights and table rows before their first use
        __syncthreads();
        // the item before leaves its wave-private area (LDS operations of a wave complete in order: no barrier needed), ahead
        // of the next loads
        if (out_n >= 0) store_outputs();
        const int next = item + step;
        const bool more = next < item_end;
        if (more) issue(next);
        depthwise(0);
        __syncthreads();                                   // the panel is complete
        pointwise(item);
        if (!more) break;
        item = next;
    }
    store_outputs();
}

} // namespace mi355x
