// DepthwiseConvolution2d 3x3 (multiplier 1, stride 1 or 2, channels % 16 == 0) on the matrix cores.
//
// The VALU kernel (Depthwise3x3Kernel) spends 17 vector instructions per output byte.  Here the nine multiply-adds of an
// output are rows of a v_mfma_i32_16x16x64_i8:
//
//     D[channel i][pixel j]  =  sum over k = (tap slot g, channel e)   A[i][16 g + e] * B[16 g + e][j]
//     A[i][16 g + e] = w[tap][c0 + i]  if e == i, else 0          (16 channels x 4 taps: four diagonal 16 x 16 blocks)
//     B[16 g + e][j] = x'[pixel j shifted by tap][c0 + e]         (16 bytes of one NHWC pixel: one ds_read_b128)
//
// One instruction covers 16 channels x 16 pixels x 4 taps; three cover the nine taps (slots 9 .. 11 carry zero weights).
// Only 1/16 of the multiplier array does useful work and it is still cheaper than the VALU: 48 matrix-core clocks per
// 256 outputs against 17 x 4 x 4 = 272 VALU clocks, and the activations need no transposition -- the B operand of lane
// (pixel j, tap slot g) is the 16 contiguous channel bytes of the halo pixel under that tap.  A lane of the result holds
// four consecutive channels of one pixel, which is what the requantization wants.  The accumulators are exact int32 sums
// started at the zero-point correction, so the bytes written are those of the VALU kernel.
//
// Work item: CB channels of a TH x TW tile of outputs; the halo tile is staged in LDS as signed bytes exactly as in the
// VALU kernel (16-byte chunks, out-of-image chunks read the prepared padding).  A wave owns one group of 16 channels
// (four waves: CB = 64 channels per block, or 32 with two waves sharing a group), keeps its weight operands and
// requantization constants in registers while the channel block stays the same, and walks the tile's groups of 16 pixels.
// (128 channels per block, eight waves, was slower everywhere: two such blocks fill a CU and their barriers bind more waves.)
// The pixel pitch in LDS is CB + 16 bytes (an odd number of 16-byte units): the 16 lanes of one tap slot then read 16
// different bank quads at stride 1.
//
// What the structure answers to (cycle stamps per phase, 112 x 112 x 32 at 64 images):
//   * One item per block leaves nothing to overlap, so a block walks several items with the next item's loads in flight
//     (in registers) while the current one is computed; two halo buffers, one barrier per item.
//   * A vector memory instruction occupies the CU's address unit for about 16 clocks whatever it moves, so a dword per
//     lane is the expensive way to store: the requantized dwords (4 channels of a pixel) go through a wave-private LDS
//     area and leave as 16 bytes per lane (16 channels of a pixel), four pixel groups per store instruction.
//   * Loads and stores of a wave complete in issue order and share one counter, so a wait for the next item's loads
//     also waits for every store issued after them.  The stores of an item are therefore issued at the start of the next
//     iteration, ahead of that iteration's loads: the wait at the following commit then covers nothing younger.
//   * The item index is decoded with multiplications by reciprocals the host provides (scalar unit), not divisions.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"
#include "dw_stem_kernels.h"

namespace mi355x
{

template <int S, int CB, int TH, int TW>
struct DwMfmaTile
{
    static constexpr int NCG = CB / 16;                  // channel groups of 16
    static constexpr int NT = 256;
    static constexpr int NW = NT / 64;
    static constexpr int NPX = TH * TW;
    static constexpr int NPG = (NPX + 15) / 16;          // pixel groups of 16 (the last may be partial)
    static constexpr int HR = (TH - 1) * S + 3;
    static constexpr int HC = (TW - 1) * S + 3;
    static constexpr int PITCH = CB + 16;
    // With 8-pixel tile rows a pixel group spans two rows: a row pitch of 128 mod 256 bytes puts the second row's
    // eight reads on the bank quads the first row's leave free (stride 1).
    static constexpr int ROWP_RAW = HC * PITCH;
    static constexpr int ROWP = (TW == 8 && S == 1) ? ((ROWP_RAW + 127) / 256 * 256 + 128) : ROWP_RAW;
    static constexpr int WPC = NW / NCG;                 // waves sharing a channel group (they split the pixel groups)
    static constexpr int UNITS = (NPG + WPC - 1) / WPC;  // pixel groups per wave and item
    static constexpr int QUADS = (UNITS + 3) / 4;        // store instructions per wave and item (four pixel groups each)
    // the pixel groups are dealt to those waves in whole rounds: the rows a last, partly empty round reads exist in LDS
    static constexpr int ROWS_READ = ((UNITS * WPC * (16 / TW)) - 1) * S + 3;
    static constexpr int HALO = (ROWS_READ > HR ? ROWS_READ : HR) * ROWP;   // one of the two halo buffers
    static constexpr int OUT = NW * QUADS * 1024;        // the waves' output areas: 4 pixel groups x 16 pixels x 16 bytes each
    static constexpr int SMEM = 2 * HALO + OUT;
};

// floor(b / d) for b * d < 2^32 with rcp = ceil(2^32 / d)
__device__ __forceinline__ int DivByInvariant(int b, int d, uint32_t rcp)
{
    return d == 1 ? b : static_cast<int>(__umulhi(static_cast<uint32_t>(b), rcp));
}

// Grid: 8 * blocks_per_xcd blocks.  Block (x = blockIdx % 8, i = blockIdx / 8) takes items x * xcd_chunk + i,
// + blocks_per_xcd, ... below (x + 1) * xcd_chunk and below total_blocks (item: channel block fastest, then tile column,
// tile row, image): the blocks of one XCD share neighbouring items and so its L2.
template <int S, bool W2, int CB, int TH, int TW>
__global__ __launch_bounds__((DwMfmaTile<S, CB, TH, TW>::NT)) void DepthwiseMfmaKernel(Dw3x3Args a)
{
    static_assert(CB == 32 || CB == 64, "32 or 64 channels per block: four waves, one or two per group of 16 channels");
    static_assert(TW == 8 || TW == 16, "a group of 16 pixels is one or two whole tile rows");
    using G = DwMfmaTile<S, CB, TH, TW>;
    constexpr int NCG = G::NCG, NT = G::NT, HR = G::HR, HC = G::HC, PITCH = G::PITCH, ROWP = G::ROWP;
    constexpr int WPC = G::WPC, UNITS = G::UNITS, QUADS = G::QUADS;
    constexpr int RPG = 16 / TW;                 // tile rows per pixel group
    constexpr int CPP = CB / 16;                 // 16-byte staging chunks per pixel
    constexpr int NCH = HR * HC * CPP;
    constexpr int NST = (NCH + NT - 1) / NT;
    extern __shared__ __attribute__((aligned(16))) uint8_t dw_mfma_lds[];     // two halo buffers, then the waves' output areas

    const int tid = threadIdx.x;
    const int xcd = blockIdx.x & 7;
    const int step = static_cast<int>(gridDim.x >> 3);
    const int item_end = min((xcd + 1) * a.xcd_chunk, a.total_blocks);
    int item = xcd * a.xcd_chunk + static_cast<int>(blockIdx.x >> 3);
    if (item >= item_end) return;

    const int xm = static_cast<int>(a.xor_mask);
    const int in_image = a.H * a.W * a.C;        // (the host checks that an image stays below 2 GiB)
    // this thread's staging chunks: the same places in every item's halo tile
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
        st_off[k] = (st_row[k] * a.W + st_col[k]) * a.C + part * 16;
        if (tid + k * NT >= NCH) st_lds[k] = -1;
    }
    v4i st[NST];
    struct Where { int cb, tx, ty, n; };
    auto decode = [&](int b) {
        Where w;
        int q = DivByInvariant(b, a.cblocks, a.rcp_cblocks);
        w.cb = b - q * a.cblocks; b = q;
        q = DivByInvariant(b, a.tiles_x, a.rcp_tiles_x);
        w.tx = b - q * a.tiles_x; b = q;
        q = DivByInvariant(b, a.tiles_y, a.rcp_tiles_y);
        w.ty = b - q * a.tiles_y; w.n = q;
        return w;
    };
    // chunks of channels past the tensor's last one: only in the last channel block of a count that is no multiple of CB
    uint32_t st_past = 0;
#pragma unroll
    for (int k = 0; k < NST; ++k)
        if ((a.C % CB) != 0 && (min(tid + k * NT, NCH - 1) % CPP) * 16 >= a.C % CB) st_past |= 1u << k;
    // all of a thread's staging loads are issued before the first is used; a chunk outside the image (or of channels that
    // do not exist) reads 16 prepared bytes that become the padding value under the xor, so no load sits in a divergent branch
    auto issue = [&](int b) {
        const Where w = decode(b);
        const int iy_org = w.ty * TH * S - a.pad_top;
        const int ix_org = w.tx * TW * S - a.pad_left;
        const uint8_t* xn = a.x + static_cast<long long>(w.n) * in_image + w.cb * CB;
        const int org = (iy_org * a.W + ix_org) * a.C;
        const uint32_t past = w.cb == a.cblocks - 1 ? st_past : 0u;
#pragma unroll
        for (int k = 0; k < NST; ++k)
        {
            const bool ok = static_cast<unsigned>(iy_org + st_row[k]) < static_cast<unsigned>(a.H) &&
                            static_cast<unsigned>(ix_org + st_col[k]) < static_cast<unsigned>(a.W) && ((past >> k) & 1u) == 0u;
            const uint8_t* src = ok ? xn + (org + st_off[k]) : a.pad16;
            st[k] = *reinterpret_cast<const v4i*>(src);
        }
    };
    auto commit = [&](int halo) {
#pragma unroll
        for (int k = 0; k < NST; ++k)
            if (st_lds[k] >= 0) *reinterpret_cast<v4i*>(dw_mfma_lds + halo + st_lds[k]) = st[k] ^ xm;
    };

    // ---- this lane's place in the operands --------------------------------------------------------------------------
    // Pixel group pg of the tile = outputs 16 pg .. 16 pg + 15 in row-major order: RPG whole tile rows, so lane (pixel j)
    // sits at row pg RPG + rj, column cj with rj, cj fixed, and everything that depends on pg is a compile-time offset.
    const int lane = tid & 63, wave = tid >> 6;
    const int j = lane & 15;                     // A: channel within the group; B and D: pixel within the group
    const int g = lane >> 4;                     // A and B: tap slot; D: channel quad; stores: pixel group within four
    const int rj = j / TW, cj = j % TW;
    const int cg = wave % NCG;
    const int pg0 = wave / NCG;                  // this wave's pixel groups: pg0, pg0 + WPC, ...
    int lds_tap[3];                              // LDS offset of this lane's B operand for pixel group pg0, tap 4 m + g
                                                 // (slots past the ninth tap read the ninth; their weights are zero)
    int wrow[3], wshift[3];                      // where that tap's weight sits in the packed dwords; shift 24 = the zero byte
#pragma unroll
    for (int m = 0; m < 3; ++m)
    {
        const int t = 4 * m + g;
        const int tc = min(t, 8);
        lds_tap[m] = ((pg0 * RPG + rj) * S + tc / 3) * ROWP + (cj * S + tc % 3) * PITCH + cg * 16;
        wrow[m] = tc / 3;
        wshift[m] = t < 9 ? 8 * (tc % 3) : 24;
    }
    // the wave's output area: unit u = 4 k + v of an item puts its dwords at [k][v][pixel j][quad g]; lane (j, g) later
    // reads the 16 bytes [k][v = g][j] and stores them (pixel j of the wave's pixel group 4 k + g, its 16 channels)
    const int out_area = 2 * G::HALO + wave * (QUADS * 1024);
    const int out_write = out_area + j * 16 + g * 4;
    const int out_read = out_area + g * 256 + j * 16;
    // byte offset of that store from the tile's first output of channel block 0, and per four pixel groups
    const int y_pg = WPC * RPG * a.Wo * a.C;
    const int y_lane = ((pg0 * RPG + rj) * a.Wo + cj) * a.C + cg * 16 + g * y_pg;
    const int image_bytes = a.Ho * a.Wo * a.C;   // (the host checks that an image stays below 2 GiB)

    v4i wa[3], wb[3], corr4;
    Fast4 f4;
    int cur_cb = -1;
    // weight operands of channel block cb: byte j of the lane's 16 is w[tap][c0 + j], the others are zero
    auto constants = [&](int cb) {
        const int c0 = cb * CB + cg * 16;
        const uint4 w4 = *reinterpret_cast<const uint4*>(a.wpack + (c0 + j) * 4);
        uint4 v4 = uint4{0u, 0u, 0u, 0u};
        if constexpr (W2) v4 = *reinterpret_cast<const uint4*>(a.wpack2 + (c0 + j) * 4);
        const int dw = j >> 2, sh = 8 * (j & 3);
#pragma unroll
        for (int m = 0; m < 3; ++m)
        {
            const uint32_t ra = wrow[m] == 0 ? w4.x : wrow[m] == 1 ? w4.y : w4.z;
            const uint32_t rb = wrow[m] == 0 ? v4.x : wrow[m] == 1 ? v4.y : v4.z;
            const int ba = static_cast<int>(((ra >> wshift[m]) & 0xffu) << sh);
            const int bb = static_cast<int>(((rb >> wshift[m]) & 0xffu) << sh);
            wa[m] = v4i{dw == 0 ? ba : 0, dw == 1 ? ba : 0, dw == 2 ? ba : 0, dw == 3 ? ba : 0};
            wb[m] = v4i{dw == 0 ? bb : 0, dw == 1 ? bb : 0, dw == 2 ? bb : 0, dw == 3 ? bb : 0};
        }
        const int cq = c0 + 4 * g;               // the four channels this lane requantizes
        corr4 = *reinterpret_cast<const v4i*>(a.corr + cq);
        f4 = LoadFast4(a.ct, cq);
    };
    // Stores go through a buffer descriptor of the item's image: a lane whose pixel lies right of the image or whose channels
    // do not exist gets an offset past the descriptor's size and a row below the image runs past it by itself, so the
    // hardware drops those stores and the loop needs neither a predicate nor address arithmetic per pixel group.
    int out_y0 = 0, out_n = -1;
    auto store_outputs = [&]() {
        const __amdgpu_buffer_rsrc_t yrsrc = __builtin_amdgcn_make_buffer_rsrc(a.y + static_cast<long long>(out_n) * image_bytes, 0, image_bytes, 0x00020000);
#pragma unroll
        for (int k = 0; k < QUADS; ++k)
        {
            const v4i v = *reinterpret_cast<const v4i*>(dw_mfma_lds + out_read + k * 1024);
            int yo = out_y0 + k * 4 * y_pg;
            // pixel groups past the wave's last one, and rows of a group past the tile's last row (they belong to the tile below)
            if (4 * k + 3 >= UNITS || ((4 * k + 3) * WPC + WPC - 1) * RPG + RPG - 1 >= TH)
                if (4 * k + g >= UNITS || (pg0 + (4 * k + g) * WPC) * RPG + rj >= TH) yo = static_cast<int>(0x80000000u);
            __builtin_amdgcn_raw_buffer_store_b128(v, yrsrc, yo, 0, 0);
        }
    };
    auto compute = [&](int b, int halo) {
        const Where w = decode(b);
        if (w.cb != cur_cb) { constants(w.cb); cur_cb = w.cb; }
        const int cq = w.cb * CB + cg * 16 + 4 * g;
        const bool lane_ok = w.tx * TW + cj < a.Wo && w.cb * CB + cg * 16 < a.C;
        out_y0 = lane_ok ? y_lane + ((w.ty * TH) * a.Wo + w.tx * TW) * a.C + w.cb * CB : static_cast<int>(0x80000000u);
        out_n = w.n;
#pragma unroll
        for (int u = 0; u < UNITS; ++u)
        {
            const int lo = halo + u * (WPC * RPG * S * ROWP);
            const v4i b0 = *reinterpret_cast<const v4i*>(dw_mfma_lds + lds_tap[0] + lo);
            const v4i b1 = *reinterpret_cast<const v4i*>(dw_mfma_lds + lds_tap[1] + lo);
            const v4i b2 = *reinterpret_cast<const v4i*>(dw_mfma_lds + lds_tap[2] + lo);
            v4i acc = corr4;
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa[0], b0, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa[1], b1, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa[2], b2, acc, 0, 0, 0);
            if constexpr (W2)
            {
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wb[0], b0, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wb[1], b1, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wb[2], b2, acc, 0, 0, 0);
            }
            const uint32_t out = Requant4Dev(acc[0], acc[1], acc[2], acc[3], f4, a.ct, cq, a.rq);
            *reinterpret_cast<uint32_t*>(dw_mfma_lds + out_write + (u >> 2) * 1024 + (u & 3) * 256) = out;
        }
    };
    issue(item);
    int buf = 0;
    while (true)
    {
        commit(buf * G::HALO);
        // every wave has finished the item before last (it read this buffer's twin) before any wave passes this barrier a
        // second time, so one barrier per item orders both the writes above and the reuse of the buffers
        __syncthreads();
        // the item before leaves its wave-private area (LDS operations of a wave complete in order: no barrier needed)
        if (out_n >= 0) store_outputs();
        const int next = item + step;
        const bool more = next < item_end;
        if (more) issue(next);
        compute(item, buf * G::HALO);
        if (!more) break;
        item = next;
        buf ^= 1;
    }
    store_outputs();
}

} // namespace mi355x
