// The plan object behind mi355x_conv2d_t, shared by the translation units that launch from it.
#pragma once

#include <hip/hip_runtime.h>

#include <string>
#include <vector>

#include "common.h"
#include "conv_kernels.h"
#include "dw_stem_kernels.h"

struct mi355x_conv2d_s
{
    mi355x_conv2d_desc d{};
    int32_t algo = MI355X_ALGO_DIRECT;
    mi355x::ConvGeom geom{};
    mi355x::Requant rq{};
    // device constants
    uint8_t* w_direct = nullptr;   // [Kh][Kw][Ci][Co] / depthwise [Kh][Kw][Co], raw codes
    int8_t*  w_mfma   = nullptr;   // [Co_pad][K_pad] signed, zero padded
    uint8_t* pad16    = nullptr;   // 16 bytes that turn into the padding value under the kernel's input xor
    int8_t*  w_stem   = nullptr;   // small-Ci conv on MFMA: [Co rounded up to 32][stem_kp]
    int8_t*  w_stem2  = nullptr;   // ... the second halves of weight differences that need two
    int      stem_kp  = 0;
    uint32_t* dw_grp  = nullptr;   // depthwise 3x3: constants per group of 4 channels for the fused dw+pw kernel
    uint32_t* w_dot4  = nullptr;   // depthwise 3x3: [C][4] dwords; small-Ci conv: [Co][Kh][RD] dwords
    uint32_t* w_dot4b = nullptr;   // depthwise 3x3 / small-Ci conv whose weight differences need two int8 halves: the second halves
    int variant = 0;               // kernel variant within an algo (see RunPlan)
    int row_dwords = 0;            // small-Ci conv: dwords per filter row
    float*   chan     = nullptr;   // [8][Co_pad] per-channel requantization constants (rows: see ChanTab)
    int32_t* corr     = nullptr;   // [Co_pad]  -zx' * sum_k w[c][k]
    int K = 0, K_pad = 0, Co_pad = 0;
    int pw_blocks_per_cu = 1, pw_n_cu = 256;     // weight-stationary kernel: blocks a CU holds at once, CUs of the device
    int pw_blocks_per_cu_64 = 0;                 // ... with 64-channel slabs, where the plan's own slab is 128 (0: not prepared)
    std::vector<float> chan_host;  // host copy, completed with the corr-folded rows once corr is known
    std::vector<float> fast_fm, fast_fb;   // per channel: the unwidened fast-path constants and the constant half-width of the
    std::vector<double> fast_cw;           // bracket (negative: no fast path), kept until the table is uploaded
    int pw_bn = 0, pw_ks = 0;      // pointwise GEMM kernel configuration (0: not applicable)
    bool bk128 = false;            // implicit GEMM walks K in 128-byte tiles
    bool halo_ok = false;          // shape fits the resident-tile kernel (weights without a zero point are checked at launch)
    unsigned concurrency = 1;      // launches of the plan's network that run side by side (mi355x_conv2d_set_concurrency)
    int tile_override = 0;         // 0: choose the MFMA tile per launch; 64 / 96 (= 128x64) / 128: the "igemm_tile" option at plan creation
    int opt_xcd_cols = 0;
    int opt_igemm_lds = 2, opt_dw_rows = 0, opt_dw_cb = 0, opt_dw_mfma = 1, opt_stem_dot4 = 0;     // the other process-wide options, as they stood at plan creation
                                   // (launches read the plan, never the mutable globals: plans may run on any host thread)
    uint32_t xor_mask = 0, pad_word = 0;
    int zw_neg = 0;                // MFMA plans: minus the zero point of the stored int8 weights (0: symmetric)
    int rowsum_bias = 0;           // ... and what the bytes between K and K_pad add to a row's sum of activations
    std::string info;

    ~mi355x_conv2d_s()
    {
        (void)hipFree(w_direct);
        (void)hipFree(w_mfma);
        (void)hipFree(pad16);
        (void)hipFree(dw_grp);
        (void)hipFree(w_stem);
        (void)hipFree(w_stem2);
        (void)hipFree(w_dot4);
        (void)hipFree(w_dot4b);
        (void)hipFree(chan);
        (void)hipFree(corr);
    }
};

// The plan object behind mi355x_fc_t: a 1x1 convolution over a 1x1 image with k input channels.
struct mi355x_fc_s
{
    mi355x_conv2d_s* conv = nullptr;
    ~mi355x_fc_s() { delete conv; }
};

namespace mi355x
{

// Arguments of the 3x3 depthwise kernel for `batch` images of this plan, exactly as mi355x_conv2d_run launches it:
// `rows_per_thread` (1 or 2) and `cbw` (32, 64 or 128 channels per block) name the template instance.  The plan must be a
// MI355X_ALGO_DEPTHWISE plan of variant 1.
int FillDw3x3Args(const mi355x_conv2d_s* p, uint32_t batch, const void* x, void* y, Dw3x3Args* a, int* rows_per_thread, int* cbw);

// Arguments of the direct-to-LDS implicit GEMM with BM x BN tiles for `batch` images of this plan (an MI355X_ALGO_MFMA plan
// whose channel count is a multiple of 128); *unit_fast tells whether the launch qualifies for the UNIT template instance.
int FillIgemmLdsArgs(const mi355x_conv2d_s* p, int bm, int bn, uint32_t batch, const void* x, void* y, IgemmArgs* a, bool* unit_fast);

} // namespace mi355x
