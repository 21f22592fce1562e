// Convolution2d / DepthwiseConvolution2d / FullyConnected entry points of the C ABI: plan creation
// (constant re-layout, per-channel requantization constants, kernel selection) and launches.
#include "common.h"
#include "conv_kernels.h"
#include "dw_stem_kernels.h"
#include "dw_mfma_kernel.h"
#include "dwpw_kernel.h"
#include "dwpw_panel_kernel.h"
#include "dwpw_stream_kernel.h"
#include "pwdw_kernel.h"
#include "pool_softmax_items.h"
#include "igemm_ksplit_kernel.h"
#include "pw_gemm_kernel.h"
#include "igemm_lds_kernel.h"
#include "big_gemm.h"
#include "halo_conv_kernel.h"
#include "plan.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <string>
#include <vector>

using namespace mi355x;

namespace
{
// An Addition waiting to be fused into the next launch of this thread (mi355x_conv2d_run_add): the launchers whose
// kernels can do it take it and mark it taken; otherwise the caller runs the Addition as a launch of its own.
struct PendingAdd
{
    const uint8_t* other = nullptr;
    AddFuse fuse{};
    bool taken = false;
};
thread_local PendingAdd* t_pending_add = nullptr;

// unit roundoff of fp32 and the relative half-width of the requantization bracket (device_math.h)
constexpr double kBracketUnit = 1.0 / 16777216.0;
constexpr double kBracketRel = 16.0 / 16777216.0;


void FoldCorrIntoTable(mi355x_conv2d_s* p, const std::vector<int32_t>& corr, int Co);
void ChoosePointwiseConfig(mi355x_conv2d_s* p);
int PreparePointwise(mi355x_conv2d_s* p);

int Upload(void** dst, const void* src, size_t bytes)
{
    MI355X_HIP(hipMalloc(dst, bytes));
    return UploadNow(*dst, src, bytes);
}

int ValidateQuant(const mi355x_quant& q, const char* what)
{
    if (!IsActivationDtype(q.dtype)) return SetError(MI355X_ERR_UNSUPPORTED, "%s: data type %d is not QAsymmS8/QAsymmU8", what, q.dtype);
    if (!(q.scale > 0.0f) || !std::isfinite(q.scale)) return SetError(MI355X_ERR_INVALID_ARGUMENT, "%s: scale must be positive and finite", what);
    return 0;
}

// `weights` in the reference layout: conv [Co][Kh][Kw][Ci]; depthwise [1][Kh][Kw][Co].
int ChooseDwMfmaTile(int stride, int Ho, int Wo, int forced);

int BuildPlan(const mi355x_conv2d_desc& d, const void* weights_host, const mi355x_const_quant* wq,
              const int32_t* bias_host, const mi355x_const_quant* bq, mi355x_conv2d_s* p)
{
    if (!weights_host || !wq) return SetError(MI355X_ERR_INVALID_ARGUMENT, "weights / weight quantization missing");
    if (d.in_h == 0 || d.in_w == 0 || d.in_c == 0 || d.out_h == 0 || d.out_w == 0 || d.out_c == 0 || d.kernel_h == 0 ||
        d.kernel_w == 0 || d.stride_x == 0 || d.stride_y == 0 || d.dilation_x == 0 || d.dilation_y == 0)
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "zero extent / stride / dilation in convolution descriptor");
    if (int rc = ValidateQuant(d.input, "input")) return rc;
    if (int rc = ValidateQuant(d.output, "output")) return rc;
    if (wq->dtype != MI355X_QSYMM_S8 && wq->dtype != MI355X_QASYMM_S8 && wq->dtype != MI355X_QASYMM_U8)
        return SetError(MI355X_ERR_UNSUPPORTED, "weights data type %d is not an 8-bit quantized type", wq->dtype);
    if (wq->n_scales != 1 && wq->n_scales != d.out_c)
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "weights carry %u scales; expected 1 or %u", wq->n_scales, d.out_c);
    if (!wq->scales) return SetError(MI355X_ERR_INVALID_ARGUMENT, "weight scales missing");
    if (wq->n_scales > 1 && wq->offset != 0)
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "per-axis weights must have offset 0");
    if (d.bias_enabled)
    {
        if (!bias_host || !bq || !bq->scales) return SetError(MI355X_ERR_INVALID_ARGUMENT, "bias enabled but bias data / quantization missing");
        if (bq->dtype != MI355X_SIGNED32) return SetError(MI355X_ERR_UNSUPPORTED, "bias must be Signed32");
        if (bq->n_scales != 1 && bq->n_scales != d.out_c)
            return SetError(MI355X_ERR_INVALID_ARGUMENT, "bias carries %u scales; expected 1 or %u", bq->n_scales, d.out_c);
        if (bq->offset != 0) return SetError(MI355X_ERR_INVALID_ARGUMENT, "bias offset must be 0");
    }
    if (d.depthwise && (d.out_c % d.in_c) != 0)
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "depthwise: out_c %u is not a multiple of in_c %u", d.out_c, d.in_c);
    if (d.activation < MI355X_ACT_NONE || d.activation > MI355X_ACT_BOUNDED_RELU)
        return SetError(MI355X_ERR_UNSUPPORTED, "activation %d cannot be fused", d.activation);
    // the output extent must be consistent with the window walk (bottom/right padding is implied, never negative reach)
    {
        const long long need_h = static_cast<long long>(d.out_h - 1) * d.stride_y + static_cast<long long>(d.kernel_h - 1) * d.dilation_y;
        const long long need_w = static_cast<long long>(d.out_w - 1) * d.stride_x + static_cast<long long>(d.kernel_w - 1) * d.dilation_x;
        if (need_h > 2ll * 1000000 || need_w > 2ll * 1000000) return SetError(MI355X_ERR_INVALID_ARGUMENT, "unreasonable geometry");
    }

    p->d = d;
    p->opt_igemm_lds = GlobalOptions().igemm_lds;
    p->opt_xcd_cols = GlobalOptions().igemm_xcd_cols;
    p->opt_dw_rows = GlobalOptions().dw_rows;
    p->opt_dw_cb = GlobalOptions().dw_cb;
    p->opt_dw_mfma = GlobalOptions().dw_mfma;
    p->opt_stem_dot4 = GlobalOptions().stem_dot4;
    const int Co = static_cast<int>(d.out_c), Ci = static_cast<int>(d.in_c);
    const int Kh = static_cast<int>(d.kernel_h), Kw = static_cast<int>(d.kernel_w);
    ConvGeom& g = p->geom;
    g.H = d.in_h; g.W = d.in_w; g.Ci = Ci; g.Ho = d.out_h; g.Wo = d.out_w; g.Co = Co;
    g.Kh = Kh; g.Kw = Kw;
    g.pad_top = d.pad_top; g.pad_left = d.pad_left; g.stride_x = d.stride_x; g.stride_y = d.stride_y;
    g.dil_x = d.dilation_x; g.dil_y = d.dilation_y;
    g.depth_mult = d.depthwise ? Co / Ci : 1;
    g.zx = d.input.offset; g.zw = wq->offset;
    g.in_u8 = d.input.dtype == MI355X_QASYMM_U8;
    g.w_u8 = wq->dtype == MI355X_QASYMM_U8;
    p->rq = MakeRequant(d.output, d.activation, d.activation_a, d.activation_b);

    p->K = d.depthwise ? Kh * Kw : Kh * Kw * Ci;
    // Every kernel accumulates sum (x - zx)(w - zw) in 32 bits.  CpuRef accumulates in float and saturates at the end, so
    // a sum that could wrap here is refused rather than computed wrongly: K * max|x - zx| * max|w - zw| must stay below 2^31.
    {
        const long long xmax = g.in_u8 ? std::max(std::abs(0 - g.zx), std::abs(255 - g.zx)) : std::max(std::abs(-128 - g.zx), std::abs(127 - g.zx));
        const size_t nw = static_cast<size_t>(d.depthwise ? 1 : Co) * Kh * Kw * (d.depthwise ? Co : Ci);
        const uint8_t* wb = static_cast<const uint8_t*>(weights_host);
        long long wmax = 0;
        for (size_t i = 0; i < nw; ++i)
        {
            const int wv = g.w_u8 ? static_cast<int>(wb[i]) : static_cast<int>(static_cast<int8_t>(wb[i]));
            wmax = std::max<long long>(wmax, std::abs(wv - g.zw));
        }
        if (static_cast<long long>(p->K) * xmax * wmax >= (1ll << 31))
            return SetError(MI355X_ERR_UNSUPPORTED, "%d taps of up to %lld x %lld could overflow the 32-bit accumulator", p->K, xmax, wmax);
    }
    p->Co_pad = (Co + 127) / 128 * 128;
    // K is padded to the implicit GEMM's k-tile.  128-byte tiles pay when a row chunk is one whole cache line, i.e. when
    // 128 consecutive K bytes are contiguous in memory (input channels a multiple of 128) and K needs no extra padding
    // for it; otherwise 64.
    p->K_pad = (p->K + 63) / 64 * 64;
    p->bk128 = (d.in_c % 128) == 0 && (p->K % 128) == 0;
    // small filter, stride 1, 64 / 128 / 256 input channels: the resident-tile kernel (halo_conv_kernel.h) walks K in
    // 128-byte tiles, so K is padded to that
    p->halo_ok = !d.depthwise && (d.in_c == 64 || d.in_c == 128 || d.in_c == 256) && d.kernel_h * d.kernel_w > 1 && d.kernel_h <= 3 &&
                 d.kernel_w <= 3 && d.stride_x == 1 && d.stride_y == 1 && d.dilation_x == 1 && d.dilation_y == 1 && d.out_w <= 224;
    if (p->halo_ok) p->K_pad = (p->K + 127) / 128 * 128;

    // ---- per-channel requantization constants, in fp32 exactly as the reference's decoders produce them ----
    std::vector<float> mult(p->Co_pad, 0.0f), biasf(p->Co_pad, 0.0f);
    for (int c = 0; c < Co; ++c)
    {
        const float sw = wq->n_scales == 1 ? wq->scales[0] : wq->scales[c];
        mult[c] = d.input.scale * sw;
        if (d.bias_enabled)
        {
            if (bq->n_scales == 1)
            {
                // ScaledInt32Decoder, or Int32Decoder when no scale is set (Decoders.hpp:40-55)
                const float sb = bq->scales[0];
                biasf[c] = sb == 0.0f ? static_cast<float>(bias_host[c]) : static_cast<float>(bias_host[c]) * sb;
            }
            else
            {
                biasf[c] = static_cast<float>(bias_host[c]) * bq->scales[c];   // ScaledInt32PerAxisDecoder
            }
        }
    }
    // fast-path coefficients: the bracket r- < f / s_out + offset' < r+ of device_math.h, one FMA per side.  A channel
    // whose constants do not qualify gets a bracket that never closes (bytes 255 and 0), so it always takes the exact path.
    {
        const int CP = p->Co_pad;
        std::vector<float> tab(static_cast<size_t>(8) * CP, 0.0f);
        const float inv = 1.0f / d.output.scale;
        // the fast path works 128 codes higher for signed outputs (Requant::pk_bias), so that is its offset
        const float zp_f = static_cast<float>(d.output.offset + (d.output.dtype == MI355X_QASYMM_U8 ? 0 : 128));
        const double max_acc = static_cast<double>(p->K) * 65025.0;
        const bool base_ok = !GlobalOptions().exact_division_epilogue && std::isnormal(inv) && std::isnormal(d.output.scale) &&
                             d.output.offset >= -255 && d.output.offset <= 255 && p->rq.fast_ok;
        p->fast_fm.assign(CP, 0.0f);
        p->fast_fb.assign(CP, 0.0f);
        p->fast_cw.assign(CP, -1.0);
        for (int c = 0; c < CP; ++c)
        {
            tab[c] = mult[c];
            tab[CP + c] = biasf[c];
            if (c >= Co) continue;                    // padding: both sides give byte 0, nothing is ever redone or stored
            tab[3 * CP + c] = tab[6 * CP + c] = 255.0f;
            if (!base_ok) continue;
            const float fm = mult[c] * inv;
            const float fb = biasf[c] * inv + zp_f;
            const double bq = std::fabs(static_cast<double>(biasf[c])) * inv;
            // constant half-width (device_math.h): 1.5 * 2^-24 * (14 |biasf/s_out| + 10 |offset'| + 64) + 2 e; the part
            // proportional to the value is the factor 1 +- e on both constants
            const double cw = 1.5 * kBracketUnit * (14.0 * bq + 10.0 * std::fabs(static_cast<double>(zp_f)) + 64.0) + 2.0 * kBracketRel;
            const bool ok = std::isfinite(fm) && std::isfinite(fb) && std::isfinite(cw) && cw < 0.125 &&
                            max_acc * std::fabs(static_cast<double>(fm)) < 268435456.0;
            if (!ok) continue;
            tab[2 * CP + c] = static_cast<float>(static_cast<double>(fm) * (1.0 + kBracketRel));
            tab[3 * CP + c] = static_cast<float>(static_cast<double>(fb) * (1.0 + kBracketRel) + cw);
            tab[4 * CP + c] = static_cast<float>(static_cast<double>(fm) * (1.0 - kBracketRel));
            tab[5 * CP + c] = static_cast<float>(static_cast<double>(fb) * (1.0 - kBracketRel) - cw);
            // until a kernel folds its zero-point correction in, rows 6/7 never close either
            tab[6 * CP + c] = 255.0f;
            tab[7 * CP + c] = 0.0f;
            p->fast_fm[c] = fm;
            p->fast_fb[c] = fb;
            p->fast_cw[c] = cw;
        }
        p->chan_host = tab;
    }

    // ---- kernel selection ----------------------------------------------------------------------------------
    const int zx_shift = g.in_u8 ? g.zx - 128 : g.zx;
    // weights as the MFMA kernels store them: int8, uint8 shifted by 128 like the activations; their zero point likewise
    const int zw_shift = g.w_u8 ? g.zw - 128 : g.zw;
    const bool mfma_ok = !d.depthwise && zw_shift >= -128 && zw_shift <= 127 && (Ci % 16) == 0 && zx_shift >= -128 && zx_shift <= 127 &&
                         p->K <= 100000;
    const bool dw_ok = d.depthwise && g.depth_mult == 1 && (Co % 4) == 0;
    // depthwise 3x3 on v_dot4 with an LDS halo tile
    // It multiplies the activations with d = w - zw, one int8 when every d fits, else two int8 halves (floor(d / 2) and
    // the rest); d = 255 has no such halves.
    bool dw3_fits = true, dw3_halves = true;
    if (dw_ok && Kh == 3 && Kw == 3 && zw_shift >= -128 && zw_shift <= 127)
    {
        const uint8_t* wb = static_cast<const uint8_t*>(weights_host);
        for (int i = 0; i < 9 * Co; ++i)
        {
            const int dv = static_cast<int>(static_cast<int8_t>(g.w_u8 ? wb[i] ^ 0x80u : wb[i])) - zw_shift;
            dw3_fits &= dv >= -128 && dv <= 127;
            dw3_halves &= dv != 255;
        }
    }
    const bool dw3_ok = dw_ok && zw_shift >= -128 && zw_shift <= 127 && zx_shift >= -128 && zx_shift <= 127 && dw3_halves && Kh == 3 &&
                        Kw == 3 && (Co % 16) == 0 && d.dilation_x == 1 && d.dilation_y == 1 && d.stride_x == d.stride_y &&
                        (d.stride_x == 1 || d.stride_x == 2);
    // stems: <= 4 input channels, rows of Kw*Ci bytes walked with v_dot4
    const int row_bytes = Kw * Ci;
    bool stem_fits = true, stem_halves = true;
    if (!d.depthwise && Ci <= 4 && zw_shift >= -128 && zw_shift <= 127)
    {
        const uint8_t* wb = static_cast<const uint8_t*>(weights_host);
        for (long long i = 0; i < static_cast<long long>(Co) * p->K; ++i)
        {
            const int dv = static_cast<int>(static_cast<int8_t>(g.w_u8 ? wb[i] ^ 0x80u : wb[i])) - zw_shift;
            stem_fits &= dv >= -128 && dv <= 127;
            stem_halves &= dv != 255;
        }
    }
    const bool stem_ok = !d.depthwise && zw_shift >= -128 && zw_shift <= 127 && zx_shift >= -128 && zx_shift <= 127 && stem_halves &&
                         Ci <= 4 && (Co % 4) == 0 && d.dilation_x == 1 && d.dilation_y == 1 &&
                         d.stride_x == d.stride_y && (d.stride_x == 1 || d.stride_x == 2) &&
                         ((Kh == 3 && row_bytes <= 12) || (Kh == 7 && row_bytes <= 24) || (Kh == 1 && row_bytes <= 4) ||
                          (Kh == 5 && row_bytes <= 20));
    int32_t algo = d.algo;
    if (algo == MI355X_ALGO_AUTO)
        algo = mfma_ok ? MI355X_ALGO_MFMA : dw_ok ? MI355X_ALGO_DEPTHWISE : stem_ok ? MI355X_ALGO_DOT4 : MI355X_ALGO_DIRECT;
    if (algo == MI355X_ALGO_DOT4 && !stem_ok)
        return SetError(MI355X_ERR_UNSUPPORTED, "dot4 kernel needs <= 4 input channels, symmetric int8 weights, stride 1 or 2, "
                                                "no dilation and a 1/3/5/7-row filter");
    if (algo == MI355X_ALGO_MFMA && !mfma_ok)
        return SetError(MI355X_ERR_UNSUPPORTED, "MFMA kernel needs a non-depthwise layer and in_c %% 16 == 0");
    if (algo == MI355X_ALGO_DEPTHWISE && !dw_ok)
        return SetError(MI355X_ERR_UNSUPPORTED, "depthwise kernel needs multiplier 1 and channels %% 4 == 0");
    if (algo < MI355X_ALGO_DIRECT || algo > MI355X_ALGO_DOT4) return SetError(MI355X_ERR_INVALID_ARGUMENT, "unknown algo %d", algo);
    p->algo = algo;

    const uint8_t* wsrc = static_cast<const uint8_t*>(weights_host);
    if (algo == MI355X_ALGO_MFMA)
    {
        std::vector<int8_t> wp(static_cast<size_t>(p->Co_pad) * p->K_pad, 0);
        std::vector<int32_t> corr(p->Co_pad, 0);
        for (int c = 0; c < Co; ++c)
        {
            long long sum = 0;
            const int8_t* src = reinterpret_cast<const int8_t*>(wsrc) + static_cast<size_t>(c) * p->K;
            int8_t* dst = wp.data() + static_cast<size_t>(c) * p->K_pad;
            for (int k = 0; k < p->K; ++k)
            {
                dst[k] = g.w_u8 ? static_cast<int8_t>(static_cast<uint8_t>(src[k]) ^ 0x80u) : src[k];
                sum += dst[k];
            }
            // sum_k (x' - zx')(w - zw') = sum_k x'w - zx' sum_k w - zw' sum_k x' + K zx' zw' over the K bytes of a row, of which
            // those outside the image are zx'; the term with sum_k x' is the kernel's
            corr[c] = static_cast<int32_t>(-static_cast<long long>(zx_shift) * sum + static_cast<long long>(zw_shift) * zx_shift * p->K);
        }
        p->zw_neg = -zw_shift;
        p->rowsum_bias = (p->K_pad - p->K) * zx_shift;     // kernels that walk K_pad bytes meet zx' beyond K
        if (int rc = Upload(reinterpret_cast<void**>(&p->w_mfma), wp.data(), wp.size())) return rc;
        if (int rc = Upload(reinterpret_cast<void**>(&p->corr), corr.data(), corr.size() * sizeof(int32_t))) return rc;
        p->xor_mask = g.in_u8 ? 0x80808080u : 0u;
        const uint32_t zb = static_cast<uint32_t>(zx_shift) & 0xffu;
        p->pad_word = zb | (zb << 8) | (zb << 16) | (zb << 24);
        {
            const std::vector<uint8_t> padbytes(16, static_cast<uint8_t>((zb ^ (g.in_u8 ? 0x80u : 0u)) & 0xffu));
            if (int rc = Upload(reinterpret_cast<void**>(&p->pad16), padbytes.data(), padbytes.size())) return rc;
        }
        p->tile_override = GlobalOptions().igemm_tile;
        if (p->bk128 && (Ci % 128) == 0)
            if (int rc = PrepareBigGemm()) return rc;
        FoldCorrIntoTable(p, corr, Co);
        ChoosePointwiseConfig(p);
        if (p->tile_override != 0) p->pw_bn = 0;     // a forced tile also forces the LDS-tiled implicit GEMM
        if (int rc = PreparePointwise(p)) return rc;
        char buf[128];
        if (p->pw_bn)
            snprintf(buf, sizeof(buf), "pointwise_gemm_mfma_i8_32x32x32 weight-stationary slab %dxK=%d, chunk %d k-steps", p->pw_bn, p->K, p->pw_ks);
        else if (p->bk128 && (Ci % 128) == 0)
            snprintf(buf, sizeof(buf), "igemm_mfma_i8_32x32x32 global_load_lds tiles 64x64..256x256 x128 K=%d", p->K);
        else
            snprintf(buf, sizeof(buf), "igemm_mfma_i8_32x32x32 tiles 128x128|128x64|64x64 x%d K=%d", p->bk128 ? 128 : 64, p->K);
        p->info = buf;
        if (p->zw_neg != 0) p->info += ", weight zero point by row sums";
        else if (p->halo_ok) p->info += "; launches of 192 or more row tiles: input tile resident in LDS for all taps";
    }
    else if (algo == MI355X_ALGO_DEPTHWISE && dw3_ok)
    {
        // [1][3][3][C] -> per channel 4 dwords, dword r = { w[r][0], w[r][1], w[r][2], 0 }
        // the kernel works in blocks of 32 channels: its per-channel arrays are padded to whole blocks
        const int C32 = (Co + 31) / 32 * 32;
        std::vector<uint32_t> wp(static_cast<size_t>(C32) * 4, 0u), wp2(static_cast<size_t>(C32) * 4, 0u);
        std::vector<int32_t> corr(C32, 0);
        for (int c = 0; c < Co; ++c)
        {
            long long sum = 0;
            for (int r = 0; r < 3; ++r)
            {
                uint32_t dw = 0, dw2 = 0;
                for (int kx = 0; kx < 3; ++kx)
                {
                    const uint8_t raw = wsrc[(r * 3 + kx) * Co + c];
                    const int dv = static_cast<int>(static_cast<int8_t>(g.w_u8 ? raw ^ 0x80u : raw)) - zw_shift;
                    const int first = dw3_fits ? dv : dv >> 1;        // floor(d / 2): -128 .. 127
                    dw |= static_cast<uint32_t>(static_cast<uint8_t>(first)) << (8 * kx);
                    dw2 |= static_cast<uint32_t>(static_cast<uint8_t>(dv - first)) << (8 * kx);
                    sum += dv;
                }
                wp[static_cast<size_t>(c) * 4 + r] = dw;
                wp2[static_cast<size_t>(c) * 4 + r] = dw2;
            }
            corr[c] = static_cast<int32_t>(-static_cast<long long>(zx_shift) * sum);
        }
        if (int rc = Upload(reinterpret_cast<void**>(&p->w_dot4), wp.data(), wp.size() * sizeof(uint32_t))) return rc;
        if (!dw3_fits)
            if (int rc = Upload(reinterpret_cast<void**>(&p->w_dot4b), wp2.data(), wp2.size() * sizeof(uint32_t))) return rc;
        if (int rc = Upload(reinterpret_cast<void**>(&p->corr), corr.data(), corr.size() * sizeof(int32_t))) return rc;
        p->xor_mask = g.in_u8 ? 0x80808080u : 0u;
        const uint32_t zb = static_cast<uint32_t>(zx_shift) & 0xffu;
        p->pad_word = zb | (zb << 8) | (zb << 16) | (zb << 24);
        p->variant = 1;
        {
            // [C/4][8][4] dwords: weight rows 0..2, corr, m+, b+, m-, b- (rows 2..5 of the channel table)
            const int CP = p->Co_pad;
            std::vector<uint32_t> grp(static_cast<size_t>(Co / 4) * 32, 0u);
            for (int c = 0; c < Co; ++c)
            {
                uint32_t* gdst = grp.data() + static_cast<size_t>(c / 4) * 32 + (c % 4);
                for (int r = 0; r < 3; ++r) gdst[r * 4] = wp[static_cast<size_t>(c) * 4 + r];
                gdst[3 * 4] = static_cast<uint32_t>(corr[c]);
                for (int r = 0; r < 4; ++r) std::memcpy(&gdst[(4 + r) * 4], &p->chan_host[static_cast<size_t>(2 + r) * CP + c], 4);
            }
            if (int rc = Upload(reinterpret_cast<void**>(&p->dw_grp), grp.data(), grp.size() * sizeof(uint32_t))) return rc;
            const std::vector<uint8_t> padbytes(16, static_cast<uint8_t>((zb ^ (g.in_u8 ? 0x80u : 0u)) & 0xffu));
            if (int rc = Upload(reinterpret_cast<void**>(&p->pad16), padbytes.data(), padbytes.size())) return rc;
        }
        {
            // rows x pixels x channels of a block's tile with one output row per thread (twice the rows with two)
            const int cbw = p->opt_dw_cb == 32 ? 32 : (Co % 128) == 0 ? 128 : (Co % 64) == 0 ? 64 : 32;
            const int pixels = (cbw == 128 ? 2 : 4) * (d.stride_x == 1 ? 4 : 2);
            char buf[96];
            if (p->opt_dw_mfma != 0)
            {
                std::snprintf(buf, sizeof(buf), "depthwise3x3_mfma16x16x64_lds stride %d", static_cast<int>(d.stride_x));
            }
            else
                std::snprintf(buf, sizeof(buf), "depthwise3x3_dot4_lds stride %d, tile %dx%dx%d", static_cast<int>(d.stride_x), cbw == 32 ? 8 : 4, pixels, cbw);
            p->info = buf;
        }
        if (p->w_dot4b) p->info += ", weights minus their zero point as two int8 halves";
    }
    else if (algo == MI355X_ALGO_DEPTHWISE)
    {
        if (int rc = Upload(reinterpret_cast<void**>(&p->w_direct), wsrc, static_cast<size_t>(Kh) * Kw * Co)) return rc;
        p->info = "depthwise_c4_valu";
    }
    else if (algo == MI355X_ALGO_DOT4)
    {
        const int RD = Kh == 3 ? 3 : Kh == 7 ? 6 : Kh == 5 ? 5 : 1;
        std::vector<uint32_t> wp(static_cast<size_t>(Co) * Kh * RD, 0u), wp2(static_cast<size_t>(Co) * Kh * RD, 0u);
        std::vector<int32_t> corr(Co, 0);
        for (int c = 0; c < Co; ++c)
        {
            long long sum = 0;
            for (int r = 0; r < Kh; ++r)
                for (int bidx = 0; bidx < row_bytes; ++bidx)
                {
                    // the weight minus the weights' zero point, whole or as floor(d / 2) and the rest
                    const uint8_t raw = wsrc[(static_cast<size_t>(c) * Kh + r) * row_bytes + bidx];
                    const int dv = static_cast<int>(static_cast<int8_t>(g.w_u8 ? raw ^ 0x80u : raw)) - zw_shift;
                    const int first = stem_fits ? dv : dv >> 1;
                    const size_t at = (static_cast<size_t>(c) * Kh + r) * RD + bidx / 4;
                    wp[at] |= static_cast<uint32_t>(static_cast<uint8_t>(first)) << (8 * (bidx % 4));
                    wp2[at] |= static_cast<uint32_t>(static_cast<uint8_t>(dv - first)) << (8 * (bidx % 4));
                    sum += dv;
                }
            corr[c] = static_cast<int32_t>(-static_cast<long long>(zx_shift) * sum);
        }
        if (int rc = Upload(reinterpret_cast<void**>(&p->w_dot4), wp.data(), wp.size() * sizeof(uint32_t))) return rc;
        if (!stem_fits)
            if (int rc = Upload(reinterpret_cast<void**>(&p->w_dot4b), wp2.data(), wp2.size() * sizeof(uint32_t))) return rc;
        if (int rc = Upload(reinterpret_cast<void**>(&p->corr), corr.data(), corr.size() * sizeof(int32_t))) return rc;
        p->xor_mask = g.in_u8 ? 0x80u : 0u;
        p->pad_word = static_cast<uint32_t>(zx_shift) & 0xffu;
        p->row_dwords = RD;
        {
            const std::vector<uint8_t> padbytes(16, static_cast<uint8_t>((p->pad_word ^ p->xor_mask) & 0xffu));
            if (int rc = Upload(reinterpret_cast<void**>(&p->pad16), padbytes.data(), padbytes.size())) return rc;
        }
        if (Co == 32 || Co == 64)
        {
            // the same rows, end to end, as the K vector of the MFMA variant
            const int kp = (Kh * RD * 4 + 31) / 32 * 32;
            const int rows = (Co + 31) / 32 * 32;
            std::vector<int8_t> wm(static_cast<size_t>(rows) * kp, 0);
            for (int c = 0; c < Co; ++c) std::memcpy(wm.data() + static_cast<size_t>(c) * kp, wp.data() + static_cast<size_t>(c) * Kh * RD, static_cast<size_t>(Kh) * RD * 4);
            if (int rc = Upload(reinterpret_cast<void**>(&p->w_stem), wm.data(), wm.size())) return rc;
            if (!stem_fits)
            {
                std::fill(wm.begin(), wm.end(), 0);
                for (int c = 0; c < Co; ++c) std::memcpy(wm.data() + static_cast<size_t>(c) * kp, wp2.data() + static_cast<size_t>(c) * Kh * RD, static_cast<size_t>(Kh) * RD * 4);
                if (int rc = Upload(reinterpret_cast<void**>(&p->w_stem2), wm.data(), wm.size())) return rc;
            }
            p->stem_kp = kp;
        }
        FoldCorrIntoTable(p, corr, Co);
        char buf[96];
        snprintf(buf, sizeof(buf), "smallci_dot4_lds %dx%dx%d stride %u, tile 32x16", Kh, Kw, Ci, d.stride_x);
        p->info = buf;
        if (p->w_dot4b) p->info += ", weights minus their zero point as two int8 halves";
    }
    else
    {
        if (d.depthwise)
        {
            if (int rc = Upload(reinterpret_cast<void**>(&p->w_direct), wsrc, static_cast<size_t>(Kh) * Kw * Co)) return rc;
        }
        else
        {
            // [Co][Kh][Kw][Ci] -> [Kh][Kw][Ci][Co]
            std::vector<uint8_t> wt(static_cast<size_t>(Co) * p->K);
            const size_t taps = static_cast<size_t>(Kh) * Kw * Ci;
            for (int c = 0; c < Co; ++c)
                for (size_t k = 0; k < taps; ++k) wt[k * Co + c] = wsrc[static_cast<size_t>(c) * taps + k];
            if (int rc = Upload(reinterpret_cast<void**>(&p->w_direct), wt.data(), wt.size())) return rc;
        }
        p->info = d.depthwise ? "direct_depthwise" : "direct_conv";
    }
    if (int rc = Upload(reinterpret_cast<void**>(&p->chan), p->chan_host.data(), p->chan_host.size() * sizeof(float))) return rc;
    p->chan_host.clear();
    p->chan_host.shrink_to_fit();
    p->fast_fm = std::vector<float>();
    p->fast_fb = std::vector<float>();
    p->fast_cw = std::vector<double>();
    return 0;
}

// Rows 6/7 of the channel table: the bracket with the zero-point correction folded in,
//   bc+- = (fb + corr * fm) (1 +- e) +- (c + 1.5 * 2^-24 * 5 |corr * fm|)
// (the accumulator then starts at zero and only the rare exact path adds corr as an integer; the wider constant covers
// the roundings of corr * fm and of the two conversions of an accumulator beyond 2^24).
void FoldCorrIntoTable(mi355x_conv2d_s* p, const std::vector<int32_t>& corr, int Co)
{
    const int CP = p->Co_pad;
    std::vector<float>& tab = p->chan_host;
    for (int c = 0; c < Co && c < static_cast<int>(p->fast_cw.size()); ++c)
    {
        if (p->fast_cw[c] < 0.0) continue;            // fast path disabled for this channel
        const double cq = static_cast<double>(corr[c]) * static_cast<double>(p->fast_fm[c]);
        const double fbc = static_cast<double>(p->fast_fb[c]) + cq;
        const double cw = p->fast_cw[c] + 1.5 * kBracketUnit * 5.0 * std::fabs(cq);
        if (!std::isfinite(fbc) || !(cw < 0.125) || std::fabs(static_cast<double>(corr[c])) >= 16777216.0) continue;
        tab[6 * CP + c] = static_cast<float>(fbc * (1.0 + kBracketRel) + cw);
        tab[7 * CP + c] = static_cast<float>(fbc * (1.0 - kBracketRel) - cw);
    }
}

// Configuration of the weight-stationary pointwise GEMM kernel, or bn == 0 when it does not apply.
void ChoosePointwiseConfig(mi355x_conv2d_s* p)
{
    const mi355x_conv2d_desc& d = p->d;
    p->pw_bn = 0;
    const bool pointwise = !d.depthwise && d.kernel_h == 1 && d.kernel_w == 1 && d.stride_x == 1 && d.stride_y == 1 &&
                           d.pad_top == 0 && d.pad_left == 0 && d.out_h == d.in_h && d.out_w == d.in_w;
    const int K = static_cast<int>(d.in_c), N = static_cast<int>(d.out_c);
    // with K beyond 128 the LDS-tiled implicit GEMM is the faster kernel (its k-tiles keep more loads in flight than a
    // wave's register chunks can); the weight-stationary kernel is for the shallow, wide-M layers
    if (!pointwise || (K % 32) != 0 || K > 128) return;
    const int budget = 80 * 1024;
    int bn = 0;
    // 128 channels per slab only with 128 input channels: with 32 or 64 a tile's arithmetic is mostly its write-out, and twice
    // as many waves with half the write-out each overlap better than the saved second read of the (small) activations
    // (64 -> 256 channels at 16 x 56 x 56 rows: 11.1 -> 10.1 us, with the Addition in the write-out 16.3 -> 13.4 us)
    const int widest = N > 64 && PwSmemBytes<128>(K) <= budget ? 128 : N > 32 && PwSmemBytes<64>(K) <= budget ? 64 : PwSmemBytes<32>(K) <= budget ? 32 : 0;
    bn = widest == 128 && K <= 64 ? 64 : widest;
    // the "pw_slab" option: another slab width than the automatic one (never wider than the layer's output)
    const int forced = GlobalOptions().pw_slab;
    if (forced != 0 && forced <= widest) bn = forced;
    if (bn == 0) return;
    const int steps = K / 32;
    p->pw_bn = bn;
    p->pw_ks = (steps % 8) == 0 ? 8 : (steps % 4) == 0 ? 4 : (steps % 2) == 0 ? 2 : 1;
}

// Plan-time set-up of the weight-stationary kernel: allow its LDS slab and ask how many blocks a CU holds at once
// (registers and LDS), so that a launch can size its grid to exactly one resident wave of blocks.
template <int BN, int KS>
int PreparePw(mi355x_conv2d_s* p, int* blocks_per_cu)
{
    auto kernel = p->zw_neg != 0 ? PwGemmKernel<BN, KS, (KS <= 2 ? 4 : 2), true> : PwGemmKernel<BN, KS, (KS <= 2 ? 4 : 2), false>;
    MI355X_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
    int per_cu = 1, dev = 0, n_cu = 256;
    MI355X_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, PwSmemBytes<BN>(p->geom.Ci)));
    MI355X_HIP(hipGetDevice(&dev));
    MI355X_HIP(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
    *blocks_per_cu = std::max(1, per_cu);
    p->pw_n_cu = std::max(1, n_cu);
    return 0;
}

template <int BN>
int PreparePwKs(mi355x_conv2d_s* p, int* blocks_per_cu)
{
    switch (p->pw_ks)
    {
    case 8: return PreparePw<BN, 8>(p, blocks_per_cu);
    case 4: return PreparePw<BN, 4>(p, blocks_per_cu);
    case 2: return PreparePw<BN, 2>(p, blocks_per_cu);
    default: return PreparePw<BN, 1>(p, blocks_per_cu);
    }
}

int PreparePointwise(mi355x_conv2d_s* p)
{
    if (p->pw_bn == 128)
    {
        // a plan that shares the device with another lane's launches runs on 64-channel slabs (see RunPlan), unless the
        // slab width was forced
        if (GlobalOptions().pw_slab == 0)
            if (int rc = PreparePwKs<64>(p, &p->pw_blocks_per_cu_64)) return rc;
        return PreparePwKs<128>(p, &p->pw_blocks_per_cu);
    }
    if (p->pw_bn == 64) return PreparePwKs<64>(p, &p->pw_blocks_per_cu);
    if (p->pw_bn == 32) return PreparePwKs<32>(p, &p->pw_blocks_per_cu);
    return 0;
}

template <int BN, int KS>
int LaunchPw(const mi355x_conv2d_s* p, long long M, const void* x, void* y, hipStream_t stream, int blocks_per_cu)
{
    const ConvGeom& g = p->geom;
    PwArgs a;
    a.x = static_cast<const uint8_t*>(x);
    a.w = p->w_mfma;
    a.ct = ChanTab{p->chan, p->Co_pad};
    a.corr = p->corr;
    a.y = static_cast<uint8_t*>(y);
    a.M = static_cast<int>(M);
    a.K = g.Ci;
    a.N = g.Co;
    a.w_stride = p->K_pad;
    a.n_slabs = (g.Co + BN - 1) / BN;
    a.xor_mask = p->xor_mask;
    a.zw_neg = p->zw_neg;
    a.rq = p->rq;
    a.res = nullptr;
    if (t_pending_add && (g.Co & 15) == 0)
    {
        a.res = t_pending_add->other;
        a.add = t_pending_add->fuse;
        t_pending_add->taken = true;
    }
    const int smem = PwSmemBytes<BN>(g.Ci);
    auto kernel = p->zw_neg != 0 ? PwGemmKernel<BN, KS, (KS <= 2 ? 4 : 2), true> : PwGemmKernel<BN, KS, (KS <= 2 ? 4 : 2), false>;
    const int n_cu = p->pw_n_cu, cached_per_cu = blocks_per_cu;            // queried once, when the plan was built
    // exactly one resident wave of blocks: every block walks its share of the row tiles
    const long long groups = ((M + 31) / 32 + 3) / 4;
    long long gm = (static_cast<long long>(n_cu) * cached_per_cu) / a.n_slabs;
    gm = gm / 8 * 8;                // the kernel deals groups out to the 8 XCDs
    if (gm < 8) gm = 8;
    if (gm > (groups + 7) / 8 * 8) gm = (groups + 7) / 8 * 8;
    a.gm = static_cast<int>(gm);
    NoteKernel("PwGemmKernel<%d, %d, %d, %s>", BN, KS, KS <= 2 ? 4 : 2, BoolName(p->zw_neg != 0));
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(a.n_slabs * gm)), dim3(256), smem, stream, a);
    MI355X_HIP(hipGetLastError());
    return 0;
}

template <int BN>
int LaunchPwKs(const mi355x_conv2d_s* p, long long M, const void* x, void* y, hipStream_t stream, int blocks_per_cu)
{
    switch (p->pw_ks)
    {
    case 8: return LaunchPw<BN, 8>(p, M, x, y, stream, blocks_per_cu);
    case 4: return LaunchPw<BN, 4>(p, M, x, y, stream, blocks_per_cu);
    case 2: return LaunchPw<BN, 2>(p, M, x, y, stream, blocks_per_cu);
    default: return LaunchPw<BN, 1>(p, M, x, y, stream, blocks_per_cu);
    }
}

template <int BM, int BN, int WM, int WN, int D, int BK, bool UT, bool AW>
int LaunchIgemmT(const mi355x_conv2d_s* p, uint32_t batch, const void* x, void* y, hipStream_t stream);

// uniform-tap variant whenever a k-tile cannot straddle two filter taps; row sums when the weights have a zero point
template <int BM, int BN, int WM, int WN, int D, int BK>
int LaunchIgemm(const mi355x_conv2d_s* p, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    const bool ut = (p->geom.Ci % BK) == 0;
    if (p->zw_neg != 0)
        return ut ? LaunchIgemmT<BM, BN, WM, WN, D, BK, true, true>(p, batch, x, y, stream)
                  : LaunchIgemmT<BM, BN, WM, WN, D, BK, false, true>(p, batch, x, y, stream);
    return ut ? LaunchIgemmT<BM, BN, WM, WN, D, BK, true, false>(p, batch, x, y, stream)
              : LaunchIgemmT<BM, BN, WM, WN, D, BK, false, false>(p, batch, x, y, stream);
}

template <int BM, int BN, int WM, int WN, int D, int BK, bool UT, bool AW>
int LaunchIgemmT(const mi355x_conv2d_s* p, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    const ConvGeom& g = p->geom;
    IgemmArgs a;
    a.x = static_cast<const uint8_t*>(x);
    a.pad16 = p->pad16;
    a.w = p->w_mfma;
    a.ct = ChanTab{p->chan, p->Co_pad};
    a.corr = p->corr;
    a.y = static_cast<uint8_t*>(y);
    const long long M = static_cast<long long>(batch) * g.Ho * g.Wo;
    if (M > 0x7fffffffll / 2) return SetError(MI355X_ERR_UNSUPPORTED, "too many output pixels for one launch (%lld)", M);
    a.M = static_cast<int>(M);
    a.H = g.H; a.W = g.W; a.Ci = g.Ci; a.Ho = g.Ho; a.Wo = g.Wo; a.Co = g.Co;
    a.Kh = g.Kh; a.Kw = g.Kw;
    a.pad_top = g.pad_top; a.pad_left = g.pad_left; a.stride_x = g.stride_x; a.stride_y = g.stride_y;
    a.dil_x = g.dil_x; a.dil_y = g.dil_y;
    a.K_pad = p->K_pad;
    a.unit = (g.Kh == 1 && g.Kw == 1 && g.stride_x == 1 && g.stride_y == 1 && g.pad_top == 0 && g.pad_left == 0 && g.Ho == g.H &&
              g.Wo == g.W) ? 1 : 0;
    if (a.unit) { a.H = 1; a.W = a.M; a.Ho = 1; a.Wo = a.M; }      // one row of M pixels
    a.tiles_m = static_cast<int>((M + BM - 1) / BM);
    a.tiles_n = (g.Co + BN - 1) / BN;
    a.xor_mask = p->xor_mask;
    a.pad_word = p->pad_word;
    a.zw_neg = p->zw_neg;
    a.rowsum_bias = p->rowsum_bias;
    a.rq = p->rq;
    const int nblocks = a.tiles_m * a.tiles_n;
    const int grid = (nblocks + 7) / 8 * 8;
    constexpr int smem = IgemmSmemBytes<BM, BN, BK>();
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&IgemmKernel<BM, BN, WM, WN, D, BK, UT, AW>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    MI355X_HIP(attr);
    NoteKernel("IgemmKernel<%d, %d, %d, %d, %d, %d, %s, %s>", BM, BN, WM, WN, D, BK, BoolName(UT), BoolName(AW));
    hipLaunchKernelGGL((IgemmKernel<BM, BN, WM, WN, D, BK, UT, AW>), dim3(grid), dim3(256), smem, stream, a);
    MI355X_HIP(hipGetLastError());
    return 0;
}

template <int BM, int BN, int WM, int WN, int ST, bool U8, bool AW>
int LaunchIgemmLdsT(const mi355x_conv2d_s* p, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    IgemmArgs a;
    bool unit_fast = false;
    if (const int rc = FillIgemmLdsArgs(p, BM, BN, batch, x, y, &a, &unit_fast)) return rc;
    const ConvGeom& g = p->geom;
    if (t_pending_add && (g.Co & 15) == 0)
    {
        a.res = t_pending_add->other;
        a.add = t_pending_add->fuse;
        t_pending_add->taken = true;
    }
    // XCD groups over the output channels where the weights outweigh a quarter of the activations a launch reads ("igemm_xcd_cols":
    // 0 that rule, 1 never, 2 wherever the column tiles halve)
    const long long w_bytes = static_cast<long long>(p->Co_pad) * a.K_pad, x_bytes = static_cast<long long>(a.M) * a.K_pad;
    const int split = p->opt_xcd_cols;
    if ((a.tiles_n & 1) == 0 && a.tiles_m >= 4 && (split == 2 || (split == 0 && 4 * w_bytes > x_bytes))) a.xcd_cols = 2;
    const int grid = 8 * IgemmLdsBlocksPerXcd(a.tiles_m, a.tiles_n, a.xcd_cols);
    constexpr int smem = IgemmLdsSmemBytes<BM, BN, ST>();
    if constexpr (BM == 64 && BN == 64 && !AW)
    {
        // pointwise layers and FullyConnected below 2 GiB per tensor: addresses without per-load vector arithmetic
        if (unit_fast)
        {
            static const hipError_t uattr = hipFuncSetAttribute(reinterpret_cast<const void*>(&IgemmLdsKernel<BM, BN, WM, WN, ST, U8, false, true>),
                                                                hipFuncAttributeMaxDynamicSharedMemorySize, smem);
            MI355X_HIP(uattr);
            NoteKernel("IgemmLdsKernel<%d, %d, %d, %d, %d, %s, false, true>", BM, BN, WM, WN, ST, BoolName(U8));
            hipLaunchKernelGGL((IgemmLdsKernel<BM, BN, WM, WN, ST, U8, false, true>), dim3(grid), dim3(64 * WM * WN), smem, stream, a);
            MI355X_HIP(hipGetLastError());
            return 0;
        }
    }
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&IgemmLdsKernel<BM, BN, WM, WN, ST, U8, AW>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    MI355X_HIP(attr);
    NoteKernel("IgemmLdsKernel<%d, %d, %d, %d, %d, %s, %s, false>", BM, BN, WM, WN, ST, BoolName(U8), BoolName(AW));
    hipLaunchKernelGGL((IgemmLdsKernel<BM, BN, WM, WN, ST, U8, AW>), dim3(grid), dim3(64 * WM * WN), smem, stream, a);
    MI355X_HIP(hipGetLastError());
    return 0;
}

// 64 x 64 tiles with K split over KG groups of four waves inside the block (weights without a zero point)
template <int KG, int ST, bool U8>
int LaunchIgemmKSplitT(const mi355x_conv2d_s* p, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    const ConvGeom& g = p->geom;
    IgemmArgs a;
    a.x = static_cast<const uint8_t*>(x);
    a.pad16 = p->pad16;
    a.w = p->w_mfma;
    a.ct = ChanTab{p->chan, p->Co_pad};
    a.corr = p->corr;
    a.y = static_cast<uint8_t*>(y);
    const long long M = static_cast<long long>(batch) * g.Ho * g.Wo;
    if (M > 0x7fffffffll / 2) return SetError(MI355X_ERR_UNSUPPORTED, "too many output pixels for one launch (%lld)", M);
    a.M = static_cast<int>(M);
    a.H = g.H; a.W = g.W; a.Ci = g.Ci; a.Ho = g.Ho; a.Wo = g.Wo; a.Co = g.Co;
    a.Kh = g.Kh; a.Kw = g.Kw;
    a.pad_top = g.pad_top; a.pad_left = g.pad_left; a.stride_x = g.stride_x; a.stride_y = g.stride_y;
    a.dil_x = g.dil_x; a.dil_y = g.dil_y;
    a.K_pad = p->K_pad;
    a.unit = (g.Kh == 1 && g.Kw == 1 && g.stride_x == 1 && g.stride_y == 1 && g.pad_top == 0 && g.pad_left == 0 && g.Ho == g.H &&
              g.Wo == g.W) ? 1 : 0;
    if (a.unit) { a.H = 1; a.W = a.M; a.Ho = 1; a.Wo = a.M; }      // one row of M pixels
    a.tiles_m = static_cast<int>((M + 63) / 64);
    a.tiles_n = (g.Co + 63) / 64;
    a.xor_mask = p->xor_mask;
    a.pad_word = p->pad_word;
    a.zw_neg = 0;
    a.rowsum_bias = 0;
    a.rq = p->rq;
    const int nblocks = a.tiles_m * a.tiles_n;
    const int grid = (nblocks + 7) / 8 * 8;
    constexpr int smem = IgemmKSplitSmemBytes<KG, ST>();
    static_assert(smem <= 160 * 1024, "LDS of one CU");
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&IgemmKSplitKernel<KG, ST, U8>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    MI355X_HIP(attr);
    NoteKernel("IgemmKSplitKernel<%d, %d, %s>", KG, ST, BoolName(U8));
    hipLaunchKernelGGL((IgemmKSplitKernel<KG, ST, U8>), dim3(grid), dim3(256 * KG), smem, stream, a);
    MI355X_HIP(hipGetLastError());
    return 0;
}

int LaunchIgemmKSplit(const mi355x_conv2d_s* p, int kg, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    const bool u8 = p->xor_mask != 0;
    if (kg == 4) return u8 ? LaunchIgemmKSplitT<4, 2, true>(p, batch, x, y, stream) : LaunchIgemmKSplitT<4, 2, false>(p, batch, x, y, stream);
    return u8 ? LaunchIgemmKSplitT<2, 3, true>(p, batch, x, y, stream) : LaunchIgemmKSplitT<2, 3, false>(p, batch, x, y, stream);
}

// the large-tile kernel of big_gemm.hip (one wave per SIMD, accumulators in AGPRs)
int LaunchBig(const mi355x_conv2d_s* p, int bm, int bn, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    const ConvGeom& g = p->geom;
    IgemmArgs a;
    a.x = static_cast<const uint8_t*>(x);
    a.pad16 = p->pad16;
    a.w = p->w_mfma;
    a.ct = ChanTab{p->chan, p->Co_pad};
    a.corr = p->corr;
    a.y = static_cast<uint8_t*>(y);
    const long long M = static_cast<long long>(batch) * g.Ho * g.Wo;
    if (M > 0x7fffffffll / 2) return SetError(MI355X_ERR_UNSUPPORTED, "too many output pixels for one launch (%lld)", M);
    if (p->Co_pad % bn != 0) return SetError(MI355X_ERR_UNSUPPORTED, "large-tile GEMM: %d padded channels are not whole %d-wide tiles", p->Co_pad, bn);
    a.M = static_cast<int>(M);
    a.H = g.H; a.W = g.W; a.Ci = g.Ci; a.Ho = g.Ho; a.Wo = g.Wo; a.Co = g.Co;
    a.Kh = g.Kh; a.Kw = g.Kw;
    a.pad_top = g.pad_top; a.pad_left = g.pad_left; a.stride_x = g.stride_x; a.stride_y = g.stride_y;
    a.dil_x = g.dil_x; a.dil_y = g.dil_y;
    a.K_pad = p->K_pad;
    a.unit = (g.Kh == 1 && g.Kw == 1 && g.stride_x == 1 && g.stride_y == 1 && g.pad_top == 0 && g.pad_left == 0 && g.Ho == g.H &&
              g.Wo == g.W) ? 1 : 0;
    if (a.unit) { a.H = 1; a.W = a.M; a.Ho = 1; a.Wo = a.M; }      // one row of M pixels
    a.tiles_m = 0; a.tiles_n = 0;                                  // the launcher fills them in
    a.xor_mask = p->xor_mask;
    a.pad_word = p->pad_word;
    a.zw_neg = p->zw_neg;
    a.rowsum_bias = p->rowsum_bias;
    a.rq = p->rq;
    return LaunchBigGemm(a, bm, bn, stream);
}

template <int BM, int BN, int WM, int WN>
int LaunchIgemmLds(const mi355x_conv2d_s* p, int stages, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    const bool u8 = p->xor_mask != 0;
    if constexpr (3 * (BM + BN) * 128 <= 160 * 1024)
    {
        if (stages == 3)
        {
            if (p->zw_neg != 0)
                return u8 ? LaunchIgemmLdsT<BM, BN, WM, WN, 3, true, true>(p, batch, x, y, stream) : LaunchIgemmLdsT<BM, BN, WM, WN, 3, false, true>(p, batch, x, y, stream);
            return u8 ? LaunchIgemmLdsT<BM, BN, WM, WN, 3, true, false>(p, batch, x, y, stream) : LaunchIgemmLdsT<BM, BN, WM, WN, 3, false, false>(p, batch, x, y, stream);
        }
    }

    if (p->zw_neg != 0)
        return u8 ? LaunchIgemmLdsT<BM, BN, WM, WN, 2, true, true>(p, batch, x, y, stream) : LaunchIgemmLdsT<BM, BN, WM, WN, 2, false, true>(p, batch, x, y, stream);
    return u8 ? LaunchIgemmLdsT<BM, BN, WM, WN, 2, true, false>(p, batch, x, y, stream) : LaunchIgemmLdsT<BM, BN, WM, WN, 2, false, false>(p, batch, x, y, stream);
}

// set around a call of LaunchHalo that only asks whether the kernel would take the launch
thread_local bool t_halo_probe = false;

template <int CI, int WM, int WN, int TP, int ST, bool U8>
int LaunchHaloT(const HaloArgs& a, int smem, hipStream_t stream)
{
    if (t_halo_probe) return 0;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&HaloConvKernel<CI, WM, WN, TP, ST, U8>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    MI355X_HIP(attr);
    NoteKernel("HaloConvKernel<%d, %d, %d, %d, %d, %s>", CI, WM, WN, TP, ST, BoolName(U8));
    const int nblocks = a.tiles_m * a.tiles_n;
    hipLaunchKernelGGL((HaloConvKernel<CI, WM, WN, TP, ST, U8>), dim3((nblocks + 7) / 8 * 8), dim3(256), smem, stream, a);
    MI355X_HIP(hipGetLastError());
    return 0;
}

template <int CI, int WM, int WN, int TP>
int LaunchHaloC(HaloArgs& a, const mi355x_conv2d_s* p, uint32_t batch, hipStream_t stream)
{
    constexpr int BN = 32 * WN, MF = WM * TP;
    const ConvGeom& g = p->geom;
    // as many whole output rows as fit the block's pixel fragments and, with the weight stages, LDS
    int R = std::min(g.Ho, (32 * MF) / g.Wo);
    auto smem_of = [&](int rows, int st) {
        const int hp = (rows + g.Kh - 1) * (g.Wo + g.Kw - 1);
        return st == 3 ? HaloSmemBytes<CI, BN, MF, 3>(hp) : HaloSmemBytes<CI, BN, MF, 2>(hp);
    };
    while (R > 1 && smem_of(R, 2) > 160 * 1024) --R;
    if (R < 1 || smem_of(R, 2) > 160 * 1024) return -1;
    a.R = R;
    a.tiles_y = (g.Ho + R - 1) / R;
    a.tiles_m = static_cast<int>(batch) * a.tiles_y;
    a.tiles_n = (g.Co + BN - 1) / BN;
    a.WP = g.Wo + g.Kw - 1;
    a.HP = (R + g.Kh - 1) * a.WP;
    a.wo_magic = static_cast<uint32_t>((0x100000000ull + g.Wo - 1) / g.Wo);
    a.wp_magic = static_cast<uint32_t>((0x100000000ull + a.WP - 1) / a.WP);
    const long long blocks = static_cast<long long>(a.tiles_m) * a.tiles_n;
    // a block is one long dependent chain (tile, k-loop, epilogue): with fewer blocks than CUs the implicit GEMM's smaller
    // tiles finish sooner
    if (blocks < 192 && !(p->tile_override == 3000 || p->tile_override == 3001)) return -1;
    // three weight stages unless two let every block of the launch be resident at once and three do not
    auto resident = [&](int st) { return 256ll * std::min(4, (160 * 1024) / smem_of(R, st)); };
    const bool three = smem_of(R, 3) <= 160 * 1024 && !(blocks > resident(3) && blocks <= resident(2));
    const bool u8 = p->xor_mask != 0;
    if (three) return u8 ? LaunchHaloT<CI, WM, WN, TP, 3, true>(a, smem_of(R, 3), stream) : LaunchHaloT<CI, WM, WN, TP, 3, false>(a, smem_of(R, 3), stream);
    return u8 ? LaunchHaloT<CI, WM, WN, TP, 2, true>(a, smem_of(R, 2), stream) : LaunchHaloT<CI, WM, WN, TP, 2, false>(a, smem_of(R, 2), stream);
}

// Returns -1 when the shape does not fit after all (the caller then takes the implicit GEMM).
int LaunchHalo(const mi355x_conv2d_s* p, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    const ConvGeom& g = p->geom;
    HaloArgs a;
    a.x = static_cast<const uint8_t*>(x);
    a.pad16 = p->pad16;
    a.w = p->w_mfma;
    a.ct = ChanTab{p->chan, p->Co_pad};
    a.corr = p->corr;
    a.y = static_cast<uint8_t*>(y);
    a.H = g.H; a.W = g.W; a.Ho = g.Ho; a.Wo = g.Wo; a.Co = g.Co;
    a.Kh = g.Kh; a.Kw = g.Kw;
    a.pad_top = g.pad_top; a.pad_left = g.pad_left;
    a.K_pad = p->K_pad;
    a.xor_mask = p->xor_mask;
    a.rq = p->rq;
    const bool wide = g.Co > 64;
    switch (g.Ci)
    {
    case 64:
    {
        // narrow output: half-height tiles (128 pixels) while the full ones would leave at most one block per CU
        const int r4 = std::max(1, std::min(g.Ho, 256 / std::max(1, g.Wo)));
        const long long blocks4 = static_cast<long long>(batch) * ((g.Ho + r4 - 1) / r4);
        if (!wide && g.Wo <= 128 && (p->tile_override == 3001 || (p->tile_override == 0 && blocks4 <= 256))) return LaunchHaloC<64, 2, 2, 2>(a, p, batch, stream);
        return wide ? LaunchHaloC<64, 1, 4, 7>(a, p, batch, stream) : LaunchHaloC<64, 2, 2, 4>(a, p, batch, stream);
    }
    case 128: return wide ? LaunchHaloC<128, 1, 4, 7>(a, p, batch, stream) : LaunchHaloC<128, 2, 2, 4>(a, p, batch, stream);
    case 256: return wide ? LaunchHaloC<256, 1, 4, 7>(a, p, batch, stream) : LaunchHaloC<256, 2, 2, 4>(a, p, batch, stream);
    default: return -1;
    }
}

// ---- 3x3 depthwise on the matrix cores -------------------------------------------------------------------------------
// Tile height (outputs) for an Ho x Wo map: 16 or 14 (16 columns) or 8 or 7 (8 columns) at stride 1, 8 or 7 at stride 2
// (the halo of a 16-column tile at stride 2 would not fit LDS).  The one that leaves the least padded work, ties to the
// earlier entry.
int ChooseDwMfmaTile(int stride, int Ho, int Wo, int forced)
{
    static const int kS1[] = {16, 14, 7, 8}, kS2[] = {7, 8};
    const int* menu = stride == 1 ? kS1 : kS2;
    const int count = stride == 1 ? 4 : 2;
    int best = menu[0];
    long long best_cost = -1;
    for (int i = 0; i < count; ++i)
    {
        const int th = menu[i], tw = th >= 14 ? 16 : 8;
        if (forced == th) return th;
        const long long cost = static_cast<long long>((Ho + th - 1) / th) * ((Wo + tw - 1) / tw) * ((th * tw + 15) / 16) * 16;
        if (best_cost < 0 || cost < best_cost) { best_cost = cost; best = th; }
    }
    return best;
}

int DeviceCuCount()
{
    static const int n = []() {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 8) return 256;
        return cus;
    }();
    return n;
}

template <int S, bool W2, int CB, int T>
int LaunchDwMfmaT(const Dw3x3Args& a, hipStream_t stream)
{
    constexpr int TW = T >= 14 ? 16 : 8;
    using G = DwMfmaTile<S, CB, T, TW>;
    constexpr int smem = G::SMEM;
    const auto kernel = &DepthwiseMfmaKernel<S, W2, CB, T, TW>;
    // blocks that fit a CU at once (LDS, registers), asked once per kernel
    static const int per_cu = [&]() {
        int n = 0;
        if (smem > 48 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, smem) != hipSuccess) return 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, G::NT, smem) != hipSuccess) return 0;
        return n;
    }();
    if (per_cu <= 0) { (void)hipGetLastError(); return SetError(MI355X_ERR_UNSUPPORTED, "depthwise kernel: no block fits a CU"); }
    // As many blocks per XCD as run at once; each walks its share of the XCD's items with the next item's loads in flight.
    // A stride between a block's items that is a multiple of the channel blocks keeps its weights in registers.
    int per_xcd = per_cu * (DeviceCuCount() / 8);
    if (per_xcd >= a.xcd_chunk) per_xcd = a.xcd_chunk;
    else if (per_xcd > a.cblocks) per_xcd -= per_xcd % a.cblocks;
    NoteKernel("DepthwiseMfmaKernel<%d, %s, %d, %d, %d>", S, BoolName(W2), CB, T, TW);
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(per_xcd) * 8u), dim3(G::NT), smem, stream, a);
    return 0;
}

template <int S, bool W2, int CB>
int LaunchDwMfmaTile(int tile, const Dw3x3Args& a, hipStream_t stream)
{
    if (tile == 7) return LaunchDwMfmaT<S, W2, CB, 7>(a, stream);
    return LaunchDwMfmaT<S, W2, CB, 8>(a, stream);
}

template <int S, bool W2>
int LaunchDwMfmaCb(int cbw, int tile, const Dw3x3Args& a, hipStream_t stream)
{
    if constexpr (S == 1)
    {
        if (tile == 16) return LaunchDwMfmaT<S, W2, 32, 16>(a, stream);
        if (tile == 14) return LaunchDwMfmaT<S, W2, 32, 14>(a, stream);
    }
    if (cbw == 64) return LaunchDwMfmaTile<S, W2, 64>(tile, a, stream);
    return LaunchDwMfmaTile<S, W2, 32>(tile, a, stream);
}

// Whether the matrix-core kernel takes this launch (else the VALU kernel does): tensors it can address with 32-bit offsets
// within an image, 16-byte aligned, and an item count its reciprocal decoding is exact for.
bool DwMfmaTakes(const mi355x_conv2d_s* p, uint32_t batch, const void* x, const void* y)
{
    const ConvGeom& g = p->geom;
    if (p->opt_dw_mfma == 0) return false;
    if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) != 0) return false;
    if (static_cast<long long>(g.Ho) * g.Wo * g.Co >= 0x40000000ll || static_cast<long long>(g.H) * g.W * g.Co >= 0x40000000ll) return false;
    // items at the smallest tile and channel block, times the largest divisor, stays below 2^32
    const long long items = static_cast<long long>(batch) * ((g.Ho + 6) / 7) * ((g.Wo + 7) / 8) * ((g.Co + 31) / 32);
    const long long divisor = std::max<long long>({(g.Ho + 6) / 7, (g.Wo + 7) / 8, (g.Co + 31) / 32});
    return items < 0x7fffffffll - 8 && items * divisor < 0xffffffffll;
}

// `a`: as filled for the VALU kernel; the tiling is replaced.
int LaunchDwMfma(const mi355x_conv2d_s* p, Dw3x3Args a, hipStream_t stream)
{
    const ConvGeom& g = p->geom;
    const int tile = ChooseDwMfmaTile(g.stride_x, g.Ho, g.Wo, p->opt_dw_mfma);
    const int tw = tile >= 14 ? 16 : 8;
    // 64 channels per block (one wave per group of 16) where the count allows; the 16-column tiles take 32 (two waves per
    // group): with 64 their halo buffers would leave two blocks per CU
    const int cbw = tw == 16 || (g.Co % 64) != 0 || p->opt_dw_cb == 32 ? 32 : 64;
    a.cblocks = (g.Co + cbw - 1) / cbw;
    a.tiles_x = (g.Wo + tw - 1) / tw; a.tiles_y = (g.Ho + tile - 1) / tile;
    const long long nb = static_cast<long long>(a.N) * a.tiles_x * a.tiles_y * a.cblocks;
    a.total_blocks = static_cast<int>(nb);
    a.xcd_chunk = static_cast<int>((nb + 7) / 8);
    const auto rcp = [](int d) { return d <= 1 ? 0u : static_cast<uint32_t>((0x100000000ull + static_cast<unsigned>(d) - 1) / static_cast<unsigned>(d)); };
    a.rcp_cblocks = rcp(a.cblocks); a.rcp_tiles_x = rcp(a.tiles_x); a.rcp_tiles_y = rcp(a.tiles_y);
    const bool w2 = p->w_dot4b != nullptr;
    int rc;
    if (g.stride_x == 1) rc = w2 ? LaunchDwMfmaCb<1, true>(cbw, tile, a, stream) : LaunchDwMfmaCb<1, false>(cbw, tile, a, stream);
    else rc = w2 ? LaunchDwMfmaCb<2, true>(cbw, tile, a, stream) : LaunchDwMfmaCb<2, false>(cbw, tile, a, stream);
    if (rc != 0) return rc;
    MI355X_HIP(hipGetLastError());
    return 0;
}

int RunPlan(const mi355x_conv2d_s* p, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    if (!p) return SetError(MI355X_ERR_INVALID_ARGUMENT, "plan is null");
    if (batch == 0) return 0;
    if (!x || !y) return SetError(MI355X_ERR_INVALID_ARGUMENT, "input / output pointer is null");
    const ConvGeom& g = p->geom;
    const long long total = static_cast<long long>(batch) * g.Ho * g.Wo * g.Co;
    const uint8_t* xin = static_cast<const uint8_t*>(x);
    uint8_t* yout = static_cast<uint8_t*>(y);
    switch (p->algo)
    {
    case MI355X_ALGO_MFMA:
        if ((reinterpret_cast<uintptr_t>(x) & 15) != 0 || ((g.Co & 15) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) != 0))
            return SetError(MI355X_ERR_INVALID_ARGUMENT, "MFMA kernel needs 16-byte aligned tensors");
    {
        const mi355x_conv2d_desc& dd = p->d;
        const long long rows = static_cast<long long>(batch) * g.Ho * g.Wo;
        const bool unit = dd.kernel_h == 1 && dd.kernel_w == 1 && dd.stride_x == 1 && dd.stride_y == 1 && dd.pad_top == 0 &&
                          dd.pad_left == 0 && dd.out_h == dd.in_h && dd.out_w == dd.in_w;
        if (unit && rows <= 4 && (g.Ci % 16) == 0 && p->tile_override == 0)
        {
            // a handful of rows: stream the weights once, no tiles
            GemvArgs a;
            a.x = xin; a.w = p->w_mfma; a.ct = ChanTab{p->chan, p->Co_pad}; a.corr = p->corr; a.y = yout;
            a.M = static_cast<int>(rows); a.K = g.Ci; a.N = g.Co; a.w_stride = p->K_pad; a.xor_mask = p->xor_mask; a.zw_neg = p->zw_neg; a.rq = p->rq;
            const dim3 grid(static_cast<unsigned>((g.Co + 15) / 16));
            NoteKernel("GemvKernel<%d>", a.M);
            switch (a.M)
            {
                case 1: hipLaunchKernelGGL(GemvKernel<1>, grid, dim3(256), 0, stream, a); break;
                case 2: hipLaunchKernelGGL(GemvKernel<2>, grid, dim3(256), 0, stream, a); break;
                case 3: hipLaunchKernelGGL(GemvKernel<3>, grid, dim3(256), 0, stream, a); break;
                default: hipLaunchKernelGGL(GemvKernel<4>, grid, dim3(256), 0, stream, a); break;
            }
            MI355X_HIP(hipGetLastError());
            return 0;
        }
        if (unit && rows <= 64 && (g.Ci % 16) == 0 && g.Ci >= 128 && p->tile_override == 0 && p->Co_pad >= (g.Co + 31) / 32 * 32 &&
            (reinterpret_cast<uintptr_t>(y) & 3) == 0)
        {
            // a few dozen rows: 32x32 tiles with K split over the block's waves
            GemvArgs a;
            a.x = xin; a.w = p->w_mfma; a.ct = ChanTab{p->chan, p->Co_pad}; a.corr = p->corr; a.y = yout;
            a.M = static_cast<int>(rows); a.K = g.Ci; a.N = g.Co; a.w_stride = p->K_pad; a.xor_mask = p->xor_mask; a.zw_neg = p->zw_neg; a.rq = p->rq;
            const dim3 grid(static_cast<unsigned>((g.Co + 31) / 32), static_cast<unsigned>((rows + 31) / 32));
            NoteKernel("SmallMGemmKernel<%d>", g.Ci <= 512 ? 4 : 8);
            if (g.Ci <= 512) hipLaunchKernelGGL(SmallMGemmKernel<4>, grid, dim3(256), 0, stream, a);
            else hipLaunchKernelGGL(SmallMGemmKernel<8>, grid, dim3(256), 0, stream, a);
            MI355X_HIP(hipGetLastError());
            return 0;
        }
        if (p->pw_bn)
        {
            const long long Mrows = static_cast<long long>(batch) * g.Ho * g.Wo;
            if (Mrows > 0x7fffffffll / 2) return SetError(MI355X_ERR_UNSUPPORTED, "too many rows for one launch (%lld)", Mrows);
            // 128-channel slabs give way to 64-channel ones where another lane's launches share the device: the smaller blocks
            // fill the gaps of the neighbour's (ResNet-50 b32 in two lanes, the four 128 -> 512 layers: 0.7065 -> 0.7031 ms per
            // step; alone on the device the wide slab is the faster one, 8.2 against 8.6 us)
            if (p->pw_bn == 128 && p->concurrency > 1 && p->pw_blocks_per_cu_64 > 0) return LaunchPwKs<64>(p, Mrows, x, y, stream, p->pw_blocks_per_cu_64);
            if (p->pw_bn == 128) return LaunchPwKs<128>(p, Mrows, x, y, stream, p->pw_blocks_per_cu);
            if (p->pw_bn == 64) return LaunchPwKs<64>(p, Mrows, x, y, stream, p->pw_blocks_per_cu);
            return LaunchPwKs<32>(p, Mrows, x, y, stream, p->pw_blocks_per_cu);
        }
        // Small filters at stride 1 over 64 / 128 / 256 channels: the input tile stays in LDS for all taps
        // -- unless the launch shares the device with another lane's launches: a block of that kernel holds a whole input
        // tile in LDS, few of them fit a CU, and beside a neighbour the implicit GEMM with 128 x 64 tiles is the faster
        // choice (ResNet-50 b32 in two lanes: 13.7 us per step for its three 3 x 3 x 64 layers; alone the kernel below
        // wins).  Measured for the 64-channel form only.
        const bool shared_device = p->concurrency > 1 && p->tile_override == 0;
        bool gemm_instead = false;
        if (p->halo_ok && p->zw_neg == 0 && p->opt_igemm_lds != 0 && (p->tile_override == 0 || (p->tile_override == 3000 || p->tile_override == 3001)))
        {
            // ... and only where the 128 x 64 tiles still give every CU a block
            const long long gemm_blocks = ((static_cast<long long>(batch) * g.Ho * g.Wo + 127) / 128) * ((g.Co + 63) / 64);
            if (shared_device && g.Ci == 64 && gemm_blocks >= 256)
            {
                t_halo_probe = true;
                gemm_instead = LaunchHalo(p, batch, x, y, stream) >= 0;
                t_halo_probe = false;
            }
            if (!gemm_instead)
            {
                const int rc = LaunchHalo(p, batch, x, y, stream);
                if (rc >= 0) return rc;
            }
        }
        // Tile choice: the large tile has the best MFMA : LDS-traffic ratio, but a launch needs several blocks per CU
        // in flight to hide global-load latency, so problems that would yield few large tiles take 64x64 tiles
        // (4x the blocks, 8 waves/SIMD).
        const long long M = static_cast<long long>(batch) * g.Ho * g.Wo;
        const long long big = ((M + 127) / 128) * ((g.Co + 127) / 128);
        // tile: 64x64 while the 128-wide tiling would leave CUs idle; k-tile: 128 bytes whenever K was padded to it
        const bool bk128 = p->bk128;
        // 256x256 tiles (16 waves) halve the operand traffic per output once they alone fill three quarters of the CUs
        const long long huge = ((M + 255) / 256) * ((g.Co + 255) / 256);
        const int tile = p->tile_override ? p->tile_override
                       : gemm_instead ? 96
                       : big < 400 ? 64 : (huge >= 192 && g.Co >= 256) ? 512 : 128;
        // channel counts that are multiples of 128: k-tiles go from global memory straight into LDS
        const int lds_stages = p->opt_igemm_lds;
        if (lds_stages != 0 && bk128 && (g.Ci % 128) == 0)
        {
            // Launches that fill the device with 256-row tiles: one wave per SIMD with a 128 x 128 (or 128 x 64) wave tile.
            // A CU's L1 delivers 30 to 45 bytes per clock from L2; only these tiles ask for less than that per MFMA clock.
            if (p->tile_override == 0 || p->tile_override >= 1000)
            {
                const long long rows256 = (M + 255) / 256;
                int bm = 0, bn = 0;
                if (p->tile_override == 2256) { bm = 256; bn = 256; }
                else if (p->tile_override == 2128) { bm = 256; bn = 128; }
                else if (p->tile_override == 1256) { bm = 128; bn = 256; }
                else if ((p->Co_pad % 256) == 0 && rows256 * (p->Co_pad / 256) >= 224) { bm = 256; bn = 256; }
                else if (rows256 * (p->Co_pad / 128) >= 224) { bm = 256; bn = 128; }
                // the large-tile kernel walks a filter's taps through a 32-bit mask per row: filters of more than 32 taps
                // (6 x 6, 7 x 7 ...) stay on the tiles below, also when a test forces the large tile
                if (bm != 0 && (unit || g.Kh * g.Kw <= 32)) return LaunchBig(p, bm, bn, batch, x, y, stream);
            }
            if ((tile == 4064 || tile == 2064) && p->zw_neg == 0) return LaunchIgemmKSplit(p, tile == 4064 ? 4 : 2, batch, x, y, stream);
            if (tile == 64 && p->tile_override == 0 && p->zw_neg == 0 && p->K_pad >= 16 * 128)
            {
                // At most one block per CU and a long K: a SIMD would hold one wave and the k-loop run at that wave's issue
                // rate.  K split over groups of waves inside the block: 17.4 -> 13.5 us for 7 x 7 x 512 -> 512, 3 x 3, 16 images.
                const long long blocks64 = ((M + 63) / 64) * ((g.Co + 63) / 64);
                if (blocks64 <= 128) return LaunchIgemmKSplit(p, 4, batch, x, y, stream);
                // two groups: only when the launch has the device to itself (beside another lane's launches the plain
                // 64 x 64 blocks of 256 threads co-run better: ResNet-50 b32 in two lanes, 6.3 us per step for five layers)
                if (blocks64 <= 256 && !shared_device) return LaunchIgemmKSplit(p, 2, batch, x, y, stream);
            }
            if (tile == 64)
            {
                // at most one block per CU: nothing else hides a k-tile's round trip, so keep two tiles on their way
                const long long blocks64 = ((M + 63) / 64) * ((g.Co + 63) / 64);
                return LaunchIgemmLds<64, 64, 2, 2>(p, (lds_stages == 2 && blocks64 <= 256) ? 3 : lds_stages, batch, x, y, stream);
            }
            if (g.Co <= 64 || tile == 96) return LaunchIgemmLds<128, 64, 2, 2>(p, lds_stages, batch, x, y, stream);
            if (tile == 256) return LaunchIgemmLds<256, 128, 4, 2>(p, lds_stages, batch, x, y, stream);
            if (tile == 512) return LaunchIgemmLds<256, 256, 4, 4>(p, lds_stages, batch, x, y, stream);
            return LaunchIgemmLds<128, 128, 2, 2>(p, lds_stages, batch, x, y, stream);
        }
        if (tile == 64) return bk128 ? LaunchIgemm<64, 64, 2, 2, 2, 128>(p, batch, x, y, stream) : LaunchIgemm<64, 64, 2, 2, 2, 64>(p, batch, x, y, stream);
        if (g.Co <= 64 || tile == 96) return bk128 ? LaunchIgemm<128, 64, 2, 2, 2, 128>(p, batch, x, y, stream) : LaunchIgemm<128, 64, 2, 2, 2, 64>(p, batch, x, y, stream);
        return bk128 ? LaunchIgemm<128, 128, 2, 2, 2, 128>(p, batch, x, y, stream) : LaunchIgemm<128, 128, 2, 2, 2, 64>(p, batch, x, y, stream);
    }
    case MI355X_ALGO_DOT4:
    {
        if ((reinterpret_cast<uintptr_t>(y) & 3) != 0) return SetError(MI355X_ERR_INVALID_ARGUMENT, "dot4 kernel needs a 4-byte aligned output");
        SmallCiArgs a;
        a.x = xin; a.wpack = p->w_dot4; a.ct = ChanTab{p->chan, p->Co_pad}; a.corr = p->corr; a.y = yout;
        a.N = static_cast<int>(batch); a.H = g.H; a.W = g.W; a.Ci = g.Ci; a.Ho = g.Ho; a.Wo = g.Wo; a.Co = g.Co;
        a.Kw = g.Kw; a.stride = g.stride_x; a.pad_top = g.pad_top; a.pad_left = g.pad_left;
        a.tiles_x = (g.Wo + 31) / 32; a.tiles_y = (g.Ho + 15) / 16;
        a.xor_mask = p->xor_mask; a.pad_byte = p->pad_word;
        // LDS row: up to 3 bytes of misalignment, 31 pixel steps, one pixel's row of RD dwords, one spare dword
        a.lp = ((3 + 31 * g.stride_x * g.Ci + 4 * p->row_dwords + 3) & ~3) + 8;
        a.ndw_recip = static_cast<uint32_t>((0x100000000ull + static_cast<unsigned long long>(a.lp / 4) - 1ull) / static_cast<unsigned long long>(a.lp / 4));
        a.vec16 = ((reinterpret_cast<uintptr_t>(y) & 15) == 0 && (g.Co % 16) == 0) ? 1 : 0;
        // 16-byte staging when every halo row starts on a 16-byte boundary and image rows are whole chunks
        a.pad16 = p->pad16;
        a.vec_stage = ((g.W * g.Ci) % 16 == 0 && (static_cast<long long>(g.H) * g.W * g.Ci) % 16 == 0 && g.pad_left == 0 &&
                       (32 * g.stride_x * g.Ci) % 16 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) ? 1 : 0;
        if (a.vec_stage) a.lp = (31 * g.stride_x * g.Ci + 4 * p->row_dwords + 4 + 15) / 16 * 16;
        a.nch_recip = static_cast<uint32_t>((0x100000000ull + static_cast<unsigned long long>(a.lp / 16) - 1ull) / static_cast<unsigned long long>(std::max(1, a.lp / 16)));
        if (a.lp > 288) return SetError(MI355X_ERR_UNSUPPORTED, "dot4 kernel: halo row of %d bytes does not fit", a.lp);
        if (static_cast<long long>(g.H) * g.W * g.Ci >= (1ll << 30)) return SetError(MI355X_ERR_UNSUPPORTED, "dot4 kernel: image too large for 32-bit offsets");
        a.rq = p->rq;
        a.w_mfma = p->w_stem; a.w_mfma2 = p->w_stem2; a.kp = p->stem_kp;
        if (p->w_stem && !p->opt_stem_dot4 && (g.Kh == 3 || g.Kh == 7))
        {
            long long nbm = static_cast<long long>(batch) * a.tiles_x * a.tiles_y;
            if (nbm > 0x7fffffffll) return SetError(MI355X_ERR_UNSUPPORTED, "grid too large");
            // 8-row tiles while the 16-row ones would give a CU fewer than three blocks: a block is one dependent chain of
            // staging, gather, MFMA and requantization, and with one or two per CU nothing runs beside it
            const bool th8 = !p->w_stem2 && nbm < 768;
            if (th8)
            {
                a.tiles_y = (g.Ho + 7) / 8;
                nbm = static_cast<long long>(batch) * a.tiles_x * a.tiles_y;
            }
            const dim3 gridm(static_cast<unsigned>(nbm));
            NoteKernel("SmallCiMfmaKernel<%d, %d, %d, %d, %s>", g.Kh, g.Kh == 3 ? 3 : 6, g.Co == 32 ? 1 : 2, th8 ? 8 : 16, BoolName(p->w_stem2 != nullptr));
            if (th8)
            {
                if (g.Kh == 3 && g.Co == 32) hipLaunchKernelGGL((SmallCiMfmaKernel<3, 3, 1, 8>), gridm, dim3(256), 0, stream, a);
                else if (g.Kh == 3) hipLaunchKernelGGL((SmallCiMfmaKernel<3, 3, 2, 8>), gridm, dim3(256), 0, stream, a);
                else if (g.Co == 32) hipLaunchKernelGGL((SmallCiMfmaKernel<7, 6, 1, 8>), gridm, dim3(256), 0, stream, a);
                else hipLaunchKernelGGL((SmallCiMfmaKernel<7, 6, 2, 8>), gridm, dim3(256), 0, stream, a);
            }
            else if (p->w_stem2)
            {
                if (g.Kh == 3 && g.Co == 32) hipLaunchKernelGGL((SmallCiMfmaKernel<3, 3, 1, 16, true>), gridm, dim3(256), 0, stream, a);
                else if (g.Kh == 3) hipLaunchKernelGGL((SmallCiMfmaKernel<3, 3, 2, 16, true>), gridm, dim3(256), 0, stream, a);
                else if (g.Co == 32) hipLaunchKernelGGL((SmallCiMfmaKernel<7, 6, 1, 16, true>), gridm, dim3(256), 0, stream, a);
                else hipLaunchKernelGGL((SmallCiMfmaKernel<7, 6, 2, 16, true>), gridm, dim3(256), 0, stream, a);
            }
            else if (g.Kh == 3 && g.Co == 32) hipLaunchKernelGGL((SmallCiMfmaKernel<3, 3, 1, 16>), gridm, dim3(256), 0, stream, a);
            else if (g.Kh == 3) hipLaunchKernelGGL((SmallCiMfmaKernel<3, 3, 2, 16>), gridm, dim3(256), 0, stream, a);
            else if (g.Co == 32) hipLaunchKernelGGL((SmallCiMfmaKernel<7, 6, 1, 16>), gridm, dim3(256), 0, stream, a);
            else hipLaunchKernelGGL((SmallCiMfmaKernel<7, 6, 2, 16>), gridm, dim3(256), 0, stream, a);
            MI355X_HIP(hipGetLastError());
            return 0;
        }
        const long long nb = static_cast<long long>(batch) * a.tiles_x * a.tiles_y;
        if (nb > 0x7fffffffll) return SetError(MI355X_ERR_UNSUPPORTED, "grid too large");
        const dim3 grid(static_cast<unsigned>(nb));
        a.wpack2 = p->w_dot4b;
        NoteKernel("SmallCiConvKernel<%d, %d, %s>", g.Kh, p->row_dwords, BoolName(p->w_dot4b != nullptr));
        if (p->w_dot4b)
        {
            if (g.Kh == 3) hipLaunchKernelGGL((SmallCiConvKernel<3, 3, true>), grid, dim3(256), 0, stream, a);
            else if (g.Kh == 7) hipLaunchKernelGGL((SmallCiConvKernel<7, 6, true>), grid, dim3(256), 0, stream, a);
            else if (g.Kh == 5) hipLaunchKernelGGL((SmallCiConvKernel<5, 5, true>), grid, dim3(256), 0, stream, a);
            else hipLaunchKernelGGL((SmallCiConvKernel<1, 1, true>), grid, dim3(256), 0, stream, a);
        }
        else if (g.Kh == 3) hipLaunchKernelGGL((SmallCiConvKernel<3, 3>), grid, dim3(256), 0, stream, a);
        else if (g.Kh == 7) hipLaunchKernelGGL((SmallCiConvKernel<7, 6>), grid, dim3(256), 0, stream, a);
        else if (g.Kh == 5) hipLaunchKernelGGL((SmallCiConvKernel<5, 5>), grid, dim3(256), 0, stream, a);
        else hipLaunchKernelGGL((SmallCiConvKernel<1, 1>), grid, dim3(256), 0, stream, a);
        MI355X_HIP(hipGetLastError());
        return 0;
    }
    case MI355X_ALGO_DEPTHWISE:
    {
        if (p->variant == 1)
        {
            if ((reinterpret_cast<uintptr_t>(x) & 15) != 0 || (reinterpret_cast<uintptr_t>(y) & 3) != 0)
                return SetError(MI355X_ERR_INVALID_ARGUMENT, "depthwise 3x3 kernel needs a 16-byte aligned input and 4-byte aligned output");
            Dw3x3Args a;
            int rows_per_thread = 1, cbw = 32;
            if (const int rc = FillDw3x3Args(p, batch, x, y, &a, &rows_per_thread, &cbw)) return rc;
            if (DwMfmaTakes(p, batch, x, y)) return LaunchDwMfma(p, a, stream);
            const bool wide = cbw == 128, mid = cbw == 64;
            const dim3 grid(static_cast<unsigned>(a.xcd_chunk) * 8u);
            const bool w2 = p->w_dot4b != nullptr;
            NoteKernel("Depthwise3x3Kernel<%d, %d, %s, %d>", g.stride_x, rows_per_thread, BoolName(w2), cbw);
            const int variant = (g.stride_x == 1 ? 0 : 4) + (rows_per_thread == 2 ? 0 : 2) + (w2 ? 1 : 0);
            switch (variant + (wide ? 8 : mid ? 16 : 0))
            {
            case 16: hipLaunchKernelGGL((Depthwise3x3Kernel<1, 2, false, 64>), grid, dim3(256), 0, stream, a); break;
            case 17: hipLaunchKernelGGL((Depthwise3x3Kernel<1, 2, true, 64>), grid, dim3(256), 0, stream, a); break;
            case 18: hipLaunchKernelGGL((Depthwise3x3Kernel<1, 1, false, 64>), grid, dim3(256), 0, stream, a); break;
            case 19: hipLaunchKernelGGL((Depthwise3x3Kernel<1, 1, true, 64>), grid, dim3(256), 0, stream, a); break;
            case 20: hipLaunchKernelGGL((Depthwise3x3Kernel<2, 2, false, 64>), grid, dim3(256), 0, stream, a); break;
            case 21: hipLaunchKernelGGL((Depthwise3x3Kernel<2, 2, true, 64>), grid, dim3(256), 0, stream, a); break;
            case 22: hipLaunchKernelGGL((Depthwise3x3Kernel<2, 1, false, 64>), grid, dim3(256), 0, stream, a); break;
            case 23: hipLaunchKernelGGL((Depthwise3x3Kernel<2, 1, true, 64>), grid, dim3(256), 0, stream, a); break;
            case 0: hipLaunchKernelGGL((Depthwise3x3Kernel<1, 2, false>), grid, dim3(256), 0, stream, a); break;
            case 1: hipLaunchKernelGGL((Depthwise3x3Kernel<1, 2, true>), grid, dim3(256), 0, stream, a); break;
            case 2: hipLaunchKernelGGL((Depthwise3x3Kernel<1, 1, false>), grid, dim3(256), 0, stream, a); break;
            case 3: hipLaunchKernelGGL((Depthwise3x3Kernel<1, 1, true>), grid, dim3(256), 0, stream, a); break;
            case 4: hipLaunchKernelGGL((Depthwise3x3Kernel<2, 2, false>), grid, dim3(256), 0, stream, a); break;
            case 5: hipLaunchKernelGGL((Depthwise3x3Kernel<2, 2, true>), grid, dim3(256), 0, stream, a); break;
            case 6: hipLaunchKernelGGL((Depthwise3x3Kernel<2, 1, false>), grid, dim3(256), 0, stream, a); break;
            case 7: hipLaunchKernelGGL((Depthwise3x3Kernel<2, 1, true>), grid, dim3(256), 0, stream, a); break;
            case 8: hipLaunchKernelGGL((Depthwise3x3Kernel<1, 2, false, 128>), grid, dim3(256), 0, stream, a); break;
            case 9: hipLaunchKernelGGL((Depthwise3x3Kernel<1, 2, true, 128>), grid, dim3(256), 0, stream, a); break;
            case 10: hipLaunchKernelGGL((Depthwise3x3Kernel<1, 1, false, 128>), grid, dim3(256), 0, stream, a); break;
            case 11: hipLaunchKernelGGL((Depthwise3x3Kernel<1, 1, true, 128>), grid, dim3(256), 0, stream, a); break;
            case 12: hipLaunchKernelGGL((Depthwise3x3Kernel<2, 2, false, 128>), grid, dim3(256), 0, stream, a); break;
            case 13: hipLaunchKernelGGL((Depthwise3x3Kernel<2, 2, true, 128>), grid, dim3(256), 0, stream, a); break;
            case 14: hipLaunchKernelGGL((Depthwise3x3Kernel<2, 1, false, 128>), grid, dim3(256), 0, stream, a); break;
            default: hipLaunchKernelGGL((Depthwise3x3Kernel<2, 1, true, 128>), grid, dim3(256), 0, stream, a); break;
            }
            MI355X_HIP(hipGetLastError());
            return 0;
        }
        if ((reinterpret_cast<uintptr_t>(x) & 3) != 0 || (reinterpret_cast<uintptr_t>(y) & 3) != 0)
            return SetError(MI355X_ERR_INVALID_ARGUMENT, "depthwise kernel needs 4-byte aligned tensors");
        const long long total4 = total / 4;
        const unsigned blocks = static_cast<unsigned>((total4 + 255) / 256);
        NoteKernel("DepthwiseC4Kernel<%s, %s>", BoolName(g.in_u8), BoolName(g.w_u8));
        if (g.in_u8 && !g.w_u8)
            hipLaunchKernelGGL((DepthwiseC4Kernel<true, false>), dim3(blocks), dim3(256), 0, stream, g, p->rq, xin, p->w_direct, ChanTab{p->chan, p->Co_pad}, yout, total4);
        else if (!g.in_u8 && !g.w_u8)
            hipLaunchKernelGGL((DepthwiseC4Kernel<false, false>), dim3(blocks), dim3(256), 0, stream, g, p->rq, xin, p->w_direct, ChanTab{p->chan, p->Co_pad}, yout, total4);
        else if (g.in_u8 && g.w_u8)
            hipLaunchKernelGGL((DepthwiseC4Kernel<true, true>), dim3(blocks), dim3(256), 0, stream, g, p->rq, xin, p->w_direct, ChanTab{p->chan, p->Co_pad}, yout, total4);
        else
            hipLaunchKernelGGL((DepthwiseC4Kernel<false, true>), dim3(blocks), dim3(256), 0, stream, g, p->rq, xin, p->w_direct, ChanTab{p->chan, p->Co_pad}, yout, total4);
        MI355X_HIP(hipGetLastError());
        return 0;
    }
    default:
    {
        const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
        NoteKernel("ConvDirectKernel<%s>", BoolName(p->d.depthwise != 0));
        if (p->d.depthwise)
            hipLaunchKernelGGL((ConvDirectKernel<true>), dim3(blocks), dim3(256), 0, stream, g, p->rq, xin, p->w_direct, ChanTab{p->chan, p->Co_pad}, yout, total);
        else
            hipLaunchKernelGGL((ConvDirectKernel<false>), dim3(blocks), dim3(256), 0, stream, g, p->rq, xin, p->w_direct, ChanTab{p->chan, p->Co_pad}, yout, total);
        MI355X_HIP(hipGetLastError());
        return 0;
    }
    }
}

} // namespace

namespace
{
template <int S, int P>
int LaunchDwPw(const mi355x_conv2d_s* dw, const mi355x_conv2d_s* pw, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    using G = DwPwGeom<S, P>;
    constexpr int D = 4;
    const ConvGeom& g = dw->geom;
    DwPwArgs a;
    a.x = static_cast<const uint8_t*>(x); a.pad16 = dw->pad16; a.dw_grp = dw->dw_grp; a.dw_ct = ChanTab{dw->chan, dw->Co_pad};
    a.N = static_cast<int>(batch); a.H = g.H; a.W = g.W; a.C = g.Co; a.Ho = g.Ho; a.Wo = g.Wo;
    a.pad_top = g.pad_top; a.pad_left = g.pad_left;
    a.tiles_x = (g.Wo + G::TW - 1) / G::TW; a.tiles_y = (g.Ho + G::TH - 1) / G::TH;
    const long long nb = static_cast<long long>(batch) * a.tiles_x * a.tiles_y;
    if (nb > 0x7fffffffll - 8) return SetError(MI355X_ERR_UNSUPPORTED, "grid too large");
    a.total_blocks = static_cast<int>(nb); a.xcd_chunk = static_cast<int>((nb + 7) / 8);
    a.dw_xor = dw->xor_mask; a.dw_rq = dw->rq;
    a.pw_w = pw->w_mfma; a.pw_wstride = pw->K_pad; a.pw_ct = ChanTab{pw->chan, pw->Co_pad}; a.pw_corr = pw->corr;
    a.y = static_cast<uint8_t*>(y); a.Co = pw->geom.Co; a.mid_xor = pw->xor_mask; a.pw_rq = pw->rq;
    const int smem = DwPwSmemBytes<S, P>(g.Co);
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&DwPwKernel<S, P, D>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    MI355X_HIP(attr);
    NoteKernel("DwPwKernel<%d, %d, %d>", S, P, D);
    hipLaunchKernelGGL((DwPwKernel<S, P, D>), dim3(static_cast<unsigned>(a.xcd_chunk) * 8u), dim3(256), smem, stream, a);
    MI355X_HIP(hipGetLastError());
    return 0;
}

// ---- depthwise 3x3 + pointwise for the wide, shallow front layers: persistent blocks, pointwise weights resident in LDS -----
// which: 1 = stride 1, 32 -> 64 channels; 2 = stride 2, 64 -> 128; 3 = stride 1, 128 -> 128; 4 = stride 2, 128 -> 256 (eight
// waves: its weights and halo leave room for one block per CU); 0 when the pair does not fit
int DwPwStreamShape(const mi355x_conv2d_s* dw, const mi355x_conv2d_s* pw)
{
    const mi355x_conv2d_desc& a = dw->d;
    if (dw->algo != MI355X_ALGO_DEPTHWISE || dw->variant != 1 || dw->w_dot4b || a.stride_x != a.stride_y || a.out_c != a.in_c) return 0;
    if (pw->zw_neg != 0 || !pw->w_mfma || pw->K_pad < static_cast<int>(a.out_c)) return 0;
    if (static_cast<long long>(a.in_h) * a.in_w * a.in_c >= (1ll << 30) || static_cast<long long>(a.out_h) * a.out_w * pw->d.out_c >= (1ll << 30)) return 0;
    if (a.stride_x == 1 && a.out_c == 32 && pw->d.out_c == 64) return 1;
    if (a.stride_x == 2 && a.out_c == 64 && pw->d.out_c == 128) return 2;
    if (a.stride_x == 1 && a.out_c == 128 && pw->d.out_c == 128) return 3;
    if (a.stride_x == 2 && a.out_c == 128 && pw->d.out_c == 256) return 4;
    return 0;
}

template <int S, int C, int NO, int TH, int TW, int NWAVES = 4>
int LaunchDwPwStreamT(DwPwStreamArgs a, const ConvGeom& g, hipStream_t stream)
{
    using G = DwPwStreamGeom<S, C, NO, TH, TW, NWAVES>;
    constexpr int smem = G::SMEM;
    static_assert(smem <= 156 * 1024, "LDS of one CU");
    const auto kernel = &DwPwStreamKernel<S, C, NO, TH, TW, NWAVES>;
    static const int per_cu = [&]() {
        int n = 0;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, smem) != hipSuccess) return 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, G::NT, smem) != hipSuccess) return 0;
        return n;
    }();
    if (per_cu <= 0) { (void)hipGetLastError(); return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel: no block fits a CU"); }
    a.tiles_x = (g.Wo + TW - 1) / TW; a.tiles_y = (g.Ho + TH - 1) / TH;
    const long long items = static_cast<long long>(a.N) * a.tiles_x * a.tiles_y;
    if (items > 0x7fffffffll - 8 || items * std::max(a.tiles_x, a.tiles_y) >= 0xffffffffll) return SetError(MI355X_ERR_UNSUPPORTED, "grid too large");
    a.total_items = static_cast<int>(items); a.xcd_chunk = static_cast<int>((items + 7) / 8);
    const auto rcp = [](int d) { return d <= 1 ? 0u : static_cast<uint32_t>((0x100000000ull + static_cast<unsigned>(d) - 1) / static_cast<unsigned>(d)); };
    a.rcp_tiles_x = rcp(a.tiles_x); a.rcp_tiles_y = rcp(a.tiles_y);
    const int per_xcd = std::min(a.xcd_chunk, per_cu * (DeviceCuCount() / 8));
    NoteKernel("DwPwStreamKernel<%d, %d, %d, %d, %d, %d>", S, C, NO, TH, TW, NWAVES);
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(per_xcd) * 8u), dim3(G::NT), smem, stream, a);
    MI355X_HIP(hipGetLastError());
    return 0;
}

int LaunchDwPwStream(const mi355x_conv2d_s* dw, const mi355x_conv2d_s* pw, int which, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    const ConvGeom& g = dw->geom;
    DwPwStreamArgs a;
    a.x = static_cast<const uint8_t*>(x); a.pad16 = dw->pad16; a.wpack = dw->w_dot4; a.dw_ct = ChanTab{dw->chan, dw->Co_pad}; a.dw_corr = dw->corr;
    a.N = static_cast<int>(batch); a.H = g.H; a.W = g.W; a.Ho = g.Ho; a.Wo = g.Wo;
    a.pad_top = g.pad_top; a.pad_left = g.pad_left;
    a.dw_xor = dw->xor_mask; a.dw_rq = dw->rq;
    a.w = pw->w_mfma; a.w_stride = pw->K_pad; a.pw_ct = ChanTab{pw->chan, pw->Co_pad}; a.pw_corr = pw->corr;
    a.y = static_cast<uint8_t*>(y);
    a.mid_xor = pw->xor_mask; a.pw_rq = pw->rq;
    if (which == 1) return LaunchDwPwStreamT<1, 32, 64, 16, 16>(a, g, stream);
    if (which == 2) return LaunchDwPwStreamT<2, 64, 128, 8, 8>(a, g, stream);
    if (which == 4) return LaunchDwPwStreamT<2, 128, 256, 8, 8, 8>(a, g, stream);
    return LaunchDwPwStreamT<1, 128, 128, 8, 8>(a, g, stream);
}

// ---- depthwise 3x3 stride 1 + pointwise over 256 / 512 channels: one block per 8 x 8 tile over all channels ---------------
// KT = channels between the layers / 128, NQ = output channels / 256; 0 when the pair does not fit that kernel
bool DwPwPanelShape(const mi355x_conv2d_s* dw, const mi355x_conv2d_s* pw, int* kt, int* nq)
{
    const mi355x_conv2d_desc& a = dw->d;
    if (dw->algo != MI355X_ALGO_DEPTHWISE || dw->variant != 1 || dw->w_dot4b || a.stride_x != a.stride_y || a.stride_x > 2) return false;
    if (a.out_c != a.in_c || (a.out_c != 256 && a.out_c != 512)) return false;
    // stride 2 (a 17 x 17 halo per 128 channels): built for 256 -> 512 channels
    if (a.stride_x == 2 && (a.out_c != 256 || pw->d.out_c != 512)) return false;
    if (pw->zw_neg != 0 || pw->K_pad != static_cast<int>(a.out_c) || !pw->bk128 || !pw->w_mfma || pw->pw_bn != 0) return false;
    if (pw->d.out_c != 256 && pw->d.out_c != 512) return false;
    if (static_cast<long long>(a.in_h) * a.in_w * a.in_c >= (1ll << 31)) return false;
    *kt = static_cast<int>(a.out_c) / 128;
    *nq = static_cast<int>(pw->d.out_c) / 256;
    return true;
}

template <int KT, int NQ, int S = 1>
int LaunchDwPwPanelT(const DwPwPanelArgs& a, hipStream_t stream)
{
    constexpr int smem = DwPwPanelGeom<KT, NQ, S>::SMEM;
    static_assert(smem <= 156 * 1024, "LDS of one CU");
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&DwPwPanelKernel<KT, NQ, S>), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    MI355X_HIP(attr);
    NoteKernel("DwPwPanelKernel<%d, %d, %d>", KT, NQ, S);
    hipLaunchKernelGGL((DwPwPanelKernel<KT, NQ, S>), dim3(static_cast<unsigned>(a.xcd_chunk) * 8u), dim3(512), smem, stream, a);
    MI355X_HIP(hipGetLastError());
    return 0;
}

int LaunchDwPwPanel(const mi355x_conv2d_s* dw, const mi355x_conv2d_s* pw, int kt, int nq, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    const ConvGeom& g = dw->geom;
    DwPwPanelArgs a;
    a.x = static_cast<const uint8_t*>(x); a.pad16 = dw->pad16; a.wpack = dw->w_dot4; a.dw_ct = ChanTab{dw->chan, dw->Co_pad}; a.dw_corr = dw->corr;
    a.N = static_cast<int>(batch); a.H = g.H; a.W = g.W; a.C = g.Co; a.Ho = g.Ho; a.Wo = g.Wo;
    a.pad_top = g.pad_top; a.pad_left = g.pad_left;
    a.tiles_x = (g.Wo + 7) / 8; a.tiles_y = (g.Ho + 7) / 8;
    const long long nb = static_cast<long long>(batch) * a.tiles_x * a.tiles_y;
    if (nb > 0x7fffffffll - 8) return SetError(MI355X_ERR_UNSUPPORTED, "grid too large");
    a.total_tiles = static_cast<int>(nb); a.xcd_chunk = static_cast<int>((nb + 7) / 8);
    a.dw_xor = dw->xor_mask; a.dw_rq = dw->rq;
    a.w = pw->w_mfma; a.K_pad = pw->K_pad; a.pw_ct = ChanTab{pw->chan, pw->Co_pad}; a.pw_corr = pw->corr;
    a.y = static_cast<uint8_t*>(y); a.Co = pw->geom.Co; a.mid_xor = pw->xor_mask; a.pw_rq = pw->rq;
#ifdef MI355X_DWPW_STAMPS
    // measurement build: the first 40 launches record wave 0's shader-clock stamps per block and print the average durations
    // between consecutive stamps, over all blocks
    static unsigned long long* d_stamps = nullptr;
    static int launches = 0;
    a.stamps = nullptr;
    if (launches < 40)
    {
        if (!d_stamps) MI355X_HIP(hipMalloc(reinterpret_cast<void**>(&d_stamps), 65536 * 16 * 8));
        a.stamps = a.total_tiles <= 65536 - 8 ? d_stamps : nullptr;
    }
    int rc = dw->d.stride_x == 2 ? LaunchDwPwPanelT<2, 2, 2>(a, stream)
             : kt == 2 ? (nq == 1 ? LaunchDwPwPanelT<2, 1>(a, stream) : LaunchDwPwPanelT<2, 2>(a, stream))
                       : (nq == 1 ? LaunchDwPwPanelT<4, 1>(a, stream) : LaunchDwPwPanelT<4, 2>(a, stream));
    if (a.stamps && rc == 0 && ++launches == 40)
    {
        MI355X_HIP(hipStreamSynchronize(stream));
        const int nblk = a.xcd_chunk * 8;
        std::vector<unsigned long long> h(static_cast<size_t>(nblk) * 16);
        MI355X_HIP(hipMemcpy(h.data(), d_stamps, h.size() * 8, hipMemcpyDeviceToHost));
        const int ns = 3 + 3 * kt + 1;
        std::vector<double> sum(ns, 0.0);
        int used = 0;
        unsigned long long tmin = ~0ull, tmax = 0;
        for (int b = 0; b < a.total_tiles; ++b)
        {
            const unsigned long long* s = &h[static_cast<size_t>(b) * 16];
            if (s[0] == 0) continue;
            ++used;
            for (int i = 1; i < ns; ++i) sum[i] += static_cast<double>(s[i] - s[i - 1]);
            tmin = std::min(tmin, s[0]); tmax = std::max(tmax, s[ns - 1]);
        }
        std::fprintf(stderr, "DwPwPanelKernel<%d, %d> stamps over %d blocks (cycles): prologue %.0f", kt, nq, used, sum[1] / used);
        for (int k = 0; k < kt; ++k) std::fprintf(stderr, " | dw%d %.0f wait %.0f gemm %.0f", k, sum[2 + 3 * k] / used, sum[3 + 3 * k] / used, sum[4 + 3 * k] / used);
        std::fprintf(stderr, " | requant %.0f stores %.0f | first start to last end %llu\n", sum[2 + 3 * kt] / used, sum[3 + 3 * kt] / used, tmax - tmin);
    }
    return rc;
#else
    if (dw->d.stride_x == 2) return LaunchDwPwPanelT<2, 2, 2>(a, stream);
    if (kt == 2) return nq == 1 ? LaunchDwPwPanelT<2, 1>(a, stream) : LaunchDwPwPanelT<2, 2>(a, stream);
    return nq == 1 ? LaunchDwPwPanelT<4, 1>(a, stream) : LaunchDwPwPanelT<4, 2>(a, stream);
#endif
}

// ---- pointwise 1x1 followed by depthwise 3x3, whole images per block ---------------------------------------------------
constexpr int kPwDwMF = 7;       // 224 pixel rows per block: one 14x14 image, four 7x7 images
// Two LDS stages and eight waves: with a K of 256 .. 512 bytes the k-loop is bound by what a CU's vector L1 delivers, not
// by round trips (four stages measured 4 % slower), and the requantization and depthwise phases, which are pure VALU
// issue, want two waves per SIMD (four waves: 16.1 us against 12.3 us for 32 images of 14 x 14 x 512).
constexpr int kPwDwStages = 2, kPwDwWaves = 8;


struct PwDwShape
{
    int G = 0, HR = 0, HC = 0, pairs = 0, S = 0, MF = 0;
};

constexpr int PwDwWavesFor(int mf) { return mf == 2 ? 4 : kPwDwWaves; }
constexpr int PwDwSmemFor(int mf) { return kPwDwStages * (mf * 32 + 64) * 128; }

// 32-pixel fragments per block for images of `hw` pixels: 7, 4 or 2 (two: four waves).  A block's phases run one after
// the other, so blocks that start together stream, requantize and write together; two smaller blocks per CU overlap
// each other's phases at the price of streaming the 64 channels' weights twice.  Measured on MobileNetV1's 7 x 7 layers
// at 64 images (step, alternated three times): with the pooling as second stage 0.2607 ms at 7 fragments, 0.2589 at 4;
// with the depthwise layer as second stage 4 fragments cost 0.5 us; 2 fragments lose 3 us for both.  At 128 images, where
// the large blocks already come two to a CU, the small ones lose 6 us; at 8 images they gain 3.  `blocks7`: blocks of the
// launch at 7 fragments.
int PwDwFragmentsFor(int hw, bool pooling, long long blocks7)
{
    const int forced = GlobalOptions().pwdw_mf;
    if ((forced == 2 || forced == 4) && hw <= forced * 32) return forced;
    if (forced == 0 && pooling && 2 * hw <= 4 * 32 && blocks7 <= 256) return 4;
    return kPwDwMF;
}

// 0 when the pair (1x1 convolution, 3x3 depthwise) can run as PwDwKernel; the shape the launch needs comes back in `sh`
// 0 when `pw` can be the first stage of PwDwKernel
int PwStageCheck(const mi355x_conv2d_s* pw)
{
    const mi355x_conv2d_desc& a = pw->d;
    const bool pointwise = pw->algo == MI355X_ALGO_MFMA && !a.depthwise && a.kernel_h == 1 && a.kernel_w == 1 && a.stride_x == 1 &&
                           a.stride_y == 1 && a.pad_top == 0 && a.pad_left == 0 && a.out_h == a.in_h && a.out_w == a.in_w;
    if (!pointwise) return SetError(MI355X_ERR_UNSUPPORTED, "first plan is not an unpadded 1x1 stride-1 convolution on the MFMA kernel");
    if (pw->zw_neg != 0) return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel needs pointwise weights without a zero point");
    if ((a.in_c % 128) != 0 || pw->K_pad != static_cast<int>(a.in_c))     // rows are fetched 128 bytes at a time: none may end inside a tile
        return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel needs the pointwise layer's input channels in whole 128-byte k-tiles");
    return 0;
}

int PwDwCheck(const mi355x_conv2d_s* pw, const mi355x_conv2d_s* dw, PwDwShape* sh)
{
    const mi355x_conv2d_desc& a = pw->d;
    const mi355x_conv2d_desc& b = dw->d;
    if (int rc = PwStageCheck(pw)) return rc;
    if (dw->algo != MI355X_ALGO_DEPTHWISE || dw->variant != 1 || !dw->dw_grp || dw->w_dot4b)
        return SetError(MI355X_ERR_UNSUPPORTED, "second plan is not a 3x3 depthwise layer on the v_dot4 kernel");
    if (b.stride_x != b.stride_y || (b.stride_x != 1 && b.stride_x != 2))
        return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel needs depthwise stride 1 or 2");
    if (a.out_c != b.in_c || a.out_h != b.in_h || a.out_w != b.in_w) return SetError(MI355X_ERR_INVALID_ARGUMENT, "the layers' shapes do not chain");
    if (a.output.dtype != b.input.dtype || a.output.scale != b.input.scale || a.output.offset != b.input.offset)
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "the first layer's output quantization is not the second layer's input quantization");
    if ((a.out_c % kPwDwBN) != 0 || b.out_c != a.out_c) return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel needs channels %% 64 == 0 and depth multiplier 1");
    const int hw = static_cast<int>(a.out_h) * static_cast<int>(a.out_w);
    if (hw > kPwDwMF * 32) return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel holds whole images: %d pixels exceed %d", hw, kPwDwMF * 32);
    PwDwShape s;
    s.S = static_cast<int>(b.stride_x);
    s.MF = PwDwFragmentsFor(hw, false, 0);
    s.G = s.MF * 32 / hw;
    s.pairs = (static_cast<int>(b.out_w) + 1) / 2;
    s.HR = (static_cast<int>(b.out_h) - 1) * s.S + 3;
    s.HC = 2 * s.S * s.pairs + 2;
    // the padded intermediate tile reuses the GEMM's stages: tiny images take fewer per block than the rows would allow
    s.G = std::min(s.G, PwDwSmemFor(s.MF) / (s.HR * s.HC * kPwDwPitch));
    if (s.G < 1) return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel: the intermediate tile does not fit LDS");
    if (sh) *sh = s;
    return 0;
}

template <int MF, int S>
int LaunchPwDwT(const PwDwArgs& a, hipStream_t stream)
{
    constexpr int smem = PwDwStageBytes<MF, kPwDwStages>(), NW = PwDwWavesFor(MF);
    static_assert(smem <= 160 * 1024 && smem == PwDwSmemFor(MF), "LDS of one CU");
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&PwDwKernel<MF, kPwDwStages, S, NW>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    MI355X_HIP(attr);
    NoteKernel("PwDwKernel<%d, %d, %d, %d, false>", MF, kPwDwStages, S, NW);
    hipLaunchKernelGGL((PwDwKernel<MF, kPwDwStages, S, NW>), dim3(static_cast<unsigned>(a.xcd_chunk) * 8u), dim3(64 * NW), smem, stream, a);
    MI355X_HIP(hipGetLastError());
    return 0;
}

// the 1x1 stage's arguments and the grid for G images per block
int FillPwStage(const mi355x_conv2d_s* pw, int G, uint32_t batch, const void* x, PwDwArgs* out)
{
    PwDwArgs a{};
    a.x = static_cast<const uint8_t*>(x); a.w = pw->w_mfma; a.K_pad = pw->K_pad; a.pw_ct = ChanTab{pw->chan, pw->Co_pad}; a.pw_corr = pw->corr;
    a.pw_xor = pw->xor_mask; a.pw_rq = pw->rq;
    a.N = static_cast<int>(batch); a.H = pw->geom.Ho; a.W = pw->geom.Wo; a.Ci = pw->geom.Ci; a.C = pw->geom.Co;
    a.G = G; a.tiles_n = a.C / kPwDwBN;
    const long long nb = (static_cast<long long>(batch) + G - 1) / G * a.tiles_n;
    if (nb > 0x7fffffffll - 8) return SetError(MI355X_ERR_UNSUPPORTED, "grid too large");
    a.total_blocks = static_cast<int>(nb); a.xcd_chunk = static_cast<int>((nb + 7) / 8);
    *out = a;
    return 0;
}

int LaunchPwDw(const mi355x_conv2d_s* pw, const mi355x_conv2d_s* dw, const PwDwShape& sh, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    PwDwArgs a;
    if (int rc = FillPwStage(pw, sh.G, batch, x, &a)) return rc;
    a.dw_grp = dw->dw_grp; a.dw_ct = ChanTab{dw->chan, dw->Co_pad}; a.dw_rq = dw->rq; a.dw_xor = dw->xor_mask; a.dw_pad = dw->pad_word;
    a.Ho = dw->geom.Ho; a.Wo = dw->geom.Wo; a.pad_top = dw->geom.pad_top; a.pad_left = dw->geom.pad_left;
    a.HR = sh.HR; a.HC = sh.HC; a.pairs = sh.pairs;
    a.y = static_cast<uint8_t*>(y);
    if (sh.MF == 2) return sh.S == 1 ? LaunchPwDwT<2, 1>(a, stream) : LaunchPwDwT<2, 2>(a, stream);
    if (sh.MF == 4) return sh.S == 1 ? LaunchPwDwT<4, 1>(a, stream) : LaunchPwDwT<4, 2>(a, stream);
    return sh.S == 1 ? LaunchPwDwT<kPwDwMF, 1>(a, stream) : LaunchPwDwT<kPwDwMF, 2>(a, stream);
}

// 0 when the pair (1x1 convolution, pooling over the whole image) can run as PwDwKernel<.., POOL>; G: images per block
int PwPoolCheck(const mi355x_conv2d_s* pw, const mi355x_pool2d_desc* pool, int* G)
{
    if (int rc = PwStageCheck(pw)) return rc;
    const mi355x_conv2d_desc& a = pw->d;
    if (pool->pool_type != 0 && pool->pool_type != 1) return SetError(MI355X_ERR_UNSUPPORTED, "Unsupported pooling algorithm %d", pool->pool_type);
    if (pool->in_h != a.out_h || pool->in_w != a.out_w || pool->channels != a.out_c)
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "the layers' shapes do not chain");
    const bool global = pool->out_h == 1 && pool->out_w == 1 && pool->pool_h == pool->in_h && pool->pool_w == pool->in_w && pool->pad_left == 0 &&
                        pool->pad_right == 0 && pool->pad_top == 0 && pool->pad_bottom == 0;
    if (!global) return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel needs a pooling window that is the whole unpadded image");
    if (a.output.dtype != pool->input.dtype || a.output.scale != pool->input.scale || a.output.offset != pool->input.offset)
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "the convolution's output quantization is not the pooling's input quantization");
    if (!IsActivationDtype(pool->output.dtype)) return SetError(MI355X_ERR_UNSUPPORTED, "pooling output: data type %d is not QAsymmS8/QAsymmU8", pool->output.dtype);
    if (!(pool->output.scale > 0.0f) || !std::isfinite(pool->output.scale))
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "pooling output: scale must be positive and finite");
    if ((a.out_c % kPwDwBN) != 0) return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel needs channels %% 64 == 0");
    const int hw = static_cast<int>(a.out_h) * static_cast<int>(a.out_w);
    if (hw > kGlobalPoolMaxTaps) return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel holds whole images: %d pixels exceed %d", hw, kGlobalPoolMaxTaps);
    if (G) *G = kPwDwMF * 32 / hw;             // images per block of 7 fragments
    return 0;
}

template <int MF>
int LaunchPwPoolT(const mi355x_conv2d_s* pw, const mi355x_pool2d_desc* pool, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    const int hw = static_cast<int>(pw->d.out_h) * static_cast<int>(pw->d.out_w);
    PwDwArgs a;
    if (int rc = FillPwStage(pw, MF * 32 / hw, batch, x, &a)) return rc;
    a.pool_in = MakeQIn(pool->input);
    a.pool_rq = MakeRequant(pool->output, MI355X_ACT_NONE, 0.0f, 0.0f);
    a.pool_is_max = pool->pool_type == 0;
    a.y = static_cast<uint8_t*>(y);
    constexpr int smem = PwDwStageBytes<MF, kPwDwStages>(), NW = PwDwWavesFor(MF);
    static_assert(MF * 32 * kPwDwPitch <= smem, "the intermediate tile reuses the GEMM's stages");
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&PwDwKernel<MF, kPwDwStages, 1, NW, true>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    MI355X_HIP(attr);
    NoteKernel("PwDwKernel<%d, %d, 1, %d, true>", MF, kPwDwStages, NW);
    hipLaunchKernelGGL((PwDwKernel<MF, kPwDwStages, 1, NW, true>), dim3(static_cast<unsigned>(a.xcd_chunk) * 8u), dim3(64 * NW), smem, stream, a);
    MI355X_HIP(hipGetLastError());
    return 0;
}

int LaunchPwPool(const mi355x_conv2d_s* pw, const mi355x_pool2d_desc* pool, int G, uint32_t batch, const void* x, void* y, hipStream_t stream)
{
    const int hw = static_cast<int>(pw->d.out_h) * static_cast<int>(pw->d.out_w);
    const int mf = PwDwFragmentsFor(hw, true, (static_cast<long long>(batch) + G - 1) / G * (pw->d.out_c / kPwDwBN));
    if (mf == 2) return LaunchPwPoolT<2>(pw, pool, batch, x, y, stream);
    if (mf == 4) return LaunchPwPoolT<4>(pw, pool, batch, x, y, stream);
    return LaunchPwPoolT<kPwDwMF>(pw, pool, batch, x, y, stream);
}
} // namespace

namespace mi355x
{
int FillIgemmLdsArgs(const mi355x_conv2d_s* p, int bm, int bn, uint32_t batch, const void* x, void* y, IgemmArgs* out, bool* unit_fast)
{
    const ConvGeom& g = p->geom;
    IgemmArgs a;
    a.x = static_cast<const uint8_t*>(x);
    a.pad16 = p->pad16;
    a.w = p->w_mfma;
    a.ct = ChanTab{p->chan, p->Co_pad};
    a.corr = p->corr;
    a.y = static_cast<uint8_t*>(y);
    const long long M = static_cast<long long>(batch) * g.Ho * g.Wo;
    if (M > 0x7fffffffll / 2) return SetError(MI355X_ERR_UNSUPPORTED, "too many output pixels for one launch (%lld)", M);
    a.M = static_cast<int>(M);
    a.H = g.H; a.W = g.W; a.Ci = g.Ci; a.Ho = g.Ho; a.Wo = g.Wo; a.Co = g.Co;
    a.Kh = g.Kh; a.Kw = g.Kw;
    a.pad_top = g.pad_top; a.pad_left = g.pad_left; a.stride_x = g.stride_x; a.stride_y = g.stride_y;
    a.dil_x = g.dil_x; a.dil_y = g.dil_y;
    a.K_pad = p->K_pad;
    a.unit = (g.Kh == 1 && g.Kw == 1 && g.stride_x == 1 && g.stride_y == 1 && g.pad_top == 0 && g.pad_left == 0 && g.Ho == g.H &&
              g.Wo == g.W) ? 1 : 0;
    if (a.unit) { a.H = 1; a.W = a.M; a.Ho = 1; a.Wo = a.M; }      // one row of M pixels
    a.tiles_m = static_cast<int>((M + bm - 1) / bm);
    a.tiles_n = (g.Co + bn - 1) / bn;
    a.xor_mask = p->xor_mask;
    a.pad_word = p->pad_word;
    a.zw_neg = p->zw_neg;
    a.rowsum_bias = p->rowsum_bias;
    a.rq = p->rq;
    // pointwise layers and FullyConnected below 2 GiB per tensor: addresses without per-load vector arithmetic
    *unit_fast = a.unit && static_cast<long long>(a.M) * a.Ci < (1ll << 31) && static_cast<long long>(p->Co_pad) * a.K_pad < (1ll << 31) &&
                 a.Ci == a.K_pad;
    *out = a;
    return 0;
}

int FillDw3x3Args(const mi355x_conv2d_s* p, uint32_t batch, const void* x, void* y, Dw3x3Args* out, int* rows_out, int* cbw_out)
{
    const ConvGeom& g = p->geom;
    Dw3x3Args a;
    a.x = static_cast<const uint8_t*>(x); a.pad16 = p->pad16; a.wpack = p->w_dot4; a.ct = ChanTab{p->chan, p->Co_pad}; a.corr = p->corr; a.y = static_cast<uint8_t*>(y);
    a.N = static_cast<int>(batch); a.H = g.H; a.W = g.W; a.C = g.Co; a.Ho = g.Ho; a.Wo = g.Wo;
    a.pad_top = g.pad_top; a.pad_left = g.pad_left;
    // 128 channels per block where the channel count allows: every pixel a block reads or writes is a whole line
    // (32 images: 56 x 56 x 128 13.1 -> 11.6 us at stride 1, 7.3 -> 6.4 us at stride 2; 28 x 28 x 256 8.1 -> 7.7 us;
    // 7 x 7 x 1024, where a 16-pixel-wide tile is mostly outside the image, 5.1 -> 4.0 us; 14 x 14 x 512 on par)
    const bool wide = (g.Co % 128) == 0 && p->opt_dw_cb != 32;
    // 64 per block for the other multiples of 64 (32 images: 112 x 112 x 64 at stride 2 10.0 -> 9.4 us, 56 x 56 x 64 7.7 -> 7.5 us, 28 x 28 x 192 6.8 -> 6.5 us)
    const bool mid = !wide && (g.Co % 64) == 0 && p->opt_dw_cb != 32;
    const int cbw = wide ? 128 : mid ? 64 : 32;
    const int tw = wide ? (g.stride_x == 1 ? 8 : 4) : (g.stride_x == 1 ? 16 : 8);
    const int th1 = cbw == 32 ? 8 : 4;       // tile rows with one output row per thread
    // two output rows per thread unless that would leave much of a tile outside a small feature map (or, with the
    // small tiles of the 64- and 128-channel blocks, fewer than two blocks per CU)
    const int opt_r = p->opt_dw_rows;
    int rows_per_thread = opt_r ? opt_r : ((g.Ho + 2 * th1 - 1) / (2 * th1) * (2 * th1) - g.Ho) * 4 <= g.Ho ? 2 : 1;
    if (cbw != 32 && !opt_r && static_cast<long long>(batch) * ((g.Wo + tw - 1) / tw) * ((g.Ho + 2 * th1 - 1) / (2 * th1)) * (g.Co / cbw) < 512)
        rows_per_thread = 1;
    const int th = th1 * rows_per_thread;
    a.tiles_x = (g.Wo + tw - 1) / tw; a.tiles_y = (g.Ho + th - 1) / th; a.cblocks = (g.Co + cbw - 1) / cbw;
    a.xor_mask = p->xor_mask; a.pad_word = p->pad_word; a.rq = p->rq;
    const long long nb = static_cast<long long>(batch) * a.tiles_x * a.tiles_y * a.cblocks;
    if (nb > 0x7fffffffll - 8) return SetError(MI355X_ERR_UNSUPPORTED, "grid too large");
    a.total_blocks = static_cast<int>(nb);
    a.xcd_chunk = static_cast<int>((nb + 7) / 8);
    a.wpack2 = p->w_dot4b;
    *out = a;
    *rows_out = rows_per_thread;
    *cbw_out = cbw;
    return 0;
}
} // namespace mi355x

extern "C" {

int mi355x_conv2d_create(const mi355x_conv2d_desc* desc, const void* weights_host, const mi355x_const_quant* weights_quant,
                         const int32_t* bias_host, const mi355x_const_quant* bias_quant, mi355x_conv2d_t* plan)
{
    if (!desc || !plan) return SetError(MI355X_ERR_INVALID_ARGUMENT, "descriptor / plan pointer is null");
    *plan = nullptr;
    auto* p = new mi355x_conv2d_s;
    int rc = BuildPlan(*desc, weights_host, weights_quant, bias_host, bias_quant, p);
    if (rc != 0) { delete p; return rc; }
    *plan = p;
    return 0;
}

int mi355x_conv2d_run(mi355x_conv2d_t plan, uint32_t batch, const void* input_dev, void* output_dev, mi355x_stream_t stream)
{
    return RunPlan(plan, batch, input_dev, output_dev, ToHip(stream));
}

int mi355x_conv2d_run_add(mi355x_conv2d_t plan, uint32_t batch, const void* input_dev, const void* other_dev, const mi355x_quant* other_quant,
                          const mi355x_quant* sum_quant, int32_t activation, float a, float b, void* output_dev, mi355x_stream_t stream)
{
    if (!plan) return SetError(MI355X_ERR_INVALID_ARGUMENT, "plan is null");
    if (!other_quant || !sum_quant) return SetError(MI355X_ERR_INVALID_ARGUMENT, "quantization of the Addition is null");
    if (activation < MI355X_ACT_NONE || activation > MI355X_ACT_BOUNDED_RELU) return SetError(MI355X_ERR_UNSUPPORTED, "activation %d", activation);
    if (batch == 0) return 0;
    if (!other_dev || !output_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "other input / output pointer is null");
    if (!input_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "input pointer is null");
    {
        // one launch reads the input and the other operand while it writes the sum: the sum may share bytes with neither
        const uintptr_t n_out = static_cast<uintptr_t>(batch) * plan->d.out_h * plan->d.out_w * plan->d.out_c;
        const uintptr_t n_in = static_cast<uintptr_t>(batch) * plan->d.in_h * plan->d.in_w * plan->d.in_c;
        const uintptr_t y0 = reinterpret_cast<uintptr_t>(output_dev), x0 = reinterpret_cast<uintptr_t>(input_dev), o0 = reinterpret_cast<uintptr_t>(other_dev);
        if (y0 < o0 + n_out && o0 < y0 + n_out) return SetError(MI355X_ERR_INVALID_ARGUMENT, "the Addition's other input may not overlap the output buffer");
        if (y0 < x0 + n_in && x0 < y0 + n_out) return SetError(MI355X_ERR_INVALID_ARGUMENT, "the convolution's input may not overlap the output buffer");
    }
    PendingAdd pending;
    pending.other = static_cast<const uint8_t*>(other_dev);
    pending.fuse = MakeAddFuse(plan->d.output, *other_quant, *sum_quant, activation, a, b);
    const bool aligned = (reinterpret_cast<uintptr_t>(other_dev) & 15) == 0 && (reinterpret_cast<uintptr_t>(output_dev) & 15) == 0;
    t_pending_add = aligned ? &pending : nullptr;
    const int rc = RunPlan(plan, batch, input_dev, output_dev, ToHip(stream));
    t_pending_add = nullptr;
    if (rc != 0 || pending.taken) return rc;
    // the kernel this launch resolved to writes its tiles some other way: the Addition runs behind it, in place
    const size_t n = static_cast<size_t>(batch) * plan->d.out_h * plan->d.out_w * plan->d.out_c;
    return mi355x_add_run(n, &plan->d.output, other_quant, sum_quant, activation, a, b, output_dev, other_dev, output_dev, stream);
}

int mi355x_conv2d_fusable(mi355x_conv2d_t dw, mi355x_conv2d_t pw)
{
    if (!dw || !pw) return SetError(MI355X_ERR_INVALID_ARGUMENT, "plan is null");
    // the other order -- 1x1 convolution first, depthwise second -- is the whole-image kernel
    if (!dw->d.depthwise && pw->d.depthwise) return PwDwCheck(dw, pw, nullptr);
    const mi355x_conv2d_desc& a = dw->d;
    const mi355x_conv2d_desc& b = pw->d;
    if (dw->algo != MI355X_ALGO_DEPTHWISE || dw->variant != 1 || !dw->dw_grp || dw->w_dot4b || (dw->d.out_c % 32) != 0)
        return SetError(MI355X_ERR_UNSUPPORTED, "first plan is not a 3x3 depthwise layer on the v_dot4 kernel");
    const bool pointwise = pw->algo == MI355X_ALGO_MFMA && !b.depthwise && b.kernel_h == 1 && b.kernel_w == 1 && b.stride_x == 1 &&
                           b.stride_y == 1 && b.pad_top == 0 && b.pad_left == 0 && b.out_h == b.in_h && b.out_w == b.in_w;
    if (!pointwise) return SetError(MI355X_ERR_UNSUPPORTED, "second plan is not an unpadded 1x1 stride-1 convolution on the MFMA kernel");
    if (pw->zw_neg != 0) return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel needs pointwise weights without a zero point");
    if (a.out_c != b.in_c || a.out_h != b.in_h || a.out_w != b.in_w) return SetError(MI355X_ERR_INVALID_ARGUMENT, "the layers' shapes do not chain");
    if (a.output.dtype != b.input.dtype || a.output.scale != b.input.scale || a.output.offset != b.input.offset)
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "the first layer's output quantization is not the second layer's input quantization");
    if ((b.out_c % 64) != 0) return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel needs output channels %% 64 == 0");
    const int smem = a.stride_x == 1 ? DwPwSmemBytes<1, 2>(static_cast<int>(a.out_c)) : DwPwSmemBytes<2, 2>(static_cast<int>(a.out_c));
    if (smem > 160 * 1024) return SetError(MI355X_ERR_UNSUPPORTED, "fused kernel: %d channels need %d bytes of LDS", a.out_c, smem);
    if (static_cast<long long>(a.in_h) * a.in_w * a.in_c >= (1ll << 31)) return SetError(MI355X_ERR_UNSUPPORTED, "image too large for 32-bit offsets");
    return 0;
}

int mi355x_conv2d_fusion_pays(mi355x_conv2d_t first, mi355x_conv2d_t second, uint32_t batch)
{
    if (!first || !second || batch == 0) return 0;
    if (!first->d.depthwise && second->d.depthwise)
    {
        // 1x1 convolution + the depthwise layer behind it, whole images per block: measured on maps of 7 x 7 with 64 images
        // per launch (512 -> 1024 channels: 12.5 us against 13.9 us as two launches); larger maps gain more as the second
        // half of a depthwise + pointwise pair
        if (GlobalOptions().pwdw_auto == 0 || PwDwCheck(first, second, nullptr) != 0) return 0;
        return first->d.out_h <= 7 && first->d.out_w <= 7 && batch >= 64 ? 1 : 0;
    }
    if (!first->d.depthwise || second->d.depthwise) return 0;
    if (GlobalOptions().dwpw_stream != 0 && DwPwStreamShape(first, second) != 0 && mi355x_conv2d_fusable(first, second) == 0)
    {
        // persistent blocks: a few items each are needed to overlap anything
        const long long items = static_cast<long long>(batch) * ((first->d.out_w + 7) / 8) * ((first->d.out_h + 7) / 8);
        return items >= 1024 ? 1 : 0;
    }
    int kt = 0, nq = 0;
    if (GlobalOptions().dwpw_panel == 0 || !DwPwPanelShape(first, second, &kt, &nq)) return 0;
    if (mi355x_conv2d_fusable(first, second) != 0) return 0;
    // a block takes a CU to itself: below about a hundred tiles per launch most of the device would idle (measured on
    // MobileNetV1: a gain at 32 images per launch, a loss at 16)
    const long long tiles = static_cast<long long>(batch) * ((first->d.out_w + 7) / 8) * ((first->d.out_h + 7) / 8);
    return tiles >= 100 ? 1 : 0;
}

int mi355x_conv2d_run_fused(mi355x_conv2d_t dw, mi355x_conv2d_t pw, uint32_t batch, const void* input_dev, void* output_dev,
                            mi355x_stream_t stream)
{
    if (int rc = mi355x_conv2d_fusable(dw, pw)) return rc;
    if (batch == 0) return 0;
    if (!input_dev || !output_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "input / output pointer is null");
    if ((reinterpret_cast<uintptr_t>(input_dev) & 15) != 0 || (reinterpret_cast<uintptr_t>(output_dev) & 15) != 0)
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "fused kernel needs 16-byte aligned tensors");
    if (!dw->d.depthwise && pw->d.depthwise)
    {
        PwDwShape sh;
        if (int rc = PwDwCheck(dw, pw, &sh)) return rc;
        return LaunchPwDw(dw, pw, sh, batch, input_dev, output_dev, ToHip(stream));
    }
    if (GlobalOptions().dwpw_stream != 0)
        if (const int which = DwPwStreamShape(dw, pw)) return LaunchDwPwStream(dw, pw, which, batch, input_dev, output_dev, ToHip(stream));
    {
        int kt = 0, nq = 0;
        if (GlobalOptions().dwpw_panel != 0 && DwPwPanelShape(dw, pw, &kt, &nq)) return LaunchDwPwPanel(dw, pw, kt, nq, batch, input_dev, output_dev, ToHip(stream));
    }
    if (dw->d.stride_x == 2) return LaunchDwPw<2, 2>(dw, pw, batch, input_dev, output_dev, ToHip(stream));
    // stride 1: the wide tile (8 x 16 pixels) while it still yields two blocks per CU, else the narrow one (8 x 8)
    const long long wide = static_cast<long long>(batch) * ((dw->d.out_w + 15) / 16) * ((dw->d.out_h + 7) / 8);
    if (wide >= 512 && DwPwSmemBytes<1, 4>(static_cast<int>(dw->d.out_c)) <= 160 * 1024)
        return LaunchDwPw<1, 4>(dw, pw, batch, input_dev, output_dev, ToHip(stream));
    return LaunchDwPw<1, 2>(dw, pw, batch, input_dev, output_dev, ToHip(stream));
}

int mi355x_conv2d_pool_fusable(mi355x_conv2d_t conv, const mi355x_pool2d_desc* pool)
{
    if (!conv || !pool) return SetError(MI355X_ERR_INVALID_ARGUMENT, "plan / pooling descriptor is null");
    return PwPoolCheck(conv, pool, nullptr);
}

int mi355x_conv2d_pool_fusion_pays(mi355x_conv2d_t conv, const mi355x_pool2d_desc* pool, uint32_t batch)
{
    if (!conv || !pool || batch == 0 || GlobalOptions().pwpool_auto == 0) return 0;
    int G = 0;
    if (PwPoolCheck(conv, pool, &G) != 0) return 0;
    // a block per (G images, 64 channels).  Measured on 7 x 7 x 1024 -> 1024 with 8 .. 128 images per launch (32 .. 512
    // blocks): the one launch is 1.2 us (8 images) to 11 us (128 images) shorter than the two; not measured below that
    const long long blocks = (static_cast<long long>(batch) + G - 1) / G * (conv->d.out_c / kPwDwBN);
    return blocks >= 32 ? 1 : 0;
}

int mi355x_conv2d_run_pooled(mi355x_conv2d_t conv, const mi355x_pool2d_desc* pool, uint32_t batch, const void* input_dev, void* output_dev,
                             mi355x_stream_t stream)
{
    if (!conv || !pool) return SetError(MI355X_ERR_INVALID_ARGUMENT, "plan / pooling descriptor is null");
    int G = 0;
    if (int rc = PwPoolCheck(conv, pool, &G)) return rc;
    if (batch == 0) return 0;
    if (!input_dev || !output_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "input / output pointer is null");
    if ((reinterpret_cast<uintptr_t>(input_dev) & 15) != 0) return SetError(MI355X_ERR_INVALID_ARGUMENT, "fused kernel needs a 16-byte aligned input");
    {
        // one launch reads the input while it writes the pooled tensor
        const uintptr_t x0 = reinterpret_cast<uintptr_t>(input_dev), y0 = reinterpret_cast<uintptr_t>(output_dev);
        const uintptr_t n_in = static_cast<uintptr_t>(batch) * conv->d.in_h * conv->d.in_w * conv->d.in_c;
        const uintptr_t n_out = static_cast<uintptr_t>(batch) * conv->d.out_c;
        if (y0 < x0 + n_in && x0 < y0 + n_out) return SetError(MI355X_ERR_INVALID_ARGUMENT, "the convolution's input may not overlap the pooled output");
    }
    return LaunchPwPool(conv, pool, G, batch, input_dev, output_dev, ToHip(stream));
}

int mi355x_conv2d_destroy(mi355x_conv2d_t plan)
{
    delete plan;
    return 0;
}

int mi355x_conv2d_set_concurrency(mi355x_conv2d_t plan, uint32_t lanes)
{
    if (!plan) return SetError(MI355X_ERR_INVALID_ARGUMENT, "plan is null");
    if (lanes == 0) return SetError(MI355X_ERR_INVALID_ARGUMENT, "the number of lanes must be at least 1");
    plan->concurrency = lanes;
    return 0;
}

int mi355x_conv2d_algo(mi355x_conv2d_t plan, int32_t* algo, char* desc_buf, size_t desc_len)
{
    if (!plan) return SetError(MI355X_ERR_INVALID_ARGUMENT, "plan is null");
    if (algo) *algo = plan->algo;
    if (desc_buf && desc_len) snprintf(desc_buf, desc_len, "%s", plan->info.c_str());
    return 0;
}

// FullyConnected = 1x1 convolution over a 1x1 image with in_c = K: row n of the input is pixel n.
int mi355x_fc_create(const mi355x_fc_desc* desc, const void* weights_host, const mi355x_const_quant* weights_quant,
                     const int32_t* bias_host, const mi355x_const_quant* bias_quant, mi355x_fc_t* plan)
{
    if (!desc || !plan) return SetError(MI355X_ERR_INVALID_ARGUMENT, "descriptor / plan pointer is null");
    *plan = nullptr;
    if (desc->k == 0 || desc->out_features == 0) return SetError(MI355X_ERR_INVALID_ARGUMENT, "zero-sized FullyConnected");
    if (!weights_host) return SetError(MI355X_ERR_INVALID_ARGUMENT, "weights missing");
    mi355x_conv2d_desc c{};
    c.in_h = c.in_w = c.out_h = c.out_w = 1;
    c.in_c = desc->k;
    c.out_c = desc->out_features;
    c.kernel_h = c.kernel_w = 1;
    c.stride_x = c.stride_y = c.dilation_x = c.dilation_y = 1;
    c.bias_enabled = desc->bias_enabled;
    c.input = desc->input;
    c.output = desc->output;
    c.activation = desc->activation;
    c.activation_a = desc->activation_a;
    c.activation_b = desc->activation_b;
    c.algo = desc->algo;

    const uint8_t* w = static_cast<const uint8_t*>(weights_host);
    std::vector<uint8_t> wt;
    if (!desc->transpose_weights)
    {
        // [K][O] -> [O][K]
        const size_t K = desc->k, O = desc->out_features;
        wt.resize(K * O);
        for (size_t k = 0; k < K; ++k)
            for (size_t o = 0; o < O; ++o) wt[o * K + k] = w[k * O + o];
        w = wt.data();
    }
    auto* cp = new mi355x_conv2d_s;
    int rc = BuildPlan(c, w, weights_quant, bias_host, bias_quant, cp);
    if (rc != 0) { delete cp; return rc; }
    auto* p = new mi355x_fc_s;
    p->conv = cp;
    *plan = p;
    return 0;
}

int mi355x_fc_run(mi355x_fc_t plan, uint32_t batch, const void* input_dev, void* output_dev, mi355x_stream_t stream)
{
    if (!plan) return SetError(MI355X_ERR_INVALID_ARGUMENT, "plan is null");
    return RunPlan(plan->conv, batch, input_dev, output_dev, ToHip(stream));
}

int mi355x_fc_destroy(mi355x_fc_t plan)
{
    delete plan;
    return 0;
}

int mi355x_fc_algo(mi355x_fc_t plan, int32_t* algo, char* desc_buf, size_t desc_len)
{
    if (!plan) return SetError(MI355X_ERR_INVALID_ARGUMENT, "plan is null");
    return mi355x_conv2d_algo(plan->conv, algo, desc_buf, desc_len);
}

} // extern "C"
