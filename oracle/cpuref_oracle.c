/*
 * CPU restatement of the Arm NN CpuRef quantized hot path -- TEST INFRASTRUCTURE ONLY.
 * See cpuref_oracle.h.  Citations are relative to the Arm NN 35.0.0 source tree.
 *
 * Build: gcc -O2 -std=c11 -ffp-contract=off -fno-fast-math -fopenmp -fPIC -shared
 * (no -march flags that enable FMA contraction; -ffp-contract=off keeps mul and add separate).
 */
#include "cpuref_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <float.h>

static __thread char g_err[256];

const char* orc_last_error(void) { return g_err; }

static int fail(const char* msg)
{
    snprintf(g_err, sizeof(g_err), "%s", msg);
    return -1;
}

/* ------------------------------------------------------------------------------------------------
 * A1/A2: src/armnn/TypesUtils.cpp:29-56
 *   Dequantize: numeric_cast<float>(value - offset) * scale     (integer subtract, then one fp32 multiply)
 *   Quantize:   clamp(float(offset) + float(round(value/scale)), lowest, max) -> cast
 *               `round` is C round(): half away from zero; value/scale is an fp32 division.
 * ---------------------------------------------------------------------------------------------- */
float orc_dequantize_s8(int8_t v, float scale, int32_t offset)  { return (float)((int32_t)v - offset) * scale; }
float orc_dequantize_u8(uint8_t v, float scale, int32_t offset) { return (float)((int32_t)v - offset) * scale; }
float orc_dequantize_s32(int32_t v, float scale, int32_t offset){ return (float)(v - offset) * scale; }

static inline float quantize_common(float value, float scale, int32_t offset, float lo, float hi)
{
    float q = value / scale;                       /* fp32 divide */
    float r = (float)round((double)q);             /* half away from zero; exact in either precision */
    float v = (float)offset + r;
    v = v > lo ? v : lo;                           /* std::max(v, lowest) */
    v = v < hi ? v : hi;                           /* std::min(., max)    */
    return v;
}

int8_t orc_quantize_s8(float v, float scale, int32_t offset)
{
    return (int8_t)quantize_common(v, scale, offset, -128.0f, 127.0f);
}

uint8_t orc_quantize_u8(float v, float scale, int32_t offset)
{
    return (uint8_t)quantize_common(v, scale, offset, 0.0f, 255.0f);
}

/* ------------------------------------------------------------------------------------------------
 * helpers mirroring TensorInfo (src/armnn/Tensor.cpp:446-495)
 * ---------------------------------------------------------------------------------------------- */
static size_t num_elements(const orc_tensor* t)
{
    size_t n = 1;
    for (uint32_t i = 0; i < t->ndim; ++i) n *= t->shape[i];
    return n;
}

static int has_per_axis(const orc_tensor* t) { return t->n_scales > 1 || t->quant_dim >= 0; }

/* GetQuantizationScale(): no scales -> 1.0f (old default); several -> the reference throws. */
static int scalar_scale(const orc_tensor* t, float* s)
{
    if (t->n_scales == 0) { *s = 1.0f; return 0; }
    if (t->n_scales > 1)  return fail("GetQuantizationScale on a tensor with multiple scales");
    *s = t->scales[0];
    return 0;
}

/* ------------------------------------------------------------------------------------------------
 * A3: Decoder<float>::DecodeTensor  -- workloads/BaseIterator.hpp:111-211 (per-tensor 8-bit),
 *     :704-830 (PerAxisIterator / QSymm8PerAxisDecoder), :307-338 (ScaledInt32Decoder),
 *     :861-911 (ScaledInt32PerAxisDecoder), selection rules workloads/Decoders.hpp:19-126.
 * ---------------------------------------------------------------------------------------------- */
int orc_decode_tensor(const orc_tensor* t, int is_depthwise, float* out)
{
    const size_t n = num_elements(t);
    float s;
    switch (t->dtype)
    {
    case ORC_QASYMM_S8:
        if (scalar_scale(t, &s)) return -1;
        for (size_t i = 0; i < n; ++i) out[i] = orc_dequantize_s8(((const int8_t*)t->data)[i], s, t->offset);
        return 0;
    case ORC_QASYMM_U8:
        if (scalar_scale(t, &s)) return -1;
        for (size_t i = 0; i < n; ++i) out[i] = orc_dequantize_u8(((const uint8_t*)t->data)[i], s, t->offset);
        return 0;
    case ORC_QSYMM_S8:
        if (has_per_axis(t))
        {
            /* QSymm8PerAxisDecoder: scale index = (i / axisFactor) % shape[quantDim]
             * (PerAxisIterator::SetIndexOnMem, BaseIterator.hpp:763-777; axisFactor =
             * GetNumElementsAfter(shape, quantDim), src/armnnUtils/TensorUtils.cpp:261-278). */
            if (t->quant_dim < 0 || (uint32_t)t->quant_dim >= t->ndim)
                return fail("per-axis tensor without a valid quantization dimension");
            const uint32_t axis_dim = t->shape[t->quant_dim];
            size_t axis_factor = 1;
            for (uint32_t i = (uint32_t)t->quant_dim + 1; i < t->ndim; ++i) axis_factor *= t->shape[i];
            for (size_t i = 0; i < n; ++i)
            {
                size_t ai = (i < axis_factor || axis_dim < 1) ? 0 : (i / axis_factor) % axis_dim;
                if (ai >= t->n_scales) return fail("per-axis scale index out of range");
                out[i] = orc_dequantize_s8(((const int8_t*)t->data)[i], t->scales[ai], t->offset);
            }
            return 0;
        }
        if (scalar_scale(t, &s)) return -1;
        for (size_t i = 0; i < n; ++i) out[i] = orc_dequantize_s8(((const int8_t*)t->data)[i], s, t->offset);
        return 0;
    case ORC_SIGNED32:
        if (has_per_axis(t))
        {
            /* ScaledInt32PerAxisDecoder::DecodeTensor: blocks of stepSize elements share scales[step];
             * stepSize = isDepthwise ? shape[2]*shape[3] : numElements/shape[0]. */
            if (t->ndim == 0 || n == 0) return 0;
            if (is_depthwise && t->ndim < 4) return fail("depthwise int32 decode needs a 4-D shape");
            const size_t step_size = is_depthwise ? (size_t)t->shape[2] * t->shape[3] : n / t->shape[0];
            if (step_size == 0) return fail("zero step size");
            const size_t step_num = n / step_size;
            for (size_t step = 0; step < step_num; ++step)
            {
                if (step >= t->n_scales) return fail("per-axis bias scale index out of range");
                for (size_t i = 0; i < step_size; ++i)
                {
                    size_t idx = step * step_size + i;
                    out[idx] = orc_dequantize_s32(((const int32_t*)t->data)[idx], t->scales[step], 0);
                }
            }
            return 0;
        }
        if (scalar_scale(t, &s)) return -1;
        if (s == 0.0f)     /* Int32Decoder: plain cast */
            for (size_t i = 0; i < n; ++i) out[i] = (float)((const int32_t*)t->data)[i];
        else               /* ScaledInt32Decoder */
            for (size_t i = 0; i < n; ++i) out[i] = (float)((const int32_t*)t->data)[i] * s;
        return 0;
    case ORC_FLOAT32:
        memcpy(out, t->data, n * sizeof(float));
        return 0;
    default:
        return fail("Unsupported target Data Type!");
    }
}

/* A4: Encoder<float>::Set -- BaseIterator.hpp:486-532 via MakeEncoder (Encoders.hpp:19-91). */
int orc_encode_tensor(const float* v, size_t n, const orc_tensor* out)
{
    float s;
    switch (out->dtype)
    {
    case ORC_QASYMM_S8:
        if (scalar_scale(out, &s)) return -1;
        for (size_t i = 0; i < n; ++i) ((int8_t*)out->data)[i] = orc_quantize_s8(v[i], s, out->offset);
        return 0;
    case ORC_QASYMM_U8:
        if (scalar_scale(out, &s)) return -1;
        for (size_t i = 0; i < n; ++i) ((uint8_t*)out->data)[i] = orc_quantize_u8(v[i], s, out->offset);
        return 0;
    case ORC_QSYMM_S8:
        if (has_per_axis(out)) return fail("per-axis output encoders are outside the restated path");
        if (scalar_scale(out, &s)) return -1;
        for (size_t i = 0; i < n; ++i) ((int8_t*)out->data)[i] = orc_quantize_s8(v[i], s, out->offset);
        return 0;
    case ORC_FLOAT32:
        memcpy(out->data, v, n * sizeof(float));
        return 0;
    default:
        return fail("Unsupported target Data Type!");
    }
}

/* ------------------------------------------------------------------------------------------------
 * A6: Convolve -- workloads/ConvImpl.cpp:68-233.  Literal loop nest and index arithmetic.
 * ---------------------------------------------------------------------------------------------- */
int orc_convolve_f32(const uint32_t in_shape[4], const float* in, const uint32_t out_shape[4], float* out,
                     const uint32_t filter_shape[4], const float* filter, const float* bias,
                     const orc_conv_params* p)
{
    if (p->bias_enabled && !bias) return fail("Bias is enabled but the bias data is invalid");
    const int nhwc = p->data_layout == ORC_NHWC;
    const unsigned ci_idx = nhwc ? 3 : 1, h_idx = nhwc ? 1 : 2, w_idx = nhwc ? 2 : 3;

    const unsigned inputChannels  = in_shape[ci_idx];
    const unsigned outputChannels = out_shape[ci_idx];
    const unsigned depthMultiplier = p->depthwise ? outputChannels / inputChannels : 1;
    const unsigned batchSize = out_shape[0];
    const unsigned outputHeight = out_shape[h_idx], outputWidth = out_shape[w_idx];
    const unsigned inputHeight = in_shape[h_idx], inputWidth = in_shape[w_idx];
    const unsigned filterHeight = p->depthwise ? filter_shape[1] : filter_shape[h_idx];
    const unsigned filterWidth  = p->depthwise ? filter_shape[2] : filter_shape[w_idx];

    for (unsigned batchIdx = 0; batchIdx < batchSize; batchIdx++)
    for (unsigned cOutput = 0; cOutput < outputChannels; cOutput++)
    for (unsigned yOutput = 0; yOutput < outputHeight; yOutput++)
    for (unsigned xOutput = 0; xOutput < outputWidth; xOutput++)
    {
        float sum = 0.0f;
        for (unsigned cInput = 0; cInput < (p->depthwise ? 1u : inputChannels); cInput++)
        {
            for (unsigned yFilter = 0; yFilter < filterHeight; yFilter++)
            for (unsigned xFilter = 0; xFilter < filterWidth; xFilter++)
            {
                unsigned filterIndex;
                if (p->depthwise)
                {
                    cInput = cOutput / depthMultiplier;
                    filterIndex = xFilter * outputChannels + cOutput + yFilter * filterWidth * outputChannels;
                }
                else if (nhwc)
                    filterIndex = cOutput * filterHeight * filterWidth * inputChannels +
                                  yFilter * filterWidth * inputChannels + xFilter * inputChannels + cInput;
                else
                    filterIndex = cOutput * filterWidth * filterHeight * inputChannels +
                                  cInput * filterWidth * filterHeight + yFilter * filterWidth + xFilter;

                unsigned yInput = yOutput * p->stride_y + yFilter * p->dilation_y;
                unsigned xInput = xOutput * p->stride_x + xFilter * p->dilation_x;
                float inputValue;
                if (yInput < p->pad_top || yInput >= inputHeight + p->pad_top ||
                    xInput < p->pad_left || xInput >= inputWidth + p->pad_left)
                {
                    inputValue = 0.0f;
                }
                else
                {
                    unsigned inputIndex;
                    if (nhwc)
                        inputIndex = batchIdx * inputHeight * inputWidth * inputChannels +
                                     (yInput - p->pad_top) * inputWidth * inputChannels +
                                     (xInput - p->pad_left) * inputChannels + cInput;
                    else
                        inputIndex = batchIdx * inputWidth * inputHeight * inputChannels +
                                     inputWidth * inputHeight * cInput +
                                     inputWidth * (yInput - p->pad_top) + xInput - p->pad_left;
                    inputValue = in[inputIndex];
                }
                sum += filter[filterIndex] * inputValue;
            }
            /* in the depthwise case the reference overwrote cInput inside the loop; the loop bound is 1,
             * so the outer loop ends after one pass whatever value cInput now holds. */
            if (p->depthwise) break;
        }
        if (p->bias_enabled) sum += bias[cOutput];

        unsigned outIdx;
        if (nhwc)
            outIdx = batchIdx * outputHeight * outputWidth * outputChannels +
                     yOutput * outputWidth * outputChannels + xOutput * outputChannels + cOutput;
        else
            outIdx = batchIdx * outputHeight * outputWidth * outputChannels +
                     cOutput * outputHeight * outputWidth + yOutput * outputWidth + xOutput;
        out[outIdx] = sum;
    }
    return 0;
}

/* Same sums in the same per-output order (cIn outer, then ky, kx; bias last), but the loop nest is turned
 * inside out so the innermost loop runs over output channels on a transposed filter.  Skipping a padding
 * tap is bit-identical to adding filter*0.0f: the running sum starts at +0.0f and x + (+-0.0f) == x for
 * every finite x that can occur (+0.0f + -0.0f == +0.0f). NHWC only. */
int orc_convolve_f32_fast(const uint32_t in_shape[4], const float* in, const uint32_t out_shape[4], float* out,
                          const uint32_t filter_shape[4], const float* filter, const float* bias,
                          const orc_conv_params* p)
{
    if (p->data_layout != ORC_NHWC) return fail("fast convolve is NHWC only");
    if (p->bias_enabled && !bias) return fail("Bias is enabled but the bias data is invalid");
    const unsigned Ci = in_shape[3], Co = out_shape[3];
    const unsigned N = out_shape[0], Ho = out_shape[1], Wo = out_shape[2];
    const unsigned H = in_shape[1], W = in_shape[2];
    const unsigned Kh = filter_shape[1], Kw = filter_shape[2];
    const unsigned M = p->depthwise ? Co / Ci : 1;

    float* wT = NULL;
    if (!p->depthwise)
    {
        /* [Co][Kh][Kw][Ci] -> [Ci][Kh][Kw][Co] : rows in the reference's tap order, columns = cOut */
        wT = (float*)malloc((size_t)Ci * Kh * Kw * Co * sizeof(float));
        if (!wT) return fail("out of memory");
        for (unsigned co = 0; co < Co; ++co)
        for (unsigned ky = 0; ky < Kh; ++ky)
        for (unsigned kx = 0; kx < Kw; ++kx)
        for (unsigned ci = 0; ci < Ci; ++ci)
            wT[(((size_t)ci * Kh + ky) * Kw + kx) * Co + co] = filter[(((size_t)co * Kh + ky) * Kw + kx) * Ci + ci];
    }

    #pragma omp parallel
    {
        float* acc = (float*)malloc((size_t)Co * sizeof(float));
        #pragma omp for collapse(2) schedule(static)
        for (unsigned n = 0; n < N; ++n)
        for (unsigned y = 0; y < Ho; ++y)
        for (unsigned x = 0; x < Wo; ++x)
        {
            for (unsigned c = 0; c < Co; ++c) acc[c] = 0.0f;
            if (!p->depthwise)
            {
                for (unsigned ci = 0; ci < Ci; ++ci)
                for (unsigned ky = 0; ky < Kh; ++ky)
                {
                    unsigned yi = y * p->stride_y + ky * p->dilation_y;
                    if (yi < p->pad_top || yi >= H + p->pad_top) continue;
                    for (unsigned kx = 0; kx < Kw; ++kx)
                    {
                        unsigned xi = x * p->stride_x + kx * p->dilation_x;
                        if (xi < p->pad_left || xi >= W + p->pad_left) continue;
                        const float v = in[(((size_t)n * H + (yi - p->pad_top)) * W + (xi - p->pad_left)) * Ci + ci];
                        const float* wr = wT + (((size_t)ci * Kh + ky) * Kw + kx) * Co;
                        for (unsigned c = 0; c < Co; ++c) acc[c] += wr[c] * v;
                    }
                }
            }
            else
            {
                for (unsigned ky = 0; ky < Kh; ++ky)
                {
                    unsigned yi = y * p->stride_y + ky * p->dilation_y;
                    if (yi < p->pad_top || yi >= H + p->pad_top) continue;
                    for (unsigned kx = 0; kx < Kw; ++kx)
                    {
                        unsigned xi = x * p->stride_x + kx * p->dilation_x;
                        if (xi < p->pad_left || xi >= W + p->pad_left) continue;
                        const float* ir = in + (((size_t)n * H + (yi - p->pad_top)) * W + (xi - p->pad_left)) * Ci;
                        const float* wr = filter + ((size_t)ky * Kw + kx) * Co;
                        if (M == 1)
                            for (unsigned c = 0; c < Co; ++c) acc[c] += wr[c] * ir[c];
                        else
                            for (unsigned c = 0; c < Co; ++c) acc[c] += wr[c] * ir[c / M];
                    }
                }
            }
            float* o = out + (((size_t)n * Ho + y) * Wo + x) * Co;
            if (p->bias_enabled) for (unsigned c = 0; c < Co; ++c) o[c] = acc[c] + bias[c];
            else                 for (unsigned c = 0; c < Co; ++c) o[c] = acc[c];
        }
        free(acc);
    }
    free(wT);
    return 0;
}

/* ------------------------------------------------------------------------------------------------
 * A8: FullyConnected -- workloads/FullyConnected.cpp:13-65
 * ---------------------------------------------------------------------------------------------- */
int orc_fully_connected_f32(uint32_t batch, uint32_t K, uint32_t O, const float* in, const float* w,
                            const float* bias, int transpose_weights, float* out)
{
    for (unsigned n = 0; n < batch; n++)
    for (unsigned channelOutput = 0; channelOutput < O; channelOutput++)
    {
        float outval = 0.f;
        for (unsigned channelInput = 0; channelInput < K; channelInput++)
        {
            float weight = transpose_weights ? w[(size_t)channelOutput * K + channelInput]
                                             : w[(size_t)channelInput * O + channelOutput];
            outval += weight * in[(size_t)n * K + channelInput];
        }
        if (bias) outval += bias[channelOutput];
        out[(size_t)n * O + channelOutput] = outval;
    }
    return 0;
}

int orc_fully_connected_f32_fast(uint32_t batch, uint32_t K, uint32_t O, const float* in, const float* w,
                                 const float* bias, int transpose_weights, float* out)
{
    const float* wk = w;          /* [K][O] */
    float* wT = NULL;
    if (transpose_weights)
    {
        wT = (float*)malloc((size_t)K * O * sizeof(float));
        if (!wT) return fail("out of memory");
        for (unsigned o = 0; o < O; ++o)
            for (unsigned k = 0; k < K; ++k) wT[(size_t)k * O + o] = w[(size_t)o * K + k];
        wk = wT;
    }
    #pragma omp parallel for schedule(static)
    for (unsigned n = 0; n < batch; ++n)
    {
        float* o = out + (size_t)n * O;
        for (unsigned c = 0; c < O; ++c) o[c] = 0.0f;
        for (unsigned k = 0; k < K; ++k)
        {
            const float v = in[(size_t)n * K + k];
            const float* wr = wk + (size_t)k * O;
            for (unsigned c = 0; c < O; ++c) o[c] += wr[c] * v;
        }
        if (bias) for (unsigned c = 0; c < O; ++c) o[c] += bias[c];
    }
    free(wT);
    return 0;
}

/* A5: workloads/Activation.cpp:33-42 */
float orc_activation_f32(float in, int function, float a, float b)
{
    switch (function)
    {
    case ORC_ACT_RELU:         return 0.f > in ? 0.f : in;                      /* std::max(0.f, in) */
    case ORC_ACT_BOUNDED_RELU: { float m = b > in ? b : in; return a < m ? a : m; } /* min(a, max(b, in)) */
    default:                   return in;
    }
}

/* ------------------------------------------------------------------------------------------------
 * Whole workloads
 * ---------------------------------------------------------------------------------------------- */
int orc_conv2d(const orc_tensor* in, const orc_tensor* weights, const orc_tensor* bias,
               const orc_tensor* out, const orc_conv_params* p, int fast)
{
    if (in->ndim != 4 || out->ndim != 4 || weights->ndim != 4) return fail("conv tensors must be 4-D");
    const size_t n_in = num_elements(in), n_w = num_elements(weights), n_out = num_elements(out);
    const unsigned c_idx = p->data_layout == ORC_NHWC ? 3 : 1;
    const unsigned Co = out->shape[c_idx];
    float* fin = (float*)malloc((n_in + 1) * sizeof(float));
    float* fw  = (float*)malloc((n_w + 1) * sizeof(float));
    float* fo  = (float*)malloc((n_out + 1) * sizeof(float));
    float* fb  = NULL;
    int rc = -1;
    if (!fin || !fw || !fo) { fail("out of memory"); goto done; }
    if (orc_decode_tensor(in, 0, fin)) goto done;
    /* ConvImpl.cpp:112 forwards `depthwise` to the filter decoder only */
    if (orc_decode_tensor(weights, p->depthwise, fw)) goto done;
    if (p->bias_enabled)
    {
        if (!bias) { fail("Bias is enabled but the bias data is invalid"); goto done; }
        /* ConvImpl.cpp:114-115: decoded with shape {outputChannels}, isDepthwise defaulted to false */
        orc_tensor b = *bias;
        b.ndim = 1; b.shape[0] = Co;
        fb = (float*)malloc(((size_t)Co + 1) * sizeof(float));
        if (!fb) { fail("out of memory"); goto done; }
        if (orc_decode_tensor(&b, 0, fb)) goto done;
    }
    if (fast) rc = orc_convolve_f32_fast(in->shape, fin, out->shape, fo, weights->shape, fw, fb, p);
    else      rc = orc_convolve_f32(in->shape, fin, out->shape, fo, weights->shape, fw, fb, p);
    if (rc == 0) rc = orc_encode_tensor(fo, n_out, out);
done:
    free(fin); free(fw); free(fo); free(fb);
    return rc;
}

int orc_fully_connected(const orc_tensor* in, const orc_tensor* weights, const orc_tensor* bias,
                        const orc_tensor* out, int bias_enabled, int transpose_weights, int fast)
{
    if (out->ndim != 2 || weights->ndim != 2 || in->ndim < 1) return fail("bad FullyConnected shapes");
    /* RefFullyConnectedWorkload.cpp:16-24 GetNumActivations: product of input dims 1.. */
    unsigned K = 1;
    for (uint32_t i = 1; i < in->ndim; ++i) K *= in->shape[i];
    const unsigned batch = in->shape[0];
    const unsigned O = out->shape[1];
    const size_t n_in = num_elements(in), n_w = num_elements(weights), n_out = (size_t)batch * O;
    if (n_w != (size_t)K * O) return fail("weight element count != K*O");
    float* fin = (float*)malloc((n_in + 1) * sizeof(float));
    float* fw  = (float*)malloc((n_w + 1) * sizeof(float));
    float* fo  = (float*)malloc((n_out + 1) * sizeof(float));
    float* fb  = NULL;
    int rc = -1;
    if (!fin || !fw || !fo) { fail("out of memory"); goto done; }
    if (orc_decode_tensor(in, 0, fin)) goto done;
    if (orc_decode_tensor(weights, 0, fw)) goto done;
    if (bias_enabled)
    {
        if (!bias) { fail("bias enabled without bias tensor"); goto done; }
        orc_tensor b = *bias;              /* FullyConnected.cpp:30-32: biasShape{outputSize} */
        b.ndim = 1; b.shape[0] = O;
        fb = (float*)malloc(((size_t)O + 1) * sizeof(float));
        if (!fb) { fail("out of memory"); goto done; }
        if (orc_decode_tensor(&b, 0, fb)) goto done;
    }
    if (fast) rc = orc_fully_connected_f32_fast(batch, K, O, fin, fw, fb, transpose_weights, fo);
    else      rc = orc_fully_connected_f32(batch, K, O, fin, fw, fb, transpose_weights, fo);
    if (rc == 0) rc = orc_encode_tensor(fo, n_out, out);
done:
    free(fin); free(fw); free(fo); free(fb);
    return rc;
}

/* RefActivationWorkload.cpp:23-36: out.Set(Activation(in.Get())) element by element */
int orc_activation(const orc_tensor* in, const orc_tensor* out, int function, float a, float b)
{
    const size_t n = num_elements(in);
    float* f = (float*)malloc((n + 1) * sizeof(float));
    if (!f) return fail("out of memory");
    int rc = orc_decode_tensor(in, 0, f);
    if (rc == 0)
    {
        for (size_t i = 0; i < n; ++i) f[i] = orc_activation_f32(f[i], function, a, b);
        rc = orc_encode_tensor(f, n, out);
    }
    free(f);
    return rc;
}

/* ------------------------------------------------------------------------------------------------
 * Pooling2d -- workloads/Pooling2d.cpp:142-303 (Max / Average; Exclude / IgnoreValue padding)
 * ---------------------------------------------------------------------------------------------- */
static int clamp_range(int* start, int* end, int max_range)
{
    if (*start < 0 || *end > max_range)
    {
        int s = *start < 0 ? 0 : *start; s = s < max_range ? s : max_range;
        int e = *end < 0 ? 0 : *end;     e = e < max_range ? e : max_range;
        *start = s; *end = e;
        return 1;
    }
    return 0;
}

static int on_padding_only(int start, int end, int max_range) { return end <= 0 || start > max_range; }

int orc_pooling2d(const orc_tensor* in, const orc_tensor* out, const orc_pool_params* p, int data_layout)
{
    if (in->ndim != 4 || out->ndim != 4) return fail("pooling tensors must be 4-D");
    if (p->pool_type != ORC_POOL_MAX && p->pool_type != ORC_POOL_AVERAGE) return fail("Unsupported pooling algorithm");
    const int nhwc = data_layout == ORC_NHWC;
    const unsigned c_idx = nhwc ? 3 : 1, h_idx = nhwc ? 1 : 2, w_idx = nhwc ? 2 : 3;
    const int batchSize = (int)out->shape[0], channels = (int)out->shape[c_idx];
    const int heightOutput = (int)out->shape[h_idx], widthOutput = (int)out->shape[w_idx];
    const int heightInput = (int)in->shape[h_idx], widthInput = (int)in->shape[w_idx];
    const int padLeft = (int)p->pad_left, padRight = (int)p->pad_right;
    const int padTop = (int)p->pad_top, padBottom = (int)p->pad_bottom;
    const int strideX = (int)p->stride_x, strideY = (int)p->stride_y;
    const int poolHeight = (int)p->pool_h, poolWidth = (int)p->pool_w;
    const float init = p->pool_type == ORC_POOL_MAX ? -FLT_MAX : 0.0f;

    const size_t n_in = num_elements(in), n_out = num_elements(out);
    float* fin = (float*)malloc((n_in + 1) * sizeof(float));
    float* fo  = (float*)malloc((n_out + 1) * sizeof(float));
    int rc = -1;
    if (!fin || !fo) { fail("out of memory"); goto done; }
    if (orc_decode_tensor(in, 0, fin)) goto done;

    for (int n = 0; n < batchSize; n++)
    for (int c = 0; c < channels; c++)
    for (int yOutput = 0; yOutput < heightOutput; yOutput++)
    {
        int hstart = yOutput * strideY - padTop;
        int hend = hstart + poolHeight;
        hend = hend < heightInput + padBottom ? hend : heightInput + padBottom;
        int height = hend - hstart;
        int hclamped = clamp_range(&hstart, &hend, heightInput);
        for (int xOutput = 0; xOutput < widthOutput; xOutput++)
        {
            int wstart = xOutput * strideX - padLeft;
            int wend = wstart + poolWidth;
            wend = wend < widthInput + padRight ? wend : widthInput + padRight;
            float result = init;
            float poolAreaSize = (float)(height * (wend - wstart));
            int outputIndex = nhwc
                ? n * heightOutput * widthOutput * channels + yOutput * widthOutput * channels + xOutput * channels + c
                : n * heightOutput * widthOutput * channels + c * heightOutput * widthOutput + yOutput * widthOutput + xOutput;
            if (on_padding_only(hstart, hend, heightInput) || on_padding_only(wstart, wend, widthInput))
            {
                fo[outputIndex] = 0.0f;
                continue;
            }
            /* Pooling2d.cpp:243 `bool clamped = hclamped |= ClampRange(...)`: the flag carries along the row */
            hclamped |= clamp_range(&wstart, &wend, widthInput);
            int clamped = hclamped;
            if (clamped && p->padding_method == ORC_PAD_EXCLUDE)
                poolAreaSize = (float)((hend - hstart) * (wend - wstart));
            for (int yInput = hstart; yInput < hend; yInput++)
            for (int xInput = wstart; xInput < wend; xInput++)
            {
                int inputIndex = nhwc
                    ? n * heightInput * widthInput * channels + yInput * widthInput * channels + xInput * channels + c
                    : n * heightInput * widthInput * channels + c * heightInput * widthInput + yInput * widthInput + xInput;
                float v = fin[inputIndex];
                if (p->pool_type == ORC_POOL_MAX) { if (v > result) result = v; }
                else result += v;
            }
            if (p->pool_type == ORC_POOL_AVERAGE) result /= poolAreaSize;
            fo[outputIndex] = result;
        }
    }
    rc = orc_encode_tensor(fo, n_out, out);
done:
    free(fin); free(fo);
    return rc;
}

/* ------------------------------------------------------------------------------------------------
 * Softmax -- workloads/Softmax.cpp:16-69
 * ---------------------------------------------------------------------------------------------- */
int orc_softmax(const orc_tensor* in, const orc_tensor* out, float beta, int axis)
{
    const int nd = (int)in->ndim;
    if (axis >= nd || axis < -nd) return fail("softmax axis out of range");
    const unsigned uAxis = axis < 0 ? (unsigned)(nd - abs(axis)) : (unsigned)axis;
    size_t outerSize = 1, innerSize = 1;
    for (unsigned i = 0; i < uAxis; ++i) outerSize *= in->shape[i];
    for (unsigned i = uAxis + 1; i < in->ndim; ++i) innerSize *= in->shape[i];
    const size_t axisSize = in->shape[uAxis];
    const size_t n = num_elements(in);
    float* fin = (float*)malloc((n + 1) * sizeof(float));
    float* fo  = (float*)malloc((n + 1) * sizeof(float));
    int rc = -1;
    if (!fin || !fo) { fail("out of memory"); goto done; }
    if (orc_decode_tensor(in, 0, fin)) goto done;
    for (size_t outer = 0; outer < outerSize; ++outer)
    for (size_t inner = 0; inner < innerSize; ++inner)
    {
        const size_t begin = outer * axisSize * innerSize + inner;
        float maxValue = -FLT_MAX;
        for (size_t i = 0; i < axisSize; ++i) { float v = fin[begin + i * innerSize]; maxValue = maxValue < v ? v : maxValue; }
        float sum = 0.0f;
        for (size_t i = 0; i < axisSize; ++i) sum += expf((fin[begin + i * innerSize] - maxValue) * beta);
        for (size_t i = 0; i < axisSize; ++i) fo[begin + i * innerSize] = expf((fin[begin + i * innerSize] - maxValue) * beta) / sum;
    }
    rc = orc_encode_tensor(fo, n, out);
done:
    free(fin); free(fo);
    return rc;
}

/* ------------------------------------------------------------------------------------------------
 * ElementwiseBinary Add -- RefElementwiseBinaryWorkload.cpp:27-107 (float decoders, std::plus) with
 * the broadcast strides of Broadcast.cpp:11-33 (a dimension of extent 1 has stride 0).
 * ---------------------------------------------------------------------------------------------- */
int orc_add(const orc_tensor* in0, const orc_tensor* in1, const orc_tensor* out)
{
    const uint32_t nd = out->ndim;
    if (in0->ndim != nd || in1->ndim != nd || nd > 6) return fail("add: ranks must match (<=6)");
    const size_t n0 = num_elements(in0), n1 = num_elements(in1), no = num_elements(out);
    float* f0 = (float*)malloc((n0 + 1) * sizeof(float));
    float* f1 = (float*)malloc((n1 + 1) * sizeof(float));
    float* fo = (float*)malloc((no + 1) * sizeof(float));
    int rc = -1;
    if (!f0 || !f1 || !fo) { fail("out of memory"); goto done; }
    if (orc_decode_tensor(in0, 0, f0) || orc_decode_tensor(in1, 0, f1)) goto done;
    size_t s0[6], s1[6];
    {
        size_t a = 1, b = 1;
        for (int j = (int)nd - 1; j >= 0; --j)
        {
            s0[j] = in0->shape[j] > 1 ? a : 0;
            s1[j] = in1->shape[j] > 1 ? b : 0;
            a *= in0->shape[j]; b *= in1->shape[j];
        }
    }
    for (size_t i = 0; i < no; ++i)
    {
        size_t rem = i, o0 = 0, o1 = 0;
        for (int j = (int)nd - 1; j >= 0; --j)
        {
            size_t idx = rem % out->shape[j]; rem /= out->shape[j];
            o0 += idx * s0[j]; o1 += idx * s1[j];
        }
        fo[i] = f0[o0] + f1[o1];
    }
    rc = orc_encode_tensor(fo, no, out);
done:
    free(f0); free(f1); free(fo);
    return rc;
}

/* ------------------------------------------------------------------------------------------------
 * Pad -- workloads/Pad.cpp:39-236.  The output is first filled with the pad value; for quantized
 * outputs through an encoder of scale 1 and offset 0 (Pad.cpp:77-84), so the value is a code.  Then
 * every input element is decoded with the input's quantization and encoded with the output's at
 * its shifted position (Pad.cpp:93-233; the nested loops there are this one index walk).
 * ---------------------------------------------------------------------------------------------- */
int orc_pad(const orc_tensor* in, const orc_tensor* out, const uint32_t* pad_before, float pad_value)
{
    const uint32_t nd = in->ndim;
    if (out->ndim != nd || nd == 0 || nd > 6) return fail("pad: ranks must match (1..6)");
    for (uint32_t d = 0; d < nd; ++d)
        if (pad_before[d] + in->shape[d] > out->shape[d]) return fail("pad: output too small");
    const size_t n_in = num_elements(in), n_out = num_elements(out);
    const size_t esz = out->dtype == ORC_FLOAT32 ? 4 : 1;
    float* f = (float*)malloc(((n_in > n_out ? n_in : n_out) + 1) * sizeof(float));
    uint8_t* packed = (uint8_t*)malloc(n_in * esz + 1);
    int rc = -1;
    if (!f || !packed) { fail("out of memory"); goto done; }
    {
        static const float one = 1.0f;
        orc_tensor fill = *out;
        if (out->dtype != ORC_FLOAT32) { fill.scales = &one; fill.n_scales = 1; fill.quant_dim = -1; fill.offset = 0; }
        for (size_t i = 0; i < n_out; ++i) f[i] = pad_value;
        if (orc_encode_tensor(f, n_out, &fill)) goto done;
    }
    if (orc_decode_tensor(in, 0, f)) goto done;
    {
        orc_tensor compact = *out;
        compact.data = packed;
        if (orc_encode_tensor(f, n_in, &compact)) goto done;
    }
    for (size_t i = 0; i < n_in; ++i)
    {
        size_t rem = i, o = 0, stride = 1;
        for (int d = (int)nd - 1; d >= 0; --d)
        {
            size_t idx = rem % in->shape[d]; rem /= in->shape[d];
            o += (idx + pad_before[d]) * stride;
            stride *= out->shape[d];
        }
        memcpy((uint8_t*)out->data + o * esz, packed + i * esz, esz);
    }
    rc = 0;
done:
    free(f); free(packed);
    return rc;
}
