// Device-side arithmetic shared by every kernel: the requantization epilogue.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"

namespace mi355x
{

// float value -> output code, exactly armnn::Quantize (src/armnn/TypesUtils.cpp:29-45):
//   clamp(float(offset) + round(value / scale), lowest, max), round = half away from zero, fp32 division,
// followed by the fused activation's integer clamp.
__device__ __forceinline__ int QuantizeDev(float f, const Requant& rq)
{
    float q = roundf(__fdiv_rn(f, rq.out_scale));
    float v = __fadd_rn(rq.out_offset_f, q);
    v = fmaxf(v, rq.type_min_f);
    v = fminf(v, rq.type_max_f);
    int r = static_cast<int>(v);
    r = max(r, rq.act_lo);
    r = min(r, rq.act_hi);
    return r;
}

// int32 accumulator of sum (x - zx)(w - zw)  ->  output code.
//   f = float(acc) * (s_in * s_w[c]) + float(bias[c]) * s_b[c]      (separate multiply and add, no FMA)
// `mult` and `biasf` are prepared on the host in fp32 exactly as the reference's decoders would produce them.
__device__ __forceinline__ int RequantDev(int acc, float mult, float biasf, const Requant& rq)
{
    float f = __fadd_rn(__fmul_rn(static_cast<float>(acc), mult), biasf);
    return QuantizeDev(f, rq);
}

} // namespace mi355x
