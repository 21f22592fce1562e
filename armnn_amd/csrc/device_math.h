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

// Same result as QuantizeDev, cheaper on average (9 VALU instructions + pack instead of ~30).
//   r' = fma(f, fl(1/scale), offset) differs from fl(f/scale) + offset by less than 2^-12 whenever |f/scale| <= 512
//   (reciprocal and fma rounding: (|r| + |r'|) * 2^-24; the correctly rounded quotient: |r| * 2^-24), so the two can
//   round to different integers only when r' lies within 2^-12 of a half-integer.  Those values (kTieWindow = 2^-11
//   either side: about 1 in 1000) take the exact division instead.  For |f/scale| > 512 both results are beyond the
//   8-bit range whatever the offset (|offset| <= 255, checked on the host) and clamp alike.
//   Round-half-even (v_rndne) serves on the fast path: it differs from round-half-away only at exact ties, which
//   are inside the window.
constexpr float kTieWindow = 1.0f / 2048.0f;

__device__ __forceinline__ int QuantizeFastDev(float f, const Requant& rq)
{
    const float r = __fmaf_rn(f, rq.inv_scale, rq.out_offset_f);
    const float k = __builtin_rintf(r);
    const float e = __fsub_rn(r, k);
    if (__builtin_expect(fabsf(e) > 0.5f - kTieWindow, 0)) return QuantizeDev(f, rq);
    return static_cast<int>(__builtin_amdgcn_fmed3f(k, rq.act_lo_f, rq.act_hi_f));
}

// int32 accumulator of sum (x - zx)(w - zw)  ->  output code.
//   f = float(acc) * (s_in * s_w[c]) + float(bias[c]) * s_b[c]      (separate multiply and add, no FMA)
// `mult` and `biasf` are prepared on the host in fp32 exactly as the reference's decoders would produce them.
__device__ __forceinline__ int RequantDev(int acc, float mult, float biasf, const Requant& rq)
{
    const float f = __fadd_rn(__fmul_rn(static_cast<float>(acc), mult), biasf);
    return rq.fast_ok ? QuantizeFastDev(f, rq) : QuantizeDev(f, rq);
}

// four codes -> one dword (byte 0 = q0), three v_perm_b32
__device__ __forceinline__ uint32_t Pack4(int q0, int q1, int q2, int q3)
{
    const uint32_t t0 = __builtin_amdgcn_perm(static_cast<uint32_t>(q1), static_cast<uint32_t>(q0), 0x0c0c0400u);
    const uint32_t t1 = __builtin_amdgcn_perm(static_cast<uint32_t>(q3), static_cast<uint32_t>(q2), 0x0c0c0400u);
    return __builtin_amdgcn_perm(t1, t0, 0x05040100u);
}

} // namespace mi355x
