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

// int32 accumulator of sum (x - zx)(w - zw) -> output code, the reference's way:
//   f = float(acc) * (s_in * s_w[c]) + float(bias[c]) * s_b[c]      (separate multiply and add, no FMA)
// `mult` and `biasf` are prepared on the host in fp32 exactly as the reference's decoders would produce them.
__device__ __forceinline__ int RequantExactDev(int acc, float mult, float biasf, const Requant& rq)
{
    return QuantizeDev(__fadd_rn(__fmul_rn(static_cast<float>(acc), mult), biasf), rq);
}

// Per-channel constants, seven rows of `stride` floats, built on the host (conv.hip):
//   row 0 mult   s_in * s_w[c]                      row 1 biasf  float(bias[c]) * s_b[c]
//   row 2 fm     fl(mult * fl(1/s_out))             row 3 fb     fl(fl(biasf * fl(1/s_out)) + offset'),
//                                                    offset' = offset + Requant::pk_bias (codes as unsigned bytes)
//   row 4 thr    tie threshold for rows 2/3 (negative: the channel always takes the exact path)
//   row 5 fbc    fb + corr * fm                     row 6 thrc   tie threshold for rows 2/5
// Rows 5/6 serve kernels whose accumulators start at zero: the zero-point correction corr[c] is then part of the
// fast-path constant, and only the exact path adds it to the accumulator as an integer.
struct ChanTab
{
    const float* p;
    int stride;
};

// Fast path with an exact fallback.
//   r' = fma(float(acc), fm, fb) approximates  t = f/s_out + offset  (f = the reference's fp32 value).  Counting every
//   rounding on both sides (three in the reference; the reciprocal, two coefficient products, the offset add and the
//   fma on ours), each relative 2^-24 to a magnitude bounded through |r'|, one gets
//       |r' - (fl(f/s_out) + offset)|  <=  2^-24 * (8 |r'| + 9 |offset| + 9 |biasf/s_out| + 7 |corr*fm|)
//   (this includes the int32 -> fp32 conversion of accumulators beyond 2^24 on either path).
//   The two can therefore round to different integers only when r' lies that close to a half-integer.  The test
//       |r' - rint(r')|  <=  thr[c] - kTieSlope * |r'|,    thr[c] = 0.5 - 1.5 * 2^-24 * (9|offset| + 9|biasf/s_out| + 7|corr*fm| + 64)
//   (1.5x margin on every term) passes everything else; values that fail it -- a few in 10^4 -- are recomputed with
//   the reference's own sequence.  Results beyond the 8-bit range clamp alike on both paths.  Round-half-even
//   (v_rndne) serves on the fast path: it differs from round-half-away only at exact ties, which fail the test.
constexpr float kTieSlope = 12.0f / 16777216.0f;

__device__ __forceinline__ uint32_t Pack4(int q0, int q1, int q2, int q3)
{
    // four codes -> one dword (byte 0 = q0), three v_perm_b32
    const uint32_t t0 = __builtin_amdgcn_perm(static_cast<uint32_t>(q1), static_cast<uint32_t>(q0), 0x0c0c0400u);
    const uint32_t t1 = __builtin_amdgcn_perm(static_cast<uint32_t>(q3), static_cast<uint32_t>(q2), 0x0c0c0400u);
    return __builtin_amdgcn_perm(t1, t0, 0x05040100u);
}

struct Fast4
{
    float4 m, b, t;      // rows 2, 3, 4: the fast path
    float4 m0, b0;       // rows 0, 1: the exact path, fetched along so that entering it waits for nothing
};

__device__ __forceinline__ Fast4 LoadFast4(const ChanTab& ct, int c)
{
    Fast4 f;
    f.m = *reinterpret_cast<const float4*>(ct.p + 2 * ct.stride + c);
    f.b = *reinterpret_cast<const float4*>(ct.p + 3 * ct.stride + c);
    f.t = *reinterpret_cast<const float4*>(ct.p + 4 * ct.stride + c);
    f.m0 = *reinterpret_cast<const float4*>(ct.p + c);
    f.b0 = *reinterpret_cast<const float4*>(ct.p + ct.stride + c);
    return f;
}

// K = rint(r'), SLOW = the value needs the exact path ("not <=" also catches NaN)
#define MI355X_FAST1(ACC, M, B, T, K, SLOW)                                   \
    {                                                                         \
        const float r_ = __fmaf_rn(static_cast<float>(ACC), M, B);            \
        K = __builtin_rintf(r_);                                              \
        const float e_ = __fsub_rn(r_, K);                                    \
        SLOW = !(fabsf(e_) <= __fmaf_rn(fabsf(r_), -kTieSlope, T));           \
    }

// r' is first clamped to a quarter code beyond the activation's range [LO, HI] (biased domain): whatever lies further out
// ends at LO or HI on either path, its distance to an integer is then exactly 0.25, and it can never look like a tie.
// K = rint(r'), U = |r' - K| + kTieSlope |r'|: the value needs the exact path when U exceeds its channel's threshold.
#define MI355X_FAST1U(ACC, M, B, LO, HI, K, U)                                                        \
    {                                                                                                 \
        const float r_ = __builtin_amdgcn_fmed3f(__fmaf_rn(static_cast<float>(ACC), M, B), LO, HI);   \
        K = __builtin_rintf(r_);                                                                      \
        U = __fmaf_rn(fabsf(r_), kTieSlope, fabsf(__fsub_rn(r_, K)));                                 \
    }

// Four consecutive channels c..c+3 of one pixel -> packed dword.
// The fast path is branch-free, 7 VALU instructions per value plus a few per quad: the four tie measures are folded
// with v_max3 / v_max and compared once against the smallest of the four thresholds (a smaller threshold only sends
// more values to the exact path), so a quad costs one compare and one scalar branch.  r' is finite whenever a
// threshold is non-negative (the host checks the constants and the accumulator range), so no NaN can hide in the
// maxima; a channel without a fast path has threshold -1, which every measure exceeds.  When some lane of the wave has
// a flagged value, the wave redoes that value's position of the quad with the reference's sequence on every lane (always
// right, and cheaper than sorting out which lanes need it); LOAD_EXACT supplies rows 0 / 1 of the table and, for kernels
// whose accumulators start at zero, the zero-point correction that only the exact path adds as an integer.
template <typename LoadExact>
__device__ __forceinline__ uint32_t Requant4Core(int a0, int a1, int a2, int a3, const float4& fm, const float4& fb,
                                                 const float4& thr, const Requant& rq, LoadExact load_exact)
{
    float k0, k1, k2, k3, u0, u1, u2, u3;
    MI355X_FAST1U(a0, fm.x, fb.x, rq.pk_lo_q, rq.pk_hi_q, k0, u0)
    MI355X_FAST1U(a1, fm.y, fb.y, rq.pk_lo_q, rq.pk_hi_q, k1, u1)
    MI355X_FAST1U(a2, fm.z, fb.z, rq.pk_lo_q, rq.pk_hi_q, k2, u2)
    MI355X_FAST1U(a3, fm.w, fb.w, rq.pk_lo_q, rq.pk_hi_q, k3, u3)
    const float umax = fmaxf(fmaxf(fmaxf(u0, u1), u2), u3);       // v_max3_f32 + v_max_f32
    const float tmin = fminf(fminf(thr.x, thr.y), fminf(thr.z, thr.w));
    // integral floats within [LO, HI] -> unsigned bytes, one instruction per value, packed as it goes
    uint32_t out = __builtin_amdgcn_cvt_pk_u8_f32(k0, 0, 0u);
    out = __builtin_amdgcn_cvt_pk_u8_f32(k1, 1, out);
    out = __builtin_amdgcn_cvt_pk_u8_f32(k2, 2, out);
    out = __builtin_amdgcn_cvt_pk_u8_f32(k3, 3, out);
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(umax <= tmin)) != 0, 0))
    {
        float4 m, b;
        int4 cr;
        load_exact(m, b, cr);
        // usually one value of the wave's 256 is flagged: only its position is redone (on every lane: the exact result is
        // always the right one)
        if (__builtin_amdgcn_ballot_w64(!(u0 <= tmin)) != 0)
            out = (out & 0xffffff00u) | (static_cast<uint32_t>(RequantExactDev(a0 + cr.x, m.x, b.x, rq) + rq.pk_bias) & 0xffu);
        if (__builtin_amdgcn_ballot_w64(!(u1 <= tmin)) != 0)
            out = (out & 0xffff00ffu) | ((static_cast<uint32_t>(RequantExactDev(a1 + cr.y, m.y, b.y, rq) + rq.pk_bias) & 0xffu) << 8);
        if (__builtin_amdgcn_ballot_w64(!(u2 <= tmin)) != 0)
            out = (out & 0xff00ffffu) | ((static_cast<uint32_t>(RequantExactDev(a2 + cr.z, m.z, b.z, rq) + rq.pk_bias) & 0xffu) << 16);
        if (__builtin_amdgcn_ballot_w64(!(u3 <= tmin)) != 0)
            out = (out & 0x00ffffffu) | ((static_cast<uint32_t>(RequantExactDev(a3 + cr.w, m.w, b.w, rq) + rq.pk_bias) & 0xffu) << 24);
    }
    return out ^ rq.pk_xor;
}

// `corr` (may be null) is an integer added to the accumulator on the exact path only (rows 5/6, see ChanTab).
__device__ __forceinline__ uint32_t Requant4Dev(int a0, int a1, int a2, int a3, const float4& fm, const float4& fb,
                                                const float4& thr, const ChanTab& ct, const int32_t* corr, int c,
                                                const Requant& rq)
{
    return Requant4Core(a0, a1, a2, a3, fm, fb, thr, rq, [&](float4& m, float4& b, int4& cr) {
        m = *reinterpret_cast<const float4*>(ct.p + c);
        b = *reinterpret_cast<const float4*>(ct.p + ct.stride + c);
        cr = int4{0, 0, 0, 0};
        if (corr) cr = *reinterpret_cast<const int4*>(corr + c);
    });
}

// constants of rows 2,3,4 (accumulator already contains the zero-point correction), exact-path rows fetched beforehand
__device__ __forceinline__ uint32_t Requant4Dev(int a0, int a1, int a2, int a3, const Fast4& f, const ChanTab&, int,
                                                const Requant& rq)
{
    return Requant4Core(a0, a1, a2, a3, f.m, f.b, f.t, rq, [&](float4& m, float4& b, int4& cr) {
        m = f.m0;
        b = f.b0;
        cr = int4{0, 0, 0, 0};
    });
}

// one channel (scalar kernels)
__device__ __forceinline__ int Requant1Dev(int acc, const ChanTab& ct, int c, const Requant& rq)
{
    float k;
    bool slow;
    MI355X_FAST1(acc, ct.p[2 * ct.stride + c], ct.p[3 * ct.stride + c], ct.p[4 * ct.stride + c], k, slow)
    if (__builtin_expect(slow, 0)) return RequantExactDev(acc, ct.p[c], ct.p[ct.stride + c], rq);
    return static_cast<int>(__builtin_amdgcn_fmed3f(k, rq.pk_lo_f, rq.pk_hi_f)) - rq.pk_bias;
}

// one channel, accumulator started at zero: rows 2/5/6 on the fast path, `corr[c]` joins the accumulator on the exact path
__device__ __forceinline__ int Requant1FoldedDev(int acc, const ChanTab& ct, const int32_t* corr, int c, const Requant& rq)
{
    float k;
    bool slow;
    MI355X_FAST1(acc, ct.p[2 * ct.stride + c], ct.p[5 * ct.stride + c], ct.p[6 * ct.stride + c], k, slow)
    if (__builtin_expect(slow, 0)) return RequantExactDev(acc + corr[c], ct.p[c], ct.p[ct.stride + c], rq);
    return static_cast<int>(__builtin_amdgcn_fmed3f(k, rq.pk_lo_f, rq.pk_hi_f)) - rq.pk_bias;
}

// value already in float (pooling, add, ...): reciprocal fast path with the exact fallback near ties.
//   r' = fma(f, fl(1/scale), offset) is within 2^-24 * (|f/scale| + |r'|) of f/scale + offset and the correctly rounded
//   quotient within 2^-24 * |f/scale|; |offset| <= 255 is checked on the host (else fast_ok = 0).
__device__ __forceinline__ int QuantizeFastDev(float f, const Requant& rq)
{
    if (!rq.fast_ok) return QuantizeDev(f, rq);
    const float r = __fmaf_rn(f, rq.inv_scale, rq.out_offset_f);
    const float k = __builtin_rintf(r);
    const float e = __fsub_rn(r, k);
    // 3 |r'| + 2 |offset| <= 3 |r'| + 510, with the same 1.5x margin as above
    if (__builtin_expect(!(fabsf(e) <= __fmaf_rn(fabsf(r), -4.5f / 16777216.0f, 0.5f - 1024.0f / 16777216.0f)), 0))
        return QuantizeDev(f, rq);
    return static_cast<int>(__builtin_amdgcn_fmed3f(k, rq.act_lo_f, rq.act_hi_f));
}

// Four float values -> packed dword of output codes: QuantizeFastDev's test per value, then v_cvt_pk_u8_f32 (convert,
// saturate, pack) in the biased domain of Requant::pk_bias.  |offset + pk_bias| <= 383 here, hence the wider constant.
__device__ __forceinline__ uint32_t QuantizePack4Dev(float f0, float f1, float f2, float f3, const Requant& rq)
{
    if (!rq.fast_ok) return Pack4(QuantizeDev(f0, rq), QuantizeDev(f1, rq), QuantizeDev(f2, rq), QuantizeDev(f3, rq));
    const float off = rq.out_offset_f + static_cast<float>(rq.pk_bias);
    const float f[4] = {f0, f1, f2, f3};
    uint32_t out = 0u;
    unsigned slow = 0u;
#pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        const float r = __fmaf_rn(f[i], rq.inv_scale, off);
        float k = __builtin_rintf(r);
        const float e = __fsub_rn(r, k);
        if (!(fabsf(e) <= __fmaf_rn(fabsf(r), -4.5f / 16777216.0f, 0.5f - 1536.0f / 16777216.0f))) slow |= 1u << i;
        if (!rq.pk_full) k = __builtin_amdgcn_fmed3f(k, rq.pk_lo_f, rq.pk_hi_f);
        out = __builtin_amdgcn_cvt_pk_u8_f32(k, i, out);
    }
    if (__builtin_expect(slow != 0u, 0))
    {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (slow & (1u << i))
                out = (out & ~(0xffu << (8 * i))) | ((static_cast<uint32_t>(QuantizeDev(f[i], rq) + rq.pk_bias) & 0xffu) << (8 * i));
    }
    return out ^ rq.pk_xor;
}

} // namespace mi355x
