// Device-side arithmetic shared by every kernel: the requantization epilogue.
#pragma once

#include <hip/hip_runtime.h>

#include <cmath>

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

// Per-channel constants, eight rows of `stride` floats, built on the host (conv.hip):
//   row 0 mult   s_in * s_w[c]                      row 1 biasf  float(bias[c]) * s_b[c]
//   rows 2..5    m+, b+, m-, b-   the bracket of the fast path (below); b carries offset' = offset + Requant::pk_bias
//                                 (codes as unsigned bytes)
//   rows 6, 7    bc+, bc-         b+ and b- with corr * m+ / corr * m- added
// Rows 6/7 serve kernels whose accumulators start at zero: the zero-point correction corr[c] is then part of the
// fast-path constants, and only the exact path adds it to the accumulator as an integer.
struct ChanTab
{
    const float* p;
    int stride;
};

// Fast path with an exact fallback.
//   With rho = float(acc) * fm + fb in real arithmetic (fm = fl(mult * fl(1/s_out)), fb = fl(fl(biasf * fl(1/s_out)) + offset'))
//   and t = fl(f / s_out) + offset' the reference's value before rounding (f = fl(fl(float(acc) * mult) + biasf)), counting
//   every rounding on both sides (three in the reference, five in the constants) gives
//       |t - rho|  <=  2^-24 * (5 |rho| + 10 |biasf / s_out| + 6 |offset'|),
//   two more |rho| where a kernel converts an accumulator beyond 2^24 without its zero-point correction.
//   The host widens that to a bracket r- < t < r+ that costs one FMA per side,
//       r+ = fma(float(acc), m+, b+),   m+ = fm (1 + e),  b+ = fb (1 + e) + c
//       r- = fma(float(acc), m-, b-),   m- = fm (1 - e),  b- = fb (1 - e) - c
//   with e = 16 * 2^-24 and c a per-channel constant that also covers the roundings of m+-, b+- and of the FMA itself
//   (conv.hip, 1.5x margin on every term; valid while -1 <= rho <= 257, and beyond that range both sides saturate).
//   v_cvt_pk_u8_f32 rounds to nearest (ties to even) and saturates to 0..255, both monotone, so when r- and r+ convert
//   to the same byte, t -- strictly between them -- rounds to that byte under any tie rule, the reference's half-away-
//   from-zero included.  Values whose two bytes differ (about two in 10^4: r lies that close to a half-integer) are
//   recomputed with the reference's own sequence.  A channel without a fast path has m+ = m- = 0, b+ = 255, b- = 0.
//   The activation's clamp, where it is narrower than 0..255, is applied to both sides before converting.

// Stores of layer outputs.  An ordinary store leaves its line dirty in the XCD's L2 until the end-of-kernel write-back,
// which then moves the whole output tensor (up to the 32 MB the eight L2s hold) after the last wave has finished, with
// nothing to overlap it.  With the sc1 bit (agent scope) the L2 writes the line through as the store is issued, so the
// write-back runs beside the rest of the kernel and the data is where the next kernel -- whose blocks run on any XCD --
// reads it from.  (The nt bit instead also helps a kernel timed alone but makes the next layer slower.)  Only for stores
// of 16 bytes per lane that cover whole lines per instruction: the depthwise blocks' and the pooling kernel's dwords,
// written through one by one, are slower than ordinary stores that L2 merges.
//   The bit is set through the buffer-store builtins (their cache-policy argument), which the compiler knows as vector
// memory instructions; a hand-written store instruction in inline assembly is invisible to its hazard and wait-count
// bookkeeping and produced wrong bytes now and then.  A buffer store takes a wave-uniform base and an unsigned 32-bit
// byte offset, so tensors of 4 GiB and more fall back to ordinary stores.
#ifndef MI355X_STORE_THROUGH
#define MI355X_STORE_THROUGH 1
#endif
typedef int StoreVec4 __attribute__((ext_vector_type(4)));

struct OutPtr
{
    __amdgpu_buffer_rsrc_t rsrc;
    uint8_t* base;
    bool through;
};

// `base` must be the same in every lane of the wave (a kernel argument, or derived from block-uniform values)
__device__ __forceinline__ OutPtr MakeOutPtr(uint8_t* base, long long bytes)
{
    OutPtr o;
    o.base = base;
    o.through = MI355X_STORE_THROUGH != 0 && bytes > 0 && bytes <= 0xffffffffll;
    o.rsrc = __builtin_amdgcn_make_buffer_rsrc(base, 0, -1, 0x00020000);
    return o;
}

constexpr int kStoreAuxSc1 = 16;     // cache-policy operand of the buffer-store builtins: bit 4 = sc1

__device__ __forceinline__ void StoreOut16(const OutPtr& o, long long offset, const StoreVec4& v)
{
    typedef unsigned int U4 __attribute__((ext_vector_type(4)));
    if (o.through) __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(U4, v), o.rsrc, static_cast<int>(offset), 0, kStoreAuxSc1);
    else *reinterpret_cast<StoreVec4*>(o.base + offset) = v;
}

__device__ __forceinline__ uint32_t Pack4(int q0, int q1, int q2, int q3)
{
    // four codes -> one dword (byte 0 = q0), three v_perm_b32
    const uint32_t t0 = __builtin_amdgcn_perm(static_cast<uint32_t>(q1), static_cast<uint32_t>(q0), 0x0c0c0400u);
    const uint32_t t1 = __builtin_amdgcn_perm(static_cast<uint32_t>(q3), static_cast<uint32_t>(q2), 0x0c0c0400u);
    return __builtin_amdgcn_perm(t1, t0, 0x05040100u);
}

struct Fast4
{
    float4 mp, bp, mm, bm;   // rows 2..5: the bracket (the rare exact path fetches rows 0 / 1 when it is entered)
};

__device__ __forceinline__ Fast4 LoadFast4(const ChanTab& ct, int c)
{
    Fast4 f;
    f.mp = *reinterpret_cast<const float4*>(ct.p + 2 * ct.stride + c);
    f.bp = *reinterpret_cast<const float4*>(ct.p + 3 * ct.stride + c);
    f.mm = *reinterpret_cast<const float4*>(ct.p + 4 * ct.stride + c);
    f.bm = *reinterpret_cast<const float4*>(ct.p + 5 * ct.stride + c);
    return f;
}

// Four consecutive channels c..c+3 of one pixel -> packed dword.
// Five VALU instructions per value on the fast path (convert, two FMAs, two converting packs; two v_med3 more when the
// activation clamps inside 0..255) and one compare and scalar branch per quad.  When some lane of the wave has a byte
// that differs between the two sides, the wave redoes that position of the quad with the reference's sequence on every
// lane (always right, and cheaper than sorting out which lanes need it); LOAD_EXACT supplies rows 0 / 1 of the table
// and, for kernels whose accumulators start at zero, the zero-point correction that only the exact path adds as an
// integer.  The constants are finite (the host checks them and the accumulator range), so no NaN reaches a conversion.
template <typename LoadExact>
__device__ __forceinline__ uint32_t Requant4Core(int a0, int a1, int a2, int a3, const float4& mp, const float4& bp,
                                                 const float4& mm, const float4& bm, const Requant& rq, LoadExact load_exact)
{
    const float f0 = static_cast<float>(a0), f1 = static_cast<float>(a1), f2 = static_cast<float>(a2), f3 = static_cast<float>(a3);
    float p0 = __fmaf_rn(f0, mp.x, bp.x), p1 = __fmaf_rn(f1, mp.y, bp.y), p2 = __fmaf_rn(f2, mp.z, bp.z), p3 = __fmaf_rn(f3, mp.w, bp.w);
    float q0 = __fmaf_rn(f0, mm.x, bm.x), q1 = __fmaf_rn(f1, mm.y, bm.y), q2 = __fmaf_rn(f2, mm.z, bm.z), q3 = __fmaf_rn(f3, mm.w, bm.w);
    if (!rq.pk_full)
    {
        p0 = __builtin_amdgcn_fmed3f(p0, rq.pk_lo_f, rq.pk_hi_f); q0 = __builtin_amdgcn_fmed3f(q0, rq.pk_lo_f, rq.pk_hi_f);
        p1 = __builtin_amdgcn_fmed3f(p1, rq.pk_lo_f, rq.pk_hi_f); q1 = __builtin_amdgcn_fmed3f(q1, rq.pk_lo_f, rq.pk_hi_f);
        p2 = __builtin_amdgcn_fmed3f(p2, rq.pk_lo_f, rq.pk_hi_f); q2 = __builtin_amdgcn_fmed3f(q2, rq.pk_lo_f, rq.pk_hi_f);
        p3 = __builtin_amdgcn_fmed3f(p3, rq.pk_lo_f, rq.pk_hi_f); q3 = __builtin_amdgcn_fmed3f(q3, rq.pk_lo_f, rq.pk_hi_f);
    }
    // round to nearest, saturate to 0..255 and pack, one instruction per value
    uint32_t out = __builtin_amdgcn_cvt_pk_u8_f32(p0, 0, 0u);
    out = __builtin_amdgcn_cvt_pk_u8_f32(p1, 1, out);
    out = __builtin_amdgcn_cvt_pk_u8_f32(p2, 2, out);
    out = __builtin_amdgcn_cvt_pk_u8_f32(p3, 3, out);
    uint32_t low = __builtin_amdgcn_cvt_pk_u8_f32(q0, 0, 0u);
    low = __builtin_amdgcn_cvt_pk_u8_f32(q1, 1, low);
    low = __builtin_amdgcn_cvt_pk_u8_f32(q2, 2, low);
    low = __builtin_amdgcn_cvt_pk_u8_f32(q3, 3, low);
    const uint32_t differ = out ^ low;
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(differ != 0u) != 0, 0))
    {
        float4 m, b;
        int4 cr;
        load_exact(m, b, cr);
        // usually one value of the wave's 256 is flagged: only its position is redone (on every lane: the exact result is
        // always the right one)
        if (__builtin_amdgcn_ballot_w64((differ & 0x000000ffu) != 0u) != 0)
            out = (out & 0xffffff00u) | (static_cast<uint32_t>(RequantExactDev(a0 + cr.x, m.x, b.x, rq) + rq.pk_bias) & 0xffu);
        if (__builtin_amdgcn_ballot_w64((differ & 0x0000ff00u) != 0u) != 0)
            out = (out & 0xffff00ffu) | ((static_cast<uint32_t>(RequantExactDev(a1 + cr.y, m.y, b.y, rq) + rq.pk_bias) & 0xffu) << 8);
        if (__builtin_amdgcn_ballot_w64((differ & 0x00ff0000u) != 0u) != 0)
            out = (out & 0xff00ffffu) | ((static_cast<uint32_t>(RequantExactDev(a2 + cr.z, m.z, b.z, rq) + rq.pk_bias) & 0xffu) << 16);
        if (__builtin_amdgcn_ballot_w64((differ & 0xff000000u) != 0u) != 0)
            out = (out & 0x00ffffffu) | ((static_cast<uint32_t>(RequantExactDev(a3 + cr.w, m.w, b.w, rq) + rq.pk_bias) & 0xffu) << 24);
    }
    return out ^ rq.pk_xor;
}

// Bracket constants given row by row (kernels that keep rows 2, 6, 4, 7 -- the corr-folded bracket -- in LDS or registers).
// `corr` (may be null) is an integer added to the accumulator on the exact path only.
__device__ __forceinline__ uint32_t Requant4Dev(int a0, int a1, int a2, int a3, const float4& mp, const float4& bp,
                                                const float4& mm, const float4& bm, const ChanTab& ct, const int32_t* corr, int c,
                                                const Requant& rq)
{
    return Requant4Core(a0, a1, a2, a3, mp, bp, mm, bm, rq, [&](float4& m, float4& b, int4& cr) {
        m = *reinterpret_cast<const float4*>(ct.p + c);
        b = *reinterpret_cast<const float4*>(ct.p + ct.stride + c);
        cr = int4{0, 0, 0, 0};
        if (corr) cr = *reinterpret_cast<const int4*>(corr + c);
    });
}

// constants of rows 2..5 (accumulator already contains the zero-point correction)
__device__ __forceinline__ uint32_t Requant4Dev(int a0, int a1, int a2, int a3, const Fast4& f, const ChanTab& ct, int c,
                                                const Requant& rq)
{
    return Requant4Dev(a0, a1, a2, a3, f.mp, f.bp, f.mm, f.bm, ct, nullptr, c, rq);
}

// one channel (scalar kernels): the same bracket, compared after rounding
__device__ __forceinline__ int RequantBracket1(int acc, int exact_acc, float mp, float bp, float mm, float bm, float m0, float b0, const Requant& rq)
{
    const float f = static_cast<float>(acc);
    const float kp = __builtin_rintf(__builtin_amdgcn_fmed3f(__fmaf_rn(f, mp, bp), rq.pk_lo_f, rq.pk_hi_f));
    const float km = __builtin_rintf(__builtin_amdgcn_fmed3f(__fmaf_rn(f, mm, bm), rq.pk_lo_f, rq.pk_hi_f));
    if (__builtin_expect(!(kp == km), 0)) return RequantExactDev(exact_acc, m0, b0, rq);
    return static_cast<int>(kp) - rq.pk_bias;
}

__device__ __forceinline__ int Requant1Dev(int acc, const ChanTab& ct, int c, const Requant& rq)
{
    return RequantBracket1(acc, acc, ct.p[2 * ct.stride + c], ct.p[3 * ct.stride + c], ct.p[4 * ct.stride + c], ct.p[5 * ct.stride + c],
                           ct.p[c], ct.p[ct.stride + c], rq);
}

// one channel, accumulator started at zero: rows 2/6/4/7 on the fast path, `corr[c]` joins the accumulator on the exact path
__device__ __forceinline__ int Requant1FoldedDev(int acc, const ChanTab& ct, const int32_t* corr, int c, const Requant& rq)
{
    return RequantBracket1(acc, acc + corr[c], ct.p[2 * ct.stride + c], ct.p[6 * ct.stride + c], ct.p[4 * ct.stride + c], ct.p[7 * ct.stride + c],
                           ct.p[c], ct.p[ct.stride + c], rq);
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

struct QIn
{
    float scale;
    int   offset;
    int   is_u8;
};

__device__ __forceinline__ float DequantDev(uint8_t code, const QIn& q)
{
    const int v = q.is_u8 ? static_cast<int>(code) : static_cast<int>(static_cast<int8_t>(code));
    return __fmul_rn(static_cast<float>(v - q.offset), q.scale);   // armnn::Dequantize, TypesUtils.cpp:47-56
}

// The four codes of a dword -> float values: signed codes are made unsigned with one xor for the dword (offset moves by
// 128 with them), then v_cvt_f32_ubyteN converts byte N directly; value - offset is an exact small integer either way,
// so the single multiplication rounds exactly as in armnn::Dequantize.
__device__ __forceinline__ void Dequant4Dev(uint32_t w, const QIn& q, float (&v)[4])
{
    const uint32_t u = q.is_u8 ? w : (w ^ 0x80808080u);
    const float off = static_cast<float>(q.is_u8 ? q.offset : q.offset + 128);
    v[0] = __fmul_rn(__fsub_rn(static_cast<float>(u & 0xffu), off), q.scale);
    v[1] = __fmul_rn(__fsub_rn(static_cast<float>((u >> 8) & 0xffu), off), q.scale);
    v[2] = __fmul_rn(__fsub_rn(static_cast<float>((u >> 16) & 0xffu), off), q.scale);
    v[3] = __fmul_rn(__fsub_rn(static_cast<float>(u >> 24), off), q.scale);
}

inline QIn MakeQIn(const mi355x_quant& q)
{
    QIn r;
    r.scale = q.scale;
    r.offset = q.offset;
    r.is_u8 = q.dtype == MI355X_QASYMM_U8;
    return r;
}

// An Addition of two quantized tensors: dequantize both, one fp32 add, quantize with the Addition's output quantization and
// its fused activation (RefElementwiseBinaryWorkload.cpp:27-107 over Decoder / Encoder).  Used by the Addition layer's
// kernel and, inside a convolution's write-out, for the Addition that follows the convolution (`own`: the convolution's
// finished output codes with quantization qa, `other`: the Addition's other input with qr) -- so the bytes are those of
// the two layers run apart.
//   The reference's sequence costs 14 vector instructions per value (two dequantizations of three, the add, a quantization
//   with its own tie test).  The value before rounding is, in exact arithmetic, a linear function of the two codes,
//     T = ua ka + ub kb + k0,   ka = sa / so, kb = sr / so, k0 = offset_out + pk_bias - oa ka - or kb   (ua, ub: codes as 0..255),
//   and the reference's own fp32 value P' (its four roundings: two products, the sum, the division) lies within
//   3.01 * 2^-24 * 255 (ka + kb) of T.  t+ = fma(ua, ka, fma(ub, kb, k0 + c)) and t- = t+ - 2c, with c above that distance plus
//   the roundings of the constants, of the two FMAs and of the subtraction (for |T| <= 512: 2^-24 (1533 ka + 1278 kb + 2048)
//   in all; c = 1.5 x that), enclose P'; beyond |T| = 512 all three saturate alike.  When t- and t+ convert to the same byte
//   (v_cvt_pk_u8_f32: round to nearest, saturate; monotone), P' -- strictly between them -- rounds to that byte under any
//   tie rule.  Otherwise (a few values in 10^4) that value is redone with the reference's sequence.  Seven instructions
//   per value on the fast path, nine when the activation clamps inside 0..255.
struct AddFuse
{
    QIn qa, qr;
    Requant rq;
    float ka, kb, k0p, two_c;
    int bracket_ok;
};

inline AddFuse MakeAddFuse(const mi355x_quant& a, const mi355x_quant& r, const mi355x_quant& out, int32_t activation, float act_a, float act_b)
{
    AddFuse f;
    f.qa = MakeQIn(a);
    f.qr = MakeQIn(r);
    f.rq = MakeRequant(out, activation, act_a, act_b);
    const double so = static_cast<double>(out.scale);
    const double ka = static_cast<double>(a.scale) / so, kb = static_cast<double>(r.scale) / so;
    const double oa = f.qa.is_u8 ? a.offset : a.offset + 128, ob = f.qr.is_u8 ? r.offset : r.offset + 128;
    const double k0 = static_cast<double>(out.offset) + f.rq.pk_bias - oa * ka - ob * kb;
    const double c = 1.5 * (1533.0 * ka + 1278.0 * kb + 2048.0) / 16777216.0;
    f.ka = static_cast<float>(ka);
    f.kb = static_cast<float>(kb);
    f.k0p = static_cast<float>(k0 + c);
    f.two_c = nextafterf(static_cast<float>(2.0 * c), 1.0e30f);
    f.bracket_ok = f.rq.fast_ok && std::isnormal(f.ka) && std::isnormal(f.kb) && ka < 1024.0 && kb < 1024.0 && std::fabs(k0) < 1048576.0 &&
                   oa >= 0.0 && oa <= 255.0 && ob >= 0.0 && ob <= 255.0;     // offsets inside the type's range: |code - offset| <= 255
    return f;
}

// four codes of each input (dwords wa, wb) -> packed dword of the four sums' codes.  CLAMP = false: the caller knows that the
// activation's clamp is the type's own range (rq.pk_full), which the conversion already applies.
template <bool CLAMP = true>
__device__ __forceinline__ uint32_t AddQuantize4Dev(uint32_t wa, uint32_t wb, const AddFuse& f)
{
    if (!f.bracket_ok)
    {
        float va[4], vb[4];
        Dequant4Dev(wa, f.qa, va);
        Dequant4Dev(wb, f.qr, vb);
        return QuantizePack4Dev(__fadd_rn(va[0], vb[0]), __fadd_rn(va[1], vb[1]), __fadd_rn(va[2], vb[2]), __fadd_rn(va[3], vb[3]), f.rq);
    }
    const uint32_t ua = f.qa.is_u8 ? wa : (wa ^ 0x80808080u), ub = f.qr.is_u8 ? wb : (wb ^ 0x80808080u);
    const float af[4] = {static_cast<float>(ua & 0xffu), static_cast<float>((ua >> 8) & 0xffu), static_cast<float>((ua >> 16) & 0xffu), static_cast<float>(ua >> 24)};
    const float bf[4] = {static_cast<float>(ub & 0xffu), static_cast<float>((ub >> 8) & 0xffu), static_cast<float>((ub >> 16) & 0xffu), static_cast<float>(ub >> 24)};
    uint32_t out = 0u, low = 0u;
#pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        float p = __fmaf_rn(af[i], f.ka, __fmaf_rn(bf[i], f.kb, f.k0p));
        float m = __fsub_rn(p, f.two_c);
        if constexpr (CLAMP)
        {
            p = __builtin_amdgcn_fmed3f(p, f.rq.pk_lo_f, f.rq.pk_hi_f);
            m = __builtin_amdgcn_fmed3f(m, f.rq.pk_lo_f, f.rq.pk_hi_f);
        }
        out = __builtin_amdgcn_cvt_pk_u8_f32(p, i, out);
        low = __builtin_amdgcn_cvt_pk_u8_f32(m, i, low);
    }
    const uint32_t differ = out ^ low;
    if (__builtin_expect(differ != 0u, 0))
    {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if ((differ >> (8 * i)) & 0xffu)
            {
                const float s = __fadd_rn(DequantDev(static_cast<uint8_t>(wa >> (8 * i)), f.qa), DequantDev(static_cast<uint8_t>(wb >> (8 * i)), f.qr));
                out = (out & ~(0xffu << (8 * i))) | ((static_cast<uint32_t>(QuantizeDev(s, f.rq) + f.rq.pk_bias) & 0xffu) << (8 * i));
            }
    }
    return out ^ f.rq.pk_xor;
}

__device__ __forceinline__ StoreVec4 AddResidual16(const StoreVec4& own, const StoreVec4& other, const AddFuse& f)
{
    StoreVec4 o;
#pragma unroll
    for (int d = 0; d < 4; ++d) o[d] = static_cast<int>(AddQuantize4Dev<true>(static_cast<uint32_t>(own[d]), static_cast<uint32_t>(other[d]), f));
    return o;
}

} // namespace mi355x
