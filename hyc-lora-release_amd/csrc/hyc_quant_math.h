// Scalar arithmetic of the integer-code rule, shared by the HIP kernels and by a
// host-side exhaustive checker (plain C99 / C++; no HIP types in here).
//
// The code rule of the reference quantiser (operators/compress_function_kernel.py:92-110)
// is   t = fp32(x) / fp32(s) (+ z);  r = roundf(t);  r = clamp(r, -2^(q-1), 2^(q-1)-1);
//      code = r + 2^(q-1).
// x and s are bf16.  An IEEE fp32 division costs ~10 VALU operations per element on
// CDNA, and the quantiser is then bound by the vector ALU rather than by HBM.  Because x
// and s carry 8-bit significands, the real quotient x/s is either exactly a half-integer
// or at least ~2^-16 (relative) away from one, so the code is a function of the real
// quotient alone, and a slightly enlarged reciprocal per column reproduces it with one
// fused multiply-add (hyc_code_fast).  That the codes equal those of the IEEE division
// followed by roundf — for every bf16 x and every bf16 s accepted by hyc_scale_is_fast —
// is established exhaustively on the CPU by tests/native/check_fastdiv.c, which includes
// this very header.
#ifndef HYC_QUANT_MATH_H
#define HYC_QUANT_MATH_H

#include <math.h>
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define HYC_HD __host__ __device__ __forceinline__
#else
#define HYC_HD static inline
#endif

HYC_HD float hyc_bits_to_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

HYC_HD uint32_t hyc_f32_to_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    return u;
}

HYC_HD float hyc_bf16_to_f32(uint16_t h) { return hyc_bits_to_f32((uint32_t)h << 16); }

// Round-to-nearest-even fp32 -> bf16 (software form; the kernels use the hardware
// conversion of gfx950, which rounds the same way).
HYC_HD uint16_t hyc_f32_to_bf16(float f) {
    uint32_t u = hyc_f32_to_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// A column may use the reciprocal path when its step is an ordinary positive number
// whose reciprocal is an ordinary number too.  Everything else (0, negative, tiny,
// huge, inf, NaN) takes the IEEE division (hyc_code_from_t).
HYC_HD int hyc_scale_is_fast(float s) { return (s >= 1e-18f) && (s <= 1e18f); }

// roundf + clamp + offset.  t is clamped first (the bounds are integers, so clamping
// before rounding is the same as after); fmaxf maps NaN to the lower bound, i.e. code 0.
// trunc(t + copysign(0.5, t)) equals roundf(t) for |t| >= 0.5 and for every |t| < 0.5
// that is not within half an ulp of 0.5; 0.5 - 2^-25 is the only fp32 value where it
// differs, and a quotient of two bf16 numbers (8-bit significands) cannot be that
// close to a half-integer without being one.
HYC_HD int hyc_code_from_t(float t, int q_bit) {
    const float half = (float)(1 << (q_bit - 1));
    t = fminf(fmaxf(t, -half), half - 1.0f);
    float v = t + copysignf(0.5f, t);
    return (int)v + (1 << (q_bit - 1));
}

// The reciprocal path.  rn = (1/s) * (1 + 2^-18) is kept per column.  x * rn is the real
// quotient pushed away from zero by a relative 2^-18 (give or take the ~2^-23 of rounding
// rn and the product): an exact tie k + 0.5 lands strictly beyond the tie on the side
// roundf sends it to, and a quotient that is not a tie cannot be pushed across one (the
// nearest tie is >= 2^-16 away, relatively, for |x/s| <= 128.5).  After that no ties are
// left, so any round-to-nearest gives roundf's answer, and the cheapest one is the rounding
// of the fused multiply-add itself: adding 1.5 * 2^23 forces the sum's unit in the last place
// to 1, which leaves the integer - offset 2^(q-1) included - in the low mantissa bits.
// Clamping that float to [HYC_MAGIC, HYC_MAGIC + 2^q - 1] saturates the code (the bounds are
// integers, so clamping after rounding equals clamping before); infinities and overflowing
// products clamp like any large value, and a NaN, which fails the comparison, becomes the
// lower bound: code 0, as in the reference.  The code is the low byte of the result.
#define HYC_MAGIC 12582912.0f            /* 1.5 * 2^23 */
#define HYC_RECIP_NUDGE 1.000003814697265625f   /* 1 + 2^-18 */

HYC_HD float hyc_recip_nudged(float s) { return (1.0f / s) * HYC_RECIP_NUDGE; }

// The kernels take the reciprocal from the hardware approximation (v_rcp_f32, 1 ulp) instead of
// an IEEE division.  The code is monotone in rn, so it is enough that both ends of a band of
// relative half-width HYC_RECIP_SLACK around hyc_recip_nudged(s) give the right codes; the
// exhaustive checker tests exactly those two ends, and the band is 4x wider than the error of
// the approximation plus the rounding of the product.
#define HYC_RECIP_SLACK 4.76837158203125e-07f    /* 2^-21 */

// Host form (compare-and-select so that signalling NaNs are dropped too); the kernels do the
// clamp with one v_med3_f32.  Returns the float whose low byte is the biased code.
HYC_HD uint32_t hyc_code_word_fast(float x, float rn, int q_bit) {
    const float lo = HYC_MAGIC, hi = HYC_MAGIC + (float)((1 << q_bit) - 1);
    float m = fmaf(x, rn, HYC_MAGIC + (float)(1 << (q_bit - 1)));
    m = (m > lo) ? m : lo;
    m = fminf(m, hi);
    return hyc_f32_to_bits(m);
}
HYC_HD int hyc_code_fast(float x, float rn, int q_bit) { return (int)(hyc_code_word_fast(x, rn, q_bit) & 0xffu); }

// Same rule with plain roundf semantics (trunc, then an exact fraction test), for
// t = x/s + z: once an arbitrary zero point has been added the half-ulp argument above
// no longer holds.
HYC_HD int hyc_code_from_t_exact(float t, int q_bit) {
    const float half = (float)(1 << (q_bit - 1));
    t = fminf(fmaxf(t, -half), half - 1.0f);
    float r = truncf(t);
    if (fabsf(t - r) >= 0.5f) r += copysignf(1.0f, t);
    return (int)r + (1 << (q_bit - 1));
}

#endif  // HYC_QUANT_MATH_H
