// Scalar arithmetic of the integer-code rule, shared by the HIP kernels and by a
// host-side exhaustive checker (plain C99 / C++; no HIP types in here).
//
// The code rule of the reference quantiser (operators/compress_function_kernel.py:92-110)
// is   t = fp32(x) / fp32(s) (+ z);  r = roundf(t);  r = clamp(r, -2^(q-1), 2^(q-1)-1);
//      code = r + 2^(q-1).
// x and s are bf16.  An IEEE fp32 division costs ~10 VALU operations per element on
// CDNA, which would make the quantiser ALU-bound before it is HBM-bound.  Because the
// divisor is constant per column, the kernels keep r = 1/s per column and recover the
// correctly rounded quotient with one multiply and two fused multiply-adds
// (hyc_quot_fast).  That this equals the IEEE quotient bit for bit — for every bf16 x
// and every bf16 s accepted by hyc_scale_is_fast — is established exhaustively on the
// CPU by tests/native/check_fastdiv.c, which includes this very header.
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

// Quotients are pre-clamped to +-HYC_QCLAMP before the correction step so that
// infinities cannot turn into NaN there.  Any |t| >= 512 saturates every supported
// code width even after adding a zero point in [-128, 127].
#define HYC_QCLAMP 1024.0f

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
// huge, inf, NaN) takes the IEEE division.
HYC_HD int hyc_scale_is_fast(float s) { return (s >= 1e-18f) && (s <= 1e18f); }

// x/s from r = 1/s (itself the IEEE reciprocal), valid when hyc_scale_is_fast(s): one
// Newton-style correction of x*r with an exact remainder.  The integer code derived
// from the result equals the code derived from the IEEE quotient for every bf16 x
// (the quotient itself may differ in the sign of zero and for subnormal x, where the
// code is 2^(q-1) either way).  Beyond +-512 only the sign matters; NaN x gives NaN.
HYC_HD float hyc_quot_fast(float x, float s, float r) {
    float q0 = x * r;
    q0 = fminf(fmaxf(q0, -HYC_QCLAMP), HYC_QCLAMP);
    float rem = fmaf(-q0, s, x);
    return fmaf(rem, r, q0);
}

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

// Cheapest form of the rule for the reciprocal path, as a signed code in
// [-2^(q-1), 2^(q-1)-1] (the caller adds the offset 2^(q-1) once per packed word).
// Instead of clamping the quotient, the INPUT is clamped to [xlo, xhi] =
// [(-2^(q-1) - 0.49) s, (2^(q-1) - 1 + 0.49) s]: inside that interval nothing changes, and
// outside it the value lands 0.49 beyond the last code, which rounds to that code — the
// same saturation, but infinities never reach the correction step and no second clamp is
// needed.  A NaN input fails the comparison and becomes xlo, i.e. the lowest code (biased
// code 0); a compare-and-select is used rather than fmaxf because fmaxf turns a
// *signalling* NaN into a quiet NaN instead of dropping it.
// The sign for the half-away rounding is taken from the clamped input (s > 0 here).
// The lower bound is derived from the upper one (lo - 0.49 = -(hi + 0.49) - 1), so a kernel
// that is short of registers keeps only xhi and recomputes xlo = -xhi - s on the fly.
HYC_HD float hyc_clamp_hi(float s, int q_bit) { return ((float)(1 << (q_bit - 1)) - 1.0f + 0.49f) * s; }
HYC_HD float hyc_clamp_lo_from_hi(float xhi, float s) { return -xhi - s; }
HYC_HD float hyc_clamp_lo(float s, int q_bit) { return hyc_clamp_lo_from_hi(hyc_clamp_hi(s, q_bit), s); }

HYC_HD int hyc_signed_code_fast(float x, float s, float r, float xlo, float xhi) {
    float xc = (x > xlo) ? x : xlo;
    xc = fminf(xc, xhi);
    const float q0 = xc * r;
    const float rem = fmaf(-q0, s, xc);
    const float q1 = fmaf(rem, r, q0);
    return (int)(q1 + copysignf(0.5f, xc));
}

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
