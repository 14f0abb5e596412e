/* hyclora.h — C ABI of the MI355X (gfx950) kernels for HyC-LoRA's activation-compression
 * path.
 *
 * Conventions shared by every entry point
 *   - All tensor arguments are raw DEVICE pointers.  "bf16" means 16-bit brain floats,
 *     row-major, innermost (channel) dimension contiguous; pointers that are read or
 *     written 16 bytes at a time must be 16-byte aligned (checked).
 *   - The caller owns every buffer, outputs and workspaces included; nothing is
 *     allocated, freed or kept between calls, nothing synchronises with the host.
 *     Work is enqueued on `stream` (a hipStream_t passed as void*; NULL = default stream).
 *   - Return value: HYC_OK (0) or a negative HYC_ERR_* code.  On error nothing was
 *     launched.  Entry points are reentrant; any thread may call with its own stream.
 *   - Each declaration cites the function of the reference (thu-ee-acts-lab/HyC-LoRA,
 *     path:line inside its checkout) whose GPU work it replaces.
 */
#ifndef HYCLORA_H
#define HYCLORA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HYC_OK 0
#define HYC_ERR_NULL (-1)      /* a required pointer is NULL */
#define HYC_ERR_QBIT (-2)      /* q_bit not in {2, 4, 8} */
#define HYC_ERR_SHAPE (-3)     /* a dimension is negative, too large, or N % 32 != 0 */
#define HYC_ERR_ALIGN (-4)     /* pointer or stride not aligned for 128-bit access */
#define HYC_ERR_RANK (-5)      /* LoRA rank unsupported (must be a multiple of 4, 4..64) */
#define HYC_ERR_LAUNCH (-6)    /* the HIP runtime refused the launch */
#define HYC_ERR_WORKSPACE (-7) /* workspace too small */
#define HYC_ERR_ARG (-8)       /* other invalid argument */

/* Text for a HYC_ERR_* code (static storage). */
const char *hyc_error_string(int code);

/* ABI revision; bumped when a signature changes. */
int hyc_abi_version(void);

/* Launch-shape knobs for benchmarking (process-wide, not thread-safe against concurrent
 * launches).  Keys: "quant_rows_per_wave" (rows each wave walks in hyc_quant_pack /
 * hyc_unpack_dequant, default 16).  Unknown key or bad value: HYC_ERR_ARG.  No
 * counterpart in the reference (its launch shapes come from triton.autotune). */
int hyc_set_tuning(const char *key, int value);

/* ---------------------------------------------------------------------------------------
 * Per-channel quantise + sub-byte pack, optionally with a zero point and/or with outlier
 * channels split off.
 *
 * Replaces: compression_quantization_kernel (operators/compress_function_kernel.py:46-112),
 * compression_quantization_with_zero_point_kernel (:228-301) and the torch gather /
 * index-assign around them in outlier_subtraction_fuse_compression_quantization
 * (operators/compress_function.py:111-143).
 *
 *   x          bf16, logical shape [B, M, N].  Element (b, m, c) lives at
 *              x + b*stride_b + m*stride_m + (c / head_dim)*stride_h + (c % head_dim)
 *              (strides in elements).  A plain [B, M, N] tensor passes head_dim = N,
 *              stride_h = 0; a [B, H, S, D] tensor read as [B, S, H*D] passes head_dim = D,
 *              stride_h = x.stride(1), stride_m = x.stride(2).  head_dim % 8 == 0.
 *   scale      bf16 [N], the per-channel step.
 *   zero_point bf16 [N] or NULL.
 *   q          uint8 [B, M, N * q_bit / 8], contiguous: the packed codes.  With
 *              epp = 8 / q_bit and w = 32 / epp, byte p*w + j of a row holds the codes of
 *              columns 32p + j + i*w (i = 0..epp-1), code i at bit q_bit*i.
 *   outlier_idx int64 [k] channel numbers or NULL (k = 0).  Those columns are copied to
 *              x_outlier (bf16 [B, M, k], column order = order of outlier_idx) and are
 *              quantised as if they were zero.  If zero_input != 0 the columns are also
 *              zeroed in x itself, as the reference does.
 *   code rule  t = fp32(x)/fp32(scale) (+ zero_point); r = roundf(t) (ties away from zero);
 *              code = clamp(r, -2^(q-1), 2^(q-1)-1) + 2^(q-1); NaN -> 0.
 */
int hyc_quant_pack(const void *x, const void *scale, const void *zero_point, void *q,
                   const int64_t *outlier_idx, int64_t k, void *x_outlier, int zero_input,
                   int64_t B, int64_t M, int64_t N,
                   int64_t stride_b, int64_t stride_m, int64_t head_dim, int64_t stride_h,
                   int q_bit, void *stream);

/* ---------------------------------------------------------------------------------------
 * Unpack + dequantise, optionally with a zero point and/or with outlier channels put back.
 *
 * Replaces: decompression_dequantization_kernel (operators/compress_function_kernel.py:149-206),
 * decompression_dequantization_with_zero_point_kernel (:323-388) and the index-assign
 * in outlier_addition_fuse_decompression_dequantization (operators/compress_function.py:147-174).
 *
 *   x (output) bf16 [B, M, N] addressed like the input of hyc_quant_pack, so the result can
 *              be written straight into a [B, H, S, D] buffer.
 *   value      bf16( (bf16(code) - 2^(q-1) [- zero_point]) * scale ); outlier columns
 *              take x_outlier[b, m, position] instead.
 */
int hyc_unpack_dequant(const void *q, const void *scale, const void *zero_point, void *x,
                       const int64_t *outlier_idx, int64_t k, const void *x_outlier,
                       int64_t B, int64_t M, int64_t N,
                       int64_t stride_b, int64_t stride_m, int64_t head_dim, int64_t stride_h,
                       int q_bit, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HYCLORA_H */
