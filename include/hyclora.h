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
 *     launched.  Entry points are reentrant; any thread may call with its own stream
 *     (hyc_set_tuning, a benchmarking aid that writes process-wide launch-shape
 *     settings, is the one exception: call it while no other thread is launching).
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

/* ABI revision; bumped when a signature changes or an entry point is added. */
int hyc_abi_version(void);

/* Launch-shape knobs, FOR BENCHMARKING ONLY: process-wide state in a library whose entry points are otherwise
 * stateless.  Results never depend on them except where said ("stats_waves": the last bits of the sums of
 * squares).  Each knob is an atomic integer that an entry point reads once per launch, so a launch on another
 * thread runs with the old or the new value of each knob, never a torn one; a pair of calls that must agree
 * (hyc_channel_stats_strips, then hyc_channel_stats) must not straddle a change.  Keys: "quant_rows_per_wave" (rows each wave walks in hyc_quant_pack,
 * default 8), "dequant_rows_per_wave" (same for hyc_unpack_dequant, default 2),
 * "quant_outlier_rows_per_wave" / "dequant_outlier_rows_per_wave" (the same two when called with
 * an outlier list; default 8 each: a wave first has to find its outlier columns in the list),
 * "norm_compress_slab" (0 / 1: whether hyc_rmsnorm_fwd_compress and, for rows wider than 4096 channels,
 * hyc_rmsnorm_bwd without a weight gradient may use the column-slab kernels, default 1)
 * and "norm_compress_rows_per_group" (rows a workgroup of that kernel walks, even; 0 = chosen from the
 * row count, the default),
 * "fuse_rows_per_wave" (same for both fused LoRA-SiLU kernels, multiple of 16; default 0 = by code width
 * and size: backward 32; forward 96 for tensors of 2^24 elements and more, else 32; at 8 bits 32 in both
 * directions for tensors of 2^24 elements and more, else 16; "fuse_fwd_rows_per_wave" / "fuse_bwd_rows_per_wave" set one of them),
 * "contract_max_groups" (column groups hyc_lora_contract cuts a row strip into, default 32; changes the
 * workspace hyc_lora_contract_workspace asks for), "stats_waves" (waves hyc_channel_stats aims to launch,
 * default 4096; sets the number of row strips hyc_channel_stats_strips returns and so the order in which the
 * sums of squares are added).  Unknown key or bad value: HYC_ERR_ARG.  No
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

/* ---------------------------------------------------------------------------------------
 * Calibration statistics, step 1: per-channel minimum, maximum and sum of squares over the
 * M rows of ONE batch element (the reference calibrates on batch element 0 only), as one partial
 * result per strip of rows.
 *
 * Replaces the torch reductions in get_statistics_only_quant (operators/compress_function.py:50-54),
 * get_statistics_only_quant_zero_point (:67-72) and get_statistics_channel_base (:86,93-97),
 * together with the x.clone() the latter starts with (:81).
 *
 *   x      bf16 [M, N] of batch element 0, element (m, c) at
 *          x + m*stride_m + (c / head_dim)*stride_h + (c % head_dim)
 *   stats  fp32 [strips*3 + 1, N] device buffer, strips = hyc_channel_stats_strips(M, N) (it follows the
 *          launch size, hyc_set_tuning "stats_waves").  Output: rows 3s, 3s+1, 3s+2 = min, max (NaN
 *          propagates as in torch) and sum of squares over the rows of strip s.  The sums are fp32, added
 *          in a fixed order: a lane of the kernel adds every eighth row of its strip in ascending order,
 *          the eight waves of a workgroup are added in order (and hyc_channel_select adds the strips in
 *          order, 32 at a time) - the same bits on every run for given M, N and "stats_waves".  The last row is scratch
 *          for hyc_channel_select.
 *   stats_bytes  size of that buffer; HYC_ERR_WORKSPACE when smaller than (strips*3 + 1)*N*4.
 */
int64_t hyc_channel_stats_strips(int64_t M, int64_t N);
int hyc_channel_stats(const void *x, int64_t M, int64_t N, int64_t stride_m, int64_t head_dim,
                      int64_t stride_h, float *stats, int64_t stats_bytes, void *stream);

/* ---------------------------------------------------------------------------------------
 * Calibration statistics, step 2: outlier channels and per-channel step / zero point.
 *
 * Replaces torch.topk + the bf16 scalar arithmetic of get_statistics_channel_base
 * (operators/compress_function.py:86-105), get_statistics_only_quant (:50-59) and
 * get_statistics_only_quant_zero_point (:67-77).
 *
 *   stats       fp32 [strips*3 + 1, N] as hyc_channel_stats left it.  Modified: on return rows 0, 1, 2 hold
 *               the minimum, maximum and sum of squares over all rows, the last row the channels' sort keys.
 *   k           number of outlier channels (0 = none).  Chosen by bf16 norm
 *               bf16(sqrt(sum of squares)) descending, ties by channel index ascending —
 *               torch.topk leaves tie order unspecified, this rule is fixed.  N <= 32768
 *               when k > 0.
 *   outlier_idx int64 [k] output, in that order (NULL when k = 0).
 *   scale       bf16 [N] output: bf16( bf16(max - min) / (2^q_bit - 1) ), with min = max = 0
 *               for the chosen channels; if add_eps != 0 a zero step becomes bf16(0 + 1e-3)
 *               (compress_function.py:104).
 *   zero_point  int8 [N] output or NULL: -round_half_even(min / step) - 2^(q_bit-1), every
 *               operation rounded to bf16, then converted like a C cast (:72,77).
 */
int hyc_channel_select(float *stats, int64_t strips, int64_t N, int64_t k, int q_bit, int add_eps,
                       int64_t *outlier_idx, void *scale, int8_t *zero_point, void *stream);

/* ---------------------------------------------------------------------------------------
 * Attention-map compression: exact k-th value.
 *
 * Replaces torch.kthvalue(x.float().flatten(), k) in get_statistics_softmax
 * (operators/compress_function.py:30-32) without the fp32 copy and without sorting: a
 * bf16 tensor has at most 65536 distinct values.
 *
 *   hyc_hist16      a bf16 [n] (n < 2^32, 16-byte aligned) -> hist uint32 [65536], cleared
 *                   here first.  Bin = order-preserving key of the bit pattern (negative
 *                   values first, NaN last).
 *   hyc_hist_select kth is 1-based, 1 <= kth <= n (the caller checks the upper bound);
 *                   *threshold (fp32, device) receives the kth-smallest value.
 */
int hyc_hist16(const void *a, int64_t n, uint32_t *hist, void *stream);
int hyc_hist_select(const uint32_t *hist, int64_t kth, float *threshold, void *stream);

/* ---------------------------------------------------------------------------------------
 * Attention-map compression: ordered compaction and dense restore.
 *
 * Replaces mask-multiply + flatten().to_sparse() in compression_softmax
 * (operators/compress_function.py:309-313) and to_dense() in decompression_softmax
 * (:316-317; models/llama/fused_llama_layer_intra_inter_full_fuse.py:414-415).
 *
 * An element is kept when a > bf16(threshold) and a != 0 (torch compares in bf16 and
 * to_sparse drops zeros), and when it is NaN (the reference multiplies by the mask first, and
 * NaN * 0 is not zero); with compare_abs != 0 when |a| > bf16(threshold) and a != 0, which is the
 * unstructured-pruning form (compression_unstructed_pruning_coo / _bitmap, :320-335).  Output order
 * is ascending flat index, as to_sparse gives.
 * The flattened tensor is processed in segments of 4096 elements;
 * hyc_sparse_num_segments(n) = ceil(n / 4096).
 *
 *   hyc_sparse_count   a bf16 [n]; threshold fp32 scalar ON THE DEVICE;
 *                      seg_counts uint32 [nseg] scratch; seg_offsets int64 [nseg + 1] output:
 *                      entries kept before each segment, last element = total kept (nnz).
 *                      The caller reads nnz back to size the outputs, as to_sparse itself does.
 *   hyc_sparse_write   same a / threshold / seg_offsets; indices int64 [nnz], values bf16 [nnz].
 *   hyc_sparse_write_bounded    the same into buffers with room for `capacity` entries, sized by
 *                      the caller without knowing nnz (no read-back before the launch): entries at
 *                      output positions >= capacity are not written.  The list is complete exactly
 *                      when seg_offsets[nseg] <= capacity, which the caller checks when it suits it;
 *                      a truncated list must not be handed to hyc_sparse_restore / hyc_softmax_bwd_restore.
 *   hyc_sparse_segment_offsets  rebuilds seg_offsets from an ascending index list (for sparse
 *                      tensors that did not come from hyc_sparse_count).
 *   hyc_sparse_restore out bf16 [n] (16-byte aligned): zeros, with values[i] at indices[i].
 */
int64_t hyc_sparse_num_segments(int64_t n);
int hyc_sparse_count(const void *a, int64_t n, const float *threshold, int compare_abs, uint32_t *seg_counts,
                     int64_t *seg_offsets, void *stream);
int hyc_sparse_write(const void *a, int64_t n, const float *threshold, int compare_abs,
                     const int64_t *seg_offsets, int64_t *indices, void *values, void *stream);
int hyc_sparse_write_bounded(const void *a, int64_t n, const float *threshold, int compare_abs,
                             const int64_t *seg_offsets, int64_t capacity, int64_t *indices, void *values,
                             void *stream);
int hyc_sparse_segment_offsets(const int64_t *indices, int64_t nnz, int64_t n, int64_t *seg_offsets,
                               void *stream);
int hyc_sparse_restore(const int64_t *indices, const void *values, const int64_t *seg_offsets,
                       int64_t n, void *out, void *stream);

/* ---------------------------------------------------------------------------------------
 * Softmax backward on a dense map: out = bf16((g - sum_row bf16(y*g)) * y), row sums in fp32.
 *
 * Replaces softmax_backward_kernel (operators/softmax_kernels.py:7-38).
 *   y, grad_y, out   bf16 [rows, n], contiguous.
 */
int hyc_softmax_bwd(const void *y, const void *grad_y, void *out, int64_t rows, int64_t n, void *stream);

/* ---------------------------------------------------------------------------------------
 * Scaled, masked softmax forward over the last dimension, optionally with the kept-entry count
 * of the compaction that follows:
 *     t = bf16(bf16(s * scale) + mask)   (mask term only if mask != NULL);   out = bf16(softmax_fp32(t)).
 *
 * Replaces the three torch passes  s = q @ k^T / sqrt(head_dim);  s = s + attention_mask;
 * a = torch.softmax(s, dim=-1, dtype=v.dtype)
 * (models/llama/fused_llama_layer_intra_inter_full_fuse.py:159-167; the scalar division is a
 * multiplication by the fp32 reciprocal in torch's device kernel, hence `scale`).
 *   s, out    bf16 [rows, n] contiguous, 16-byte aligned (out may alias s); n % 8 == 0, n <= 8192.
 *   mask      bf16 or NULL; row r adds mask[(r / rows_per_batch) * mask_stride_b +
 *             (r % mask_rows) * mask_stride_row + 0..n-1]  (a [B,1,S,S] mask over [B,H,S,S] scores:
 *             mask_rows = S, rows_per_batch = H*S, strides S*S and S; a stride of 0 broadcasts: stride_b = 0 one
 *             mask for all batches, stride_row = 0 one mask row for all queries, as a padding mask).
 *   threshold, seg_counts, seg_offsets   all NULL, or all given: then seg_counts / seg_offsets are
 *             filled exactly as hyc_sparse_count(out, rows*n, threshold, ...) would fill them, without
 *             another pass over the map (seg_counts holds ceil(rows*n / 4096) counters).  Needs
 *             n <= 4096 (otherwise HYC_ERR_SHAPE: call hyc_sparse_count afterwards instead).  Rows of
 *             512, 1024, 2048 or 4096 elements with rows*n % 4096 == 0 tile the segments and give one
 *             count per wave; other row lengths add their counts with integer atomics into counters
 *             the call zeroes first (one more small launch; the result is the same).
 */
int hyc_softmax_fwd(const void *s, const void *mask, void *out, int64_t rows, int64_t n, float scale,
                    int64_t mask_rows, int64_t rows_per_batch, int64_t mask_stride_b, int64_t mask_stride_row,
                    const float *threshold, uint32_t *seg_counts, int64_t *seg_offsets, void *stream);

/* ---------------------------------------------------------------------------------------
 * Dense restore and softmax backward in one pass over the compressed map: saves reading the
 * restored map back (1 of the 4 dense passes of restore + backward).
 *
 * Replaces a_o.to_dense() followed by softmax_backward(a, grad_a)
 * (models/llama/fused_llama_layer_intra_inter_full_fuse.py:414-415,432; operators/softmax_kernels.py:7-38).
 *   indices / values / seg_offsets  as produced by hyc_sparse_count + hyc_sparse_write for a map of
 *                                   rows*n elements;
 *   grad_y, out   bf16 [rows, n];   a_out  bf16 [rows, n] or NULL (the restored map);
 *   out_scale     the bf16 gradient is multiplied by this and rounded again: 1.0f, or 1/sqrt(head_dim) to fold
 *                 in the layer's grad_s = grad_s / math.sqrt(head_dim) (…full_fuse.py:436; a multiplication by
 *                 the fp32 reciprocal in torch's device kernel);
 *   n a multiple of 8, 8 <= n <= 4096; other row lengths: HYC_ERR_SHAPE (use hyc_sparse_restore +
 *   hyc_softmax_bwd).  Rows of 512, 1024, 2048 or 4096 elements with rows*n % 4096 == 0 tile the
 *   map's segments (one segment per wave); for other shapes a wave takes the whole rows that fit
 *   into 4096 elements and filters the entries of the one or two segments they lie in.  Either way
 *   the results are the bits of hyc_sparse_restore followed by hyc_softmax_bwd.
 */
int hyc_softmax_bwd_restore(const int64_t *indices, const void *values, const int64_t *seg_offsets,
                            const void *grad_y, void *a_out, void *out, int64_t rows, int64_t n,
                            float out_scale, void *stream);

/* ---------------------------------------------------------------------------------------
 * RMSNorm forward: rstd = 1/sqrt(mean(x^2) + eps) in fp32, y = bf16(x * rstd * weight).
 *
 * Replaces _rms_norm_fwd_fused (operators/rmsnorm_kernels.py:10-54).
 *   x, y    bf16 [rows, N] contiguous; N % 8 == 0, N <= 65536.
 *   weight  [N], bf16 or fp32 (weight_is_fp32).   rstd  fp32 [rows] output.
 */
int hyc_rmsnorm_fwd(const void *x, const void *weight, int weight_is_fp32, void *y, float *rstd,
                    int64_t rows, int64_t N, float eps, void *stream);

/* ---------------------------------------------------------------------------------------
 * RMSNorm backward: dx = (w*dy - (x^*c1 + c2)) * rstd with x^ = x*rstd, c1 = mean(x^*w*dy),
 * c2 = mean(w*dy) — the reference keeps LayerNorm's c2 term and so does this; optionally
 * dw = sum_rows dy*x^.
 *
 * Replaces _rms_norm_bwd_dx_fused (operators/rmsnorm_kernels.py:58-113) and, when dw is
 * requested, _rms_norm_bwd_dwdb (operators/rmsnorm_updatable_kernels.py:117-137) — with a
 * deterministic two-stage fp32 reduction instead of the spin-lock accumulation.
 *   dy, x, dx  bf16 [rows, N] contiguous; N % 8 == 0, N <= 8192.
 *   dw         [N] in the weight's dtype, 16-byte aligned, or NULL.  When given, workspace
 *              (16-byte aligned) must hold hyc_rmsnorm_bwd_workspace(rows, N) bytes (fp32
 *              partial rows).
 */
int64_t hyc_rmsnorm_bwd_workspace(int64_t rows, int64_t N);
int hyc_rmsnorm_bwd(const void *dy, const void *x, const void *weight, int weight_is_fp32,
                    const float *rstd, void *dx, void *dw, void *workspace, int64_t workspace_bytes,
                    int64_t rows, int64_t N, void *stream);

/* hyc_rmsnorm_bwd with the weight gradient for callers that cannot allocate device memory or
 * carry a workspace: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  No counterpart in the reference.  Same kernels, same results bit for bit; the fp32
 * partial rows live in a file-scope device array of the library instead of a caller workspace
 * (hyc_rmsnorm_bwd_static_max_bytes() = 16 MiB per GPU, resident from the time the library is
 * loaded on a device until the process ends).  Allocates nothing and frees nothing.
 *   dw must be given (without it hyc_rmsnorm_bwd needs no workspace either).
 *   N > 8192, or a shape whose partial rows would exceed the array: HYC_ERR_WORKSPACE, nothing launched.
 *   Every call on one GPU uses that GPU's one array: calls that overlap in time on the same GPU
 *   (different streams or threads) race on it; calls on one stream are ordered and safe.  Nothing
 *   in the array needs clearing between calls: each launch overwrites all it later reads.
 */
int64_t hyc_rmsnorm_bwd_static_max_bytes(void);
int hyc_rmsnorm_bwd_static(const void *dy, const void *x, const void *weight, int weight_is_fp32,
                           const float *rstd, void *dx, void *dw, int64_t rows, int64_t N, void *stream);

/* The same with the gradient that arrives over the residual connection added in the same pass:
 * dx = bf16(bf16(dx of hyc_rmsnorm_bwd) + residual), i.e. the bits of that call followed by a bf16
 * add.  Replaces `grad_norm_2 + grad_output` / `grad_norm_1 + grad_medium` after the norm backward
 * in the layers (models/llama/fused_llama_layer_intra_inter_full_fuse.py:391-393, :491-493).
 *   residual   bf16 [rows, N] contiguous, 16-byte aligned; must not overlap dx.
 */
int hyc_rmsnorm_bwd_add(const void *dy, const void *x, const void *weight, int weight_is_fp32,
                        const float *rstd, const void *residual, void *dx, void *dw, void *workspace,
                        int64_t workspace_bytes, int64_t rows, int64_t N, void *stream);

/* RMSNorm backward that reads its input from the channel-base compressed copy (what
 * hyc_rmsnorm_fwd_compress or hyc_quant_pack with an outlier list left: codes, steps, outlier
 * values) instead of a dense tensor; dx is the same bits as hyc_unpack_dequant followed by
 * hyc_rmsnorm_bwd (or _add, with a residual).  Replaces
 * outlier_addition_fuse_decompression_dequantization + rmsnorm_backward (+ the add) in the layers'
 * backward (models/llama/fused_llama_layer_intra_inter_full_fuse.py:386-393, :486-493).
 *   q_x, scale_x, outlier_table, k, x_outlier   as in hyc_rmsnorm_fwd_compress (k may be 0).
 *   residual   bf16 [rows, N] or NULL.   No dw.
 * Only for rows that are a whole number of 512-column slabs (N % 512 == 0, N <= 8192) and an even
 * number of rows: HYC_ERR_SHAPE otherwise (callers then dequantise and use hyc_rmsnorm_bwd).
 */
int hyc_rmsnorm_bwd_codes(const void *dy, const void *q_x, const void *scale_x, const uint16_t *outlier_table,
                          int64_t k, const void *x_outlier, int q_bit, const void *weight, int weight_is_fp32,
                          const float *rstd, const void *residual, void *dx, int64_t rows, int64_t N,
                          void *stream);

/* ---------------------------------------------------------------------------------------
 * NF4 block-wise weight dequantisation to bf16, bitsandbytes 0.43.2 layout (the version the
 * reference pins in requirements.txt:3).
 *
 * Replaces BF.dequantize_nf4(w, quant_state) (models/utils/compute_utils.py:19, :29):
 *   out[i] = bf16(table[code_i] * absmax[i / blocksize]),  code of an even i in the high nibble of
 *   packed[i / 2];  nested != 0 ("double quant"): absmax is uint8 [n / blocksize] and the block's
 *   statistic is code2[absmax[b]] * absmax2[b / blocksize2] + *offset (fp32; offset is a device
 *   scalar, NULL = 0);  nested == 0: absmax is fp32.
 *   table  fp32 [16] (the NF4 code book; the quant state carries it), code2 fp32 [256];
 *   n even, blocksize % 8 == 0; packed 4-byte aligned, out 16-byte aligned.
 */
int hyc_nf4_dequant(const void *packed, const void *absmax, int nested, const float *code2, const float *absmax2,
                    const float *offset, int64_t blocksize2, const float *table, void *out, int64_t n, int64_t blocksize,
                    void *stream);

/* ---------------------------------------------------------------------------------------
 * LayerNorm over the last dimension (the encoder layers' norm).
 *
 * hyc_layernorm_fwd replaces _layer_norm_fwd_fused / layernorm_forward
 * (operators/layernorm_kernels.py:9-56, :125-147): mean and rstd = 1/sqrt(var + eps) in fp32 (variance
 * from the centred values), y = (x - mean)*rstd*w + b rounded once to bf16.
 * hyc_layernorm_bwd replaces _layer_norm_bwd_dx_fused / layernorm_backward (:60-121, :150-198):
 * dx = (w*dy - (x^*c1 + c2))*rstd with c1 = mean(x^ * w*dy), c2 = mean(w*dy).  The reference computes
 * dw / db partials under a spin lock and discards them (returns (dx, None, None)); so there are none here.
 *   x, y, dy, dx  bf16 [rows, N] contiguous, 16-byte aligned; N % 8 == 0, N <= 8192.
 *   weight, bias  [N], both bf16 (params_are_fp32 == 0) or both fp32;  mean, rstd  fp32 [rows].
 */
int hyc_layernorm_fwd(const void *x, const void *weight, const void *bias, int params_are_fp32, void *y,
                      float *mean, float *rstd, int64_t rows, int64_t N, float eps, void *stream);
int hyc_layernorm_bwd(const void *dy, const void *x, const void *weight, int params_are_fp32,
                      const float *mean, const float *rstd, void *dx, int64_t rows, int64_t N, void *stream);

/* ---------------------------------------------------------------------------------------
 * RMSNorm forward fused with the compressions a decoder layer applies around it: the row is read
 * once and yields the normalised output, its quantised copy and the channel-base compressed copy
 * of the input.
 *
 * Replaces the sequence rmsnorm_forward(x, w, eps); compression_pack_channel_base(x, ...);
 * compression_pack_quant_base(x_norm, ...) with frozen statistics
 * (models/llama/fused_llama_layer_intra_inter_full_fuse.py:97-126; kernels
 * operators/rmsnorm_kernels.py:10-54 and operators/compress_function_kernel.py:46-112).  Results are
 * bit-identical to hyc_rmsnorm_fwd followed by hyc_quant_pack on y and on x.
 *   x, y        bf16 [rows, N] contiguous; N % 32 == 0, N <= 8192;  rstd fp32 [rows].
 *   scale_y,q_y steps bf16 [N] and packed codes uint8 [rows, N*q_bit/8] of y; q_y NULL: skipped.
 *   scale_x,q_x the same for x with the outlier channels zeroed; q_x NULL: skipped.
 *   outlier_table uint16 [N] from hyc_outlier_table (1 + list position of an outlier channel, else 0),
 *   k           number of outlier channels, x_outlier bf16 [rows, k] (column order = list order).
 *
 * hyc_outlier_table builds that table from a channel list (int64 [k], k <= 65535).
 */
int hyc_outlier_table(const int64_t *outlier_idx, int64_t k, int64_t N, uint16_t *table, void *stream);
int hyc_rmsnorm_fwd_compress(const void *x, const void *weight, int weight_is_fp32, void *y, float *rstd,
                             int64_t rows, int64_t N, float eps, int q_bit, const void *scale_y, void *q_y,
                             const void *scale_x, void *q_x, const uint16_t *outlier_table, int64_t k,
                             void *x_outlier, void *stream);

/* hyc_rmsnorm_fwd_compress that also forms, from the normalised output while it is still on the chip,
 * the LoRA-A down projections of up to four adapters that take this output as their input:
 * adapter_out[g] = bf16( y @ adapter_weight[g]^T ), fp32 accumulation over the whole row, one rounding.
 * Replaces `x_norm @ lora_A^T` of lora_forward for q, k and v (gate and up), each of which reads the
 * [rows, N] output again (models/utils/compute_utils.py:22 as called from
 * models/llama/fused_llama_layer_intra_inter_full_fuse.py:111-117, :218-226).
 *   n_adapters 1..4; adapter_weight / adapter_rank / adapter_out are HOST arrays of that length:
 *   adapter_weight[g]  bf16 [rank, N] row-major on the device (lora_A.weight as nn.Linear keeps it), 16-byte aligned;
 *   adapter_rank[g]    1..64; the ranks, each rounded up to a multiple of 16, may add up to 64 at most
 *                      (HYC_ERR_RANK otherwise);
 *   adapter_out[g]     bf16 [rows, rank] contiguous on the device.
 *   The norm weight is bf16.  q_y, q_x may be NULL (no compressed copy), as in hyc_rmsnorm_fwd_compress;
 *   y, rstd and the codes are the same bits as from that call.
 * Only for rows that are a whole number of 512-column slabs (N % 512 == 0, N <= 8192) and an even
 * number of rows: HYC_ERR_SHAPE otherwise (callers then use a library GEMM on y).
 */
int hyc_rmsnorm_fwd_compress_lora(const void *x, const void *weight, void *y, float *rstd, int64_t rows, int64_t N,
                                  float eps, int q_bit, const void *scale_y, void *q_y, const void *scale_x,
                                  void *q_x, const uint16_t *outlier_table, int64_t k, void *x_outlier,
                                  int n_adapters, const void *const *adapter_weight, const int64_t *adapter_rank,
                                  void *const *adapter_out, void *stream);

/* ---------------------------------------------------------------------------------------
 * Rotary position embedding, in place: for every (b, s, h) the head x[b,s,h,:] = (x1 | x2) becomes
 * (x1*cos[s] - x2*sin[s] | x2*cos[s] + x1*sin[s]); backward != 0 uses -sin.
 *
 * Replaces _rope_embedding / rope_forward / rope_backward (operators/rope_kernels.py:36-78, :81-126).
 *   x        bf16, element (b,s,h,d) at x + b*stride_b + s*stride_s + h*stride_h + d; head_dim % 16 == 0;
 *            strides multiples of 8 elements (a [B,S,H,D] tensor: S*H*D, H*D, D; a [B,H,S,D] tensor
 *            is rotated in place with H*S*D, D, S*D).
 *   cos, sin angle tables, row s at + s*stride_{cos,sin} elements; only the first head_dim/2 entries of a
 *            row are read.  bf16 tables (table_is_fp32 == 0): bf16 rounding after every multiply and
 *            add, as bf16 Triton arithmetic; fp32 tables: fp32 arithmetic, one rounding on the store.
 */
int hyc_rope(void *x, const void *cos, const void *sin, int table_is_fp32, int64_t B, int64_t S, int64_t H,
             int64_t head_dim, int64_t stride_b, int64_t stride_s, int64_t stride_h, int64_t stride_cos,
             int64_t stride_sin, int backward, void *stream);

/* ---------------------------------------------------------------------------------------
 * Element-wise operators on n contiguous bf16 elements (16-byte aligned pointers).
 *
 *   hyc_silu_bwd  out = g * (sig * (1 + x*(1 - sig))), sig = bf16(sigmoid(x)), bf16 after
 *                 every operation.  Replaces silu_backward_kernel (operators/silu_kernels.py:12-45).
 *   hyc_silu_mul  out = (sig(x1) * x1) * x2.  Replaces triton_silu_hadamard_kernel (:73-106).
 *   hyc_silu_once_mul  out = bf16(silu(x1)) * x2, silu evaluated in fp32 and rounded once.  Replaces
 *                 `fn = torch.nn.functional.silu(gate); hadamard = up * fn`, the form in which the backward
 *                 of the layers without the fused LoRA kernels recomputes the gated product
 *                 (models/llama/fused_llama_layer_intra_inter.py:362,370).
 *   hyc_gelu_bwd  out = d/dx[tanh-GELU](x) * g, evaluated in fp32.  Replaces
 *                 gelu_backward_kernel (operators/gelu_kernels.py:19-58).
 */
int hyc_silu_bwd(const void *x, const void *g, void *out, int64_t n, void *stream);
int hyc_silu_mul(const void *x1, const void *x2, void *out, int64_t n, void *stream);
int hyc_silu_once_mul(const void *x1, const void *x2, void *out, int64_t n, void *stream);
/* Backward of o = silu(x) * u in one pass: grad_x = hyc_silu_bwd(x, bf16(g * u)), grad_u = g * silu(x) with
 * silu(x) as hyc_silu_once_mul forms it (F.silu).  Replaces F.silu + two products + silu_backward in the layers
 * that do not use the fused LoRA kernels (models/llama/fused_llama_layer_intra_inter.py:362-381). */
int hyc_silu_mul_bwd(const void *x, const void *u, const void *g, void *grad_x, void *grad_u, int64_t n,
                     void *stream);
int hyc_gelu_bwd(const void *x, const void *g, void *out, int64_t n, void *stream);

/* ---------------------------------------------------------------------------------------
 * Fused LoRA-SiLU-Hadamard forward: quantises the two frozen-weight outputs for backward
 * while producing the gated product.
 *     q1 = pack(code(x1; s1)),  q2 = pack(code(x2; s2))           (same rule as hyc_quant_pack)
 *     y1 = x1 + bf16(xa1 . b1); y2 = x2 + bf16(xa2 . b2)          (MFMA, fp32 accumulation)
 *     o  = (y1 * bf16(sigmoid(y1))) * y2                          (bf16 after every operation)
 *
 * Replaces triton_fuse_silu_forward_kernel
 * (operators/triton_fuse_lora_silu_hadamard_forward_kernels.py:28-149).
 *   xa1, xa2 bf16 [T, R] contiguous (x @ lora_A);   b1, b2 bf16 [R, N] contiguous (lora_B), or with
 *   b_transposed = 1 both [N, R] contiguous, the layout torch.nn.Linear keeps lora_B.weight in (the
 *   reference copies them to [R, N] first, …forward_kernels.py:166-167);
 *   x1, x2   bf16 [T, N] contiguous;                s1, s2 bf16 [N];
 *   q1, q2   uint8 [T, N*q_bit/8];                  o      bf16 [T, N].
 *   R: multiple of 4, 4..64 (the reference needs a power of two >= 16); N % 32 == 0; any T.
 */
int hyc_lora_silu_mul_fwd(const void *xa1, const void *b1, const void *x1, const void *s1,
                          const void *xa2, const void *b2, const void *x2, const void *s2,
                          void *q1, void *q2, void *o, int64_t T, int64_t N, int64_t R, int q_bit,
                          int b_transposed, void *stream);

/* ---------------------------------------------------------------------------------------
 * Fused LoRA-SiLU-Hadamard backward: dequantises q1, q2, recomputes y1, y2 and the gated
 * product o, and produces
 *     grad_gate = (g * y2) * (sig * (1 + y1*(1 - sig))),   grad_up = g * (y1 * sig).
 *
 * Replaces triton_fuse_silu_backward_kernel
 * (operators/triton_fuse_lora_silu_hadamard_backward_kernels.py:28-149).
 *   grad_o, o, grad_gate, grad_up  bf16 [T, N] contiguous; the rest as in the forward.
 */
int hyc_lora_silu_mul_bwd(const void *xa1, const void *b1, const void *q1, const void *s1,
                          const void *xa2, const void *b2, const void *q2, const void *s2,
                          const void *grad_o, void *o, void *grad_gate, void *grad_up,
                          int64_t T, int64_t N, int64_t R, int q_bit, int b_transposed, void *stream);

/* ---------------------------------------------------------------------------------------
 * LoRA add around the compressed copy of a projection's frozen part:
 *     hyc_lora_add          y = bf16(x + bf16(xa . b)), and with a residual (bf16 [T, N], or NULL)
 *                           y = bf16(residual + bf16(x + bf16(xa . b)))    (y may be x or residual: in place)
 *     hyc_lora_add_quant    the same y, and q = pack(code(x; scale [, zero_point])) from the one
 *                           read of x (code rule and layout of hyc_quant_pack)
 *     hyc_lora_add_restore  x = value of hyc_unpack_dequant(q; scale [, zero_point]), then the
 *                           same y; the dense x is never written
 * bit-identical to the separate steps.
 *
 * Replaces the product, the add and the quantiser / dequantiser call between them:
 * lora_forward (models/utils/compute_utils.py:21-24) with compression_pack_quant_base on the
 * frozen part (models/llama/fused_llama_layer_intra_inter_full_fuse.py:128-140; zero-point form
 * models/llama_flash_attn/fused_llama_layer_intra_inter.py:129-138); the rebuild of q, k, v, gate,
 * up in backward (…full_fuse.py:416-417, :439-441, :447-449); and `grad_x += grad_medium @ A^T`
 * of lora_backward (compute_utils.py:34-35) through the plain form; the residual covers the add that
 * follows a projection (`x + o_final`, `x_medium + down`, …full_fuse.py:198,250) and the running sum of
 * input gradients (`grad_x += grad_x_temp`, :477,481).
 *   xa bf16 [T, R] contiguous;  x, y bf16 [T, N] contiguous;
 *   b bf16 [R, N] contiguous (b_transposed 0) or [N, R] contiguous (b_transposed 1: the layout
 *   torch.nn.Linear keeps lora_B.weight in, so no copy of the adapter is needed);
 *   scale, zero_point bf16 [N] (zero_point NULL: symmetric codes);  q uint8 [T, N*q_bit/8].
 *   R: multiple of 4, 4..64; N % 32 == 0; any T.
 * Tuning keys "add_rows_per_wave", "add_quant_rows_per_wave", "add_restore_rows_per_wave" (multiples of
 * 16; defaults 0 = 32, 48 or 64 chosen per shape so that the waves fill their generations, 48, 48).
 */
int hyc_lora_add(const void *xa, const void *b, int b_transposed, const void *x, const void *residual,
                 void *y, int64_t T, int64_t N, int64_t R, void *stream);
int hyc_lora_add_quant(const void *xa, const void *b, int b_transposed, const void *x, const void *scale,
                       const void *zero_point, void *q, void *y, int64_t T, int64_t N, int64_t R,
                       int q_bit, void *stream);
int hyc_lora_add_restore(const void *xa, const void *b, int b_transposed, const void *q,
                         const void *scale, const void *zero_point, void *y, int64_t T, int64_t N,
                         int64_t R, int q_bit, void *stream);

/* hyc_lora_add_quant / hyc_lora_add_restore with the rotary position embedding applied to the sum
 * before it is stored: y = rope(bf16(x + bf16(xa . b))), the codes still those of x.  Same value as
 * the plain entry point followed by hyc_rope on y viewed as [T / seq_len, seq_len, N / 128, 128]
 * (row t takes table row t % seq_len), bit for bit.  Heads of 128 dims only (a column tile is one head):
 * N % 128 == 0.  cos, sin, table_is_fp32, stride_cos, stride_sin as in hyc_rope.
 * Replaces rope_forward on q and k after the projection and after their rebuild in backward
 * (models/llama/fused_llama_layer_intra_inter_full_fuse.py:151-152, :444, :452). */
int hyc_lora_add_quant_rope(const void *xa, const void *b, int b_transposed, const void *x, const void *scale,
                            const void *zero_point, void *q, void *y, const void *cos, const void *sin,
                            int table_is_fp32, int64_t seq_len, int64_t stride_cos, int64_t stride_sin,
                            int64_t T, int64_t N, int64_t R, int q_bit, void *stream);
int hyc_lora_add_restore_rope(const void *xa, const void *b, int b_transposed, const void *q,
                              const void *scale, const void *zero_point, void *y, const void *cos,
                              const void *sin, int table_is_fp32, int64_t seq_len, int64_t stride_cos,
                              int64_t stride_sin, int64_t T, int64_t N, int64_t R, int q_bit, void *stream);

/* Up to four operand sets of hyc_lora_add_quant[_rope] / hyc_lora_add_restore[_rope] in ONE launch: the q, k
 * and v projections of a layer share their rows, rank and code width, and each alone ([4096, 4096] or, with
 * grouped-query heads, [4096, 1024]) is one short generation of waves whose launch is mostly ramp and drain.
 * Each member's outputs are the same bits as its own call.  All members with a zero point or all without
 * (HYC_ERR_ARG otherwise); cos / sin NULL: no rotation for that member.
 * Replaces the three lora_forward + quantiser sequences of the q, k, v projections and their three
 * dequantise + add (+ rope) sequences in backward
 * (models/llama/fused_llama_layer_intra_inter_full_fuse.py:105-152, :416-452). */
typedef struct hyc_lora_add_member {
    const void *xa;             /* bf16 [T, R] */
    const void *b;              /* bf16 [R, N] or, with b_transposed, [N, R] */
    const void *x;              /* quantise: the frozen part, bf16 [T, N]; restore: unused */
    const void *scale;          /* bf16 [N] */
    const void *zero_point;     /* bf16 [N] or NULL */
    void *q;                    /* uint8 [T, N*q_bit/8]: output of quantise, input of restore */
    void *y;                    /* bf16 [T, N] */
    const void *cos_t;          /* rotation tables as in hyc_rope, or NULL */
    const void *sin_t;
    int64_t seq_len, stride_cos, stride_sin;
    int64_t N;
    int b_transposed;
    int table_is_fp32;
} hyc_lora_add_member;
int hyc_lora_add_quant_group(const hyc_lora_add_member *members, int count, int64_t T, int64_t R, int q_bit,
                             void *stream);
int hyc_lora_add_restore_group(const hyc_lora_add_member *members, int count, int64_t T, int64_t R, int q_bit,
                               void *stream);

/* ---------------------------------------------------------------------------------------
 * The skinny LoRA products that stream a whole [T, N] tensor X for a rank-R result, from one read
 * of X and with fp32 accumulation over the whole contraction:
 *     p1 = bf16( U^T . X )   [R, N]      U bf16 [T, R]
 *     p2 = bf16( X . V^T )   [T, R]      V bf16 [R, N] (v_transposed 0) or [N, R] (v_transposed 1)
 * X is dense bf16 [T, N] (x), or - p1 only - the packed codes of hyc_quant_pack (q, scale,
 * optional zero_point, q_bit; x NULL), dequantised in registers to the value hyc_unpack_dequant
 * gives.  Pass p1 or p2 as NULL to skip that product.  With p1_transposed, p1 is written as [N, R] - the
 * memory layout of a lora_B weight, whose gradient xa^T @ grad_y is (the same values, transposed).
 *
 * Replaces the rank-R GEMMs of lora_forward / lora_backward (models/utils/compute_utils.py:22,
 * :30-33): x @ A (p2, V = lora_A.weight), grad_y @ B^T with xa^T @ grad_y (p2 and p1 of X = grad_y),
 * x^T @ grad_medium (p1), the last one without the decompression_dequantization call in front of it
 * (models/llama/fused_llama_layer_intra_inter_full_fuse.py:375-383, :469-481).  The reference
 * rounds per batch element and sums the batch in bf16; here the sum over all T rows is one fp32
 * accumulation rounded once.
 *   R even, 2..64; N % 32 == 0; any T.
 *   workspace: device scratch of hyc_lora_contract_workspace(T, N, R, p1 != NULL, p2 != NULL) bytes,
 *   16-byte aligned, contents undefined on entry and exit; partial sums are combined in a fixed
 *   order (no atomics), so results are reproducible.  Tuning key "contract_max_groups" (default 32):
 *   upper bound on the column groups a row strip is split into (each adds a plane of p2 partials).
 */
int64_t hyc_lora_contract_workspace(int64_t T, int64_t N, int64_t R, int want_p1, int want_p2);
int hyc_lora_contract(const void *x, const void *q, const void *scale, const void *zero_point, int q_bit,
                      const void *u, const void *v, int v_transposed, void *p1, int p1_transposed, void *p2,
                      void *workspace, int64_t workspace_bytes, int64_t T, int64_t N, int64_t R,
                      void *stream);

/* ---------------------------------------------------------------------------------------
 * Sum of two or three LoRA adds in one pass:  y = t_0 (+) t_1 [(+) t_2],  t_i = bf16(x_i + bf16(xa_i . b_i)),
 * every (+) a bf16 addition in that order - the bits of hyc_lora_add(x_0), then hyc_lora_add(x_1, residual = y),
 * then hyc_lora_add(x_2, residual = y).
 *
 * Replaces the accumulation of the input gradients of projections that share an input in the layers'
 * backward - `grad_x = ...; grad_x += grad_x_temp` after each lora_backward of q, k, v and of gate, up
 * (models/llama/fused_llama_layer_intra_inter_full_fuse.py:403-462 with models/utils/compute_utils.py:28-36) -
 * without writing and re-reading the running sum.
 *
 *   members  count (2 or 3) operand sets in host memory (copied at the call): xa bf16 [T, R], b the LoRA
 *            operand [R, N] (or [N, R] with b_transposed), x bf16 [T, N] (for the backward: grad_y @ W);
 *   y        bf16 [T, N]; may be one of the x_i.
 *   R a multiple of 4 up to 16 (HYC_ERR_RANK beyond: call hyc_lora_add in a chain); N % 32 == 0.
 */
typedef struct {
    const void *xa;
    const void *b;
    int b_transposed;
    const void *x;
} hyc_lora_sum_member;
int hyc_lora_add_sum(const hyc_lora_sum_member *members, int count, void *y, int64_t T, int64_t N, int64_t R,
                     void *stream);

/* ---------------------------------------------------------------------------------------
 * Memory-only probe, FOR BENCHMARKING: loads n_reads and stores n_writes bf16 [T, N] tensors (1..3 each,
 * arrays of device pointers in host memory, 16-byte aligned, N % 8 == 0) with the access shape of the
 * kernels of this library and no arithmetic of the path, so that the rate the memory system gives a
 * read / write mix can be put beside the kernel that has that mix (bench.py does, for the fused LoRA-SiLU
 * kernels).  What is stored is the xor of what was loaded.  No counterpart in the reference.
 *   shape 0: a wave owns 128 columns and four rows per instruction and walks rows_per_wave rows (multiple
 *            of 16) in 16-row tiles, as the fused LoRA-SiLU / LoRA-add kernels do;
 *   shape 1: a wave owns 512 columns (1 KiB) of one row per instruction, rows_per_wave a multiple of 4,
 *            as the quantiser does.
 */
int hyc_stream_probe(const void *const *reads, int n_reads, void *const *writes, int n_writes, int64_t T,
                     int64_t N, int shape, int rows_per_wave, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HYCLORA_H */
