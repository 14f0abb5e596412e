"""CPU oracle for the HyC-LoRA activation-compression path.  TEST INFRASTRUCTURE ONLY.

This module restates, with plain torch-CPU / numpy operations, what the reference's
operators compute.  It is the checker that the HIP kernels are compared against and
the thing timed as the CPU baseline; nothing in the shipped package may import it.
Only tests, the smoke check and the benchmark's cpu_baseline leg use it.

Every function cites the reference file:line it follows (paths relative to the
reference checkout).

Pinning status (what independent evidence holds each function in place):
  * quant_codes / pack_codes / unpack_codes / dequant: pinned by the scalar C
    restatement in oracle/scalar_ref.c (an independent loop-level implementation),
    by hand-computed known answers, by round trips, by |x - x^| <= s/2, and by the
    q=8 identity layout (tests/test_oracle_quant.py), and by the committed known-answer vectors
    of tests/golden/kat.json (scalar numpy arithmetic, tests/test_golden.py).
  * scale_* / outlier_channels: reduce to torch.max/min/norm plus two bf16 scalar
    operations; pinned by closed forms and planted outlier channels.
  * softmax_threshold / softmax_compress / softmax_restore: pinned against
    torch.sort / torch.nonzero on small inputs.
  * softmax_fwd: pinned to tolerance against a float64 softmax of the same rounded logits,
    by unit row sums, exact zeros under a -inf mask and shift invariance.
  * softmax_bwd, rmsnorm_fwd, silu_*, gelu_bwd, fused_*: pinned to tolerance against
    torch.autograd of the fp32 composite.  rmsnorm_bwd follows the reference's
    formula, which keeps LayerNorm's mean term c2 = mean(w * dy).  That term is pinned on rows
    whose mean is exactly zero (built as v | -v): there the formula IS the backward of
    F.layer_norm, so the oracle must equal float64 autograd of layer_norm and must differ
    from autograd of a true RMSNorm by exactly c2 * rstd - a dropped or sign-flipped term
    fails both (tests/test_oracle_norm.py; the same check on the GPU kernel in
    tests/test_gpu_elementwise_norm.py).
  * layernorm_fwd / layernorm_bwd: pinned against torch.nn.functional.layer_norm and its
    autograd in float64 (an independent library routine), tests/test_oracle_layernorm.py.
  * nf4_dequant: bitsandbytes (0.43.2, pinned in the reference's requirements.txt) is not installed,
    so its published format is restated; pinned by the published NF4 code book, hand-computed
    bytes (nibble order, nested statistics) and exact round trips of on-grid weights
    (tests/test_oracle_nf4.py).  "parity unpinned" against bitsandbytes' own output.
  * rope: pinned against the textbook rotate-half form x*cos + rotate_half(x)*sin with
    full-width tables, against an explicit complex-number rotation in float64, and by
    norm preservation / forward-then-backward identity (tests/test_oracle_rope.py).
  * lora_add / lora_products: a library matmul of the operands (float32 rounded to bf16 before
    the add, as lora_forward does; float64 for the products) - they reduce to library routines,
    and the CPU tests check them against explicit loops on small inputs (tests/test_oracle_lora.py).
The reference ships no tests, golden vectors or CPU implementation of its Triton
kernels, so there is nothing of its own to check against.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

BF16 = torch.bfloat16       # what the arithmetic rounds to after each operation.  Tests may bind this name to
                            # float64 to run the same code without intermediate rounding.
WIRE = torch.bfloat16       # dtype of a dequantised activation: part of the format (the product code * step is
                            # rounded to bf16 once, compress_function_kernel.py:200-204), not of the arithmetic
F32 = torch.float32


# --------------------------------------------------------------------------------------
# shape helpers (operators/compress_function.py:6-13)
# --------------------------------------------------------------------------------------
def hidden_to_head_shape(x: torch.Tensor, num_heads: int) -> torch.Tensor:
    b, s, h = x.shape
    return x.reshape(b, s, num_heads, h // num_heads).transpose(1, 2)


def head_to_hidden_shape(x: torch.Tensor) -> torch.Tensor:
    b, _, s, _ = x.shape
    return x.transpose(1, 2).reshape(b, s, -1)


def _as_bmn(x: torch.Tensor) -> torch.Tensor:
    """4-D [B,H,S,D] activations are viewed as [B,S,H*D] (compress_function.py:46-48,82-84)."""
    if x.dim() == 4:
        return head_to_hidden_shape(x)
    return x


# --------------------------------------------------------------------------------------
# statistics
# --------------------------------------------------------------------------------------
def scale_only_quant(x: torch.Tensor, q_bit: int) -> torch.Tensor:
    """Per-channel step from batch element 0 (compress_function.py:45-59).

    s[c] = bf16( bf16(max_m x[0,m,c] - min_m x[0,m,c]) / (2^q - 1) ), shape [1, N].
    """
    x = _as_bmn(x).to(BF16)
    x0 = x[0]
    hi = x0.max(dim=-2, keepdim=True).values
    lo = x0.min(dim=-2, keepdim=True).values
    return ((hi - lo) / (2 ** q_bit - 1)).to(BF16)


def scale_zero_point(x: torch.Tensor, q_bit: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-channel step and zero point (compress_function.py:62-77).

    z = -round_half_even(min / s) - 2^(q-1), all in bf16, then cast to int8.
    """
    x = _as_bmn(x).to(BF16)
    x0 = x[0]
    hi = x0.max(dim=-2, keepdim=True).values
    lo = x0.min(dim=-2, keepdim=True).values
    s = (hi - lo) / (2 ** q_bit - 1)
    z = -torch.round(lo / s) - (2 ** (q_bit - 1))
    return s.to(BF16), z.to(torch.int8)


def channel_norms(x: torch.Tensor) -> torch.Tensor:
    """bf16 L2 norm of every channel of batch element 0 (compress_function.py:86)."""
    x = _as_bmn(x).to(BF16)
    return x[0].abs().norm(dim=-2)


def outlier_channels(x: torch.Tensor, ratio: float) -> torch.Tensor:
    """k = int(N*ratio) channels with the largest bf16 norm (compress_function.py:86-87).

    torch.topk leaves the order of equal norms unspecified; the deterministic rule used
    here (and by the HIP path) is: norm descending, then channel index ascending.
    """
    nrm = channel_norms(x)
    k = int(nrm.shape[-1] * ratio)
    order = torch.sort(nrm.float(), descending=True, stable=True).indices
    return order[:k].to(torch.int64)


def channel_stats(x: torch.Tensor, ratio: float, q_bit: int,
                  idx: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Outlier channel list and the per-channel step of the remainder
    (compress_function.py:80-105).  The outlier columns are zeroed before min/max, so
    their step is 0 and becomes bf16(1e-3) by the final fix-up (:104).

    idx may be supplied to evaluate the step for a given channel list.
    """
    x = _as_bmn(x).to(BF16).clone()
    if idx is None:
        idx = outlier_channels(x, ratio)
    x[:, :, idx] = 0
    x0 = x[0]
    s = (x0.max(dim=-2, keepdim=True).values - x0.min(dim=-2, keepdim=True).values) / (2 ** q_bit - 1)
    s += (s == 0) * 1e-3
    return idx, s.to(BF16)


def softmax_threshold(a: torch.Tensor, ratio: float) -> torch.Tensor:
    """Exact order statistic used as the keep-threshold (compress_function.py:30-32)."""
    k = int(a.numel() * (1 - ratio))
    return torch.kthvalue(a.float().flatten(), k).values


def update_dict(old: dict, new: dict, iteration: int) -> dict:
    """Running mean of calibration statistics (compress_function.py:15-27)."""
    for name in old.keys():
        if name == 'outlier_channel_index' or old[name] is None:
            old[name] = new[name]
        else:
            old[name] = (iteration * old[name] + new[name]) / (iteration + 1)
    return old


# --------------------------------------------------------------------------------------
# integer codes, packing
# --------------------------------------------------------------------------------------
def round_half_away(t: torch.Tensor) -> torch.Tensor:
    """C roundf on an fp32 tensor (libdevice round, compress_function_kernel.py:103)."""
    r = torch.trunc(t)
    frac = t - r                       # exact: |t| < 2^23 or t is already integral
    return torch.where(frac.abs() >= 0.5, r + torch.sign(t), r)


def quant_codes(x: torch.Tensor, s: torch.Tensor, q_bit: int,
                z: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Unpacked codes 0..2^q-1 as uint8 [B,M,N] (compress_function_kernel.py:92-110, :292).

    t = fp32(x)/fp32(s) (+ fp32(z)), IEEE division; r = roundf(t); clamp to
    [-2^(q-1), 2^(q-1)-1]; code = r + 2^(q-1).  A NaN t gives code 0 (what the
    reference's float->uint conversion yields).
    """
    x = _as_bmn(x).to(BF16)
    s = s.to(BF16).reshape(1, 1, -1)
    t = x.float() / s.float()
    if z is not None:
        t = t + z.to(BF16).reshape(1, 1, -1).float()
    half = 2 ** (q_bit - 1)
    r = round_half_away(t)
    r = torch.clamp(r, -half, half - 1) + half
    r = torch.where(torch.isnan(t), torch.zeros_like(r), r)
    return r.to(torch.uint8)


def pack_codes(c: torch.Tensor, q_bit: int) -> torch.Tensor:
    """Pack codes [.., N] into bytes [.., N*q/8] (compress_function_kernel.py:77-85,96-112).

    Columns are processed in blocks of 32.  With epp = 8/q elements per byte and
    w = 32/epp bytes per block, byte p*w + j holds the elements at columns
    32p + j + i*w (i = 0..epp-1), element i at bit offset q*i.
    """
    epp = 8 // q_bit
    w = 32 // epp
    n = c.shape[-1]
    assert n % 32 == 0
    blk = c.reshape(*c.shape[:-1], n // 32, epp, w).to(torch.int32)
    out = torch.zeros(*c.shape[:-1], n // 32, w, dtype=torch.int32, device=c.device)
    for i in range(epp):
        out |= blk[..., i, :] << (q_bit * i)
    return out.reshape(*c.shape[:-1], n // epp).to(torch.uint8)


def unpack_codes(p: torch.Tensor, q_bit: int) -> torch.Tensor:
    """Inverse of pack_codes (compress_function_kernel.py:193-206)."""
    epp = 8 // q_bit
    w = 32 // epp
    nb = p.shape[-1]
    blk = p.reshape(*p.shape[:-1], nb // w, 1, w).to(torch.int32)
    shifts = (torch.arange(epp, dtype=torch.int32, device=p.device) * q_bit).reshape(epp, 1)
    c = (blk >> shifts) & (2 ** q_bit - 1)
    return c.reshape(*p.shape[:-1], nb * epp).to(torch.uint8)


def compress(x, s, q_bit, z=None):
    """compression_quantization[_with_zero_point] (compress_function.py:178-210,245-274)."""
    return pack_codes(quant_codes(x, s, q_bit, z), q_bit)


def dequant(c: torch.Tensor, s: torch.Tensor, q_bit: int,
            z: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x^ = bf16( (bf16(code) - 2^(q-1) [- bf16(z)]) * s ) (compress_function_kernel.py:200-204,382-388)."""
    s = s.to(BF16).reshape(1, 1, -1)
    v = c.to(BF16) - (2 ** (q_bit - 1))
    if z is not None:
        v = v - z.to(BF16).reshape(1, 1, -1)
    return (v * s).to(WIRE)


def decompress(p, s, q_bit, z=None, is_head=False, num_heads=1):
    """decompression_dequantization[_with_zero_point] (compress_function.py:214-241,278-306)."""
    x = dequant(unpack_codes(p, q_bit), s, q_bit, z)
    if is_head:
        x = hidden_to_head_shape(x, num_heads)
    return x


def compress_channel_base(x, s, idx, q_bit):
    """outlier_subtraction_fuse_compression_quantization (compress_function.py:111-143):
    gather the outlier columns (in idx order), zero them, quantise the rest."""
    x = _as_bmn(x).to(BF16).clone()
    x_outlier = x[:, :, idx]
    x[:, :, idx] = 0
    return x_outlier, compress(x, s, q_bit)


def decompress_channel_base(p, s, x_outlier, idx, q_bit, is_head=False, num_heads=1):
    """outlier_addition_fuse_decompression_dequantization (compress_function.py:147-174)."""
    x = decompress(p, s, q_bit)
    x[:, :, idx] = x_outlier.to(x.dtype)
    if is_head:
        x = hidden_to_head_shape(x, num_heads)
    return x


# --------------------------------------------------------------------------------------
# attention-map compression
# --------------------------------------------------------------------------------------
def softmax_compress(a: torch.Tensor, thr) -> Tuple[torch.Tensor, torch.Tensor]:
    """(a * (a > thr)).flatten().to_sparse() as (int64 indices ascending, bf16 values)
    (compress_function.py:309-313), literally: the product with the mask, then the non-zero
    entries.  So a kept element is one with a > thr and a != 0 - or a NaN (NaN * 0 = NaN != 0)."""
    flat = a.flatten()
    prod = flat * (flat > thr)
    idx = torch.nonzero(prod).flatten()
    return idx, flat[idx]            # = prod[idx] as numbers; the element itself so that a NaN keeps its payload


def softmax_restore(idx, vals, shape) -> torch.Tensor:
    """to_dense().reshape(shape) (compress_function.py:316-317)."""
    out = torch.zeros(math.prod(shape), dtype=vals.dtype, device=vals.device)
    out[idx] = vals
    return out.reshape(shape)


def softmax_fwd(s: torch.Tensor, scale: float, mask=None) -> torch.Tensor:
    """bf16(softmax_fp32(bf16(bf16(s * scale) + mask))): `q @ k^T / sqrt(d)` (a multiplication by the
    fp32 reciprocal in torch's device kernel), `+ attention_mask`, `torch.softmax(dtype=bf16)` with
    its fp32 internals (fused_llama_layer_intra_inter_full_fuse.py:159-167)."""
    t = (s.to(BF16).float() * torch.tensor(scale, dtype=F32)).to(BF16)
    if mask is not None:
        t = t + mask.to(BF16)
    return torch.softmax(t.float(), dim=-1).to(BF16)


def softmax_bwd(y: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """o = bf16((g - sum_row bf16(y*g)) * y), row sum in fp32 (softmax_kernels.py:31-35)."""
    yg = (y.to(BF16) * g.to(BF16)).float()
    ssum = yg.sum(dim=-1, keepdim=True)
    return ((g.float() - ssum) * y.float()).to(BF16)


# --------------------------------------------------------------------------------------
# rotary position embedding
# --------------------------------------------------------------------------------------
def rope(x, cos, sin, backward=False):
    """x [B,S,H,D] -> rotated copy.  Halves (x1|x2) -> (x1*c - x2*s | x2*c + x1*s) with c, s the FIRST
    half of table row s (rope_kernels.py:54-59, :72-78); backward negates s (:61-63).  x is
    converted to the table's dtype and every product and sum is a tensor operation of that dtype
    (bf16 tables: rounded after each operation; fp32 tables: fp32), result rounded to x's dtype."""
    cos, sin = cos.squeeze(), sin.squeeze()
    S, half = x.shape[1], x.shape[-1] // 2
    c = cos[:S, :half][None, :, None, :]
    s = sin[:S, :half][None, :, None, :]
    if backward:
        s = -s
    x1, x2 = x[..., :half].to(c.dtype), x[..., half:].to(c.dtype)
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1).to(x.dtype)


# --------------------------------------------------------------------------------------
# norms and element-wise backward operators
# --------------------------------------------------------------------------------------
def rmsnorm_fwd(x, w, eps):
    """rstd = 1/sqrt(mean(x^2)+eps) in fp32; y = bf16(x*rstd*w) (rmsnorm_kernels.py:34-54)."""
    xf = x.float()
    rstd = 1.0 / torch.sqrt((xf * xf).mean(dim=-1) + eps)
    y = (xf * rstd.unsqueeze(-1) * w.float()).to(x.dtype)
    return y, rstd.reshape(-1)


def rmsnorm_bwd(dy, x, w, rstd):
    """dx = (w*dy - (x^*c1 + c2)) * rstd with c1 = mean(x^*w*dy), c2 = mean(w*dy)
    (rmsnorm_kernels.py:92-100: the reference keeps LayerNorm's c2 term);
    dw = sum_rows dy*x^ (rmsnorm_updatable_kernels.py:102,117-137)."""
    n = x.shape[-1]
    xf = x.float().reshape(-1, n)
    dyf = dy.float().reshape(-1, n)
    xhat = xf * rstd.reshape(-1, 1)
    wdy = w.float() * dyf
    c1 = (xhat * wdy).mean(dim=-1, keepdim=True)
    c2 = wdy.mean(dim=-1, keepdim=True)
    dx = ((wdy - (xhat * c1 + c2)) * rstd.reshape(-1, 1)).to(dy.dtype).reshape(dy.shape)
    dw = (dyf * xhat).sum(dim=0).to(w.dtype)
    return dx, dw


def layernorm_fwd(x, w, b, eps):
    """(y bf16, mean fp32 [rows], rstd fp32 [rows]): mean and centred variance in fp32,
    y = (x - mean)*rstd*w + b rounded once (layernorm_kernels.py:27-56)."""
    xf = x.float()
    mean = xf.sum(-1, keepdim=True) / x.shape[-1]
    d = xf - mean
    var = (d * d).sum(-1, keepdim=True) / x.shape[-1]
    rstd = 1.0 / torch.sqrt(var + eps)
    y = (d * rstd) * w.float() + b.float()
    return y.to(x.dtype), mean.reshape(-1), rstd.reshape(-1)


def layernorm_bwd(dy, x, w, mean, rstd):
    """dx = (w*dy - (x^*c1 + c2))*rstd, c1 = mean(x^*w*dy), c2 = mean(w*dy), fp32 (layernorm_kernels.py:92-104)."""
    n = x.shape[-1]
    shp = x.shape[:-1] + (1,)
    xh = (x.float() - mean.reshape(shp)) * rstd.reshape(shp)
    wdy = w.float() * dy.float()
    c1 = (xh * wdy).sum(-1, keepdim=True) / n
    c2 = wdy.sum(-1, keepdim=True) / n
    return ((wdy - (xh * c1 + c2)) * rstd.reshape(shp)).to(dy.dtype)


def _sig_bf16(x):
    return torch.sigmoid(x.float()).to(BF16)


def silu_bwd(x, g):
    """g * (sig * (1 + x*(1-sig))), bf16 after every operation (silu_kernels.py:42-43)."""
    x = x.to(BF16); g = g.to(BF16)
    sig = _sig_bf16(x)
    return g * (sig * (1 + x * (1 - sig)))


def silu_mul(x1, x2):
    """(sig(x1)*x1)*x2 in bf16 (silu_kernels.py:103-104)."""
    x1 = x1.to(BF16); x2 = x2.to(BF16)
    return (_sig_bf16(x1) * x1) * x2


def silu_mul_bwd(x, u, g):
    """Backward of the gated product silu(x) * u: (silu_bwd(x, g*u), g * F.silu(x)), every product rounded to
    bf16 and silu itself evaluated in fp32 and rounded once - the composition the layers write out
    (fused_llama_layer_intra_inter.py:362-381)."""
    x = x.to(BF16); u = u.to(BF16); g = g.to(BF16)
    return silu_bwd(x, g * u), g * torch.nn.functional.silu(x)


GELU_GAMMA = 0.7978845608028654
GELU_KAPPA = 0.044715


def gelu_bwd(x, g):
    """Derivative of tanh-GELU times g (gelu_kernels.py:49-56).  Evaluated in fp32 with
    one final rounding; the reference's intermediate precision is not recoverable from
    its source, so this operator is held to tolerance only."""
    xf = x.float(); gf = g.float()
    x2 = xf * xf
    y = GELU_GAMMA * (xf + GELU_KAPPA * x2 * xf)
    t = torch.tanh(y)
    o = 0.5 * ((1 + t) + xf * ((1 - t * t) * GELU_GAMMA * (1 + 3 * GELU_KAPPA * x2))) * gf
    return o.to(x.dtype)


# --------------------------------------------------------------------------------------
# fused LoRA-SiLU-Hadamard
# --------------------------------------------------------------------------------------
def _lora_term(xa, b):
    """bf16( sum_r xa[.,r] * b[r,.] ) with fp32 accumulation (tl.dot(...).to(bf16),
    triton_fuse_lora_silu_hadamard_forward_kernels.py:119)."""
    return (xa.float() @ b.float()).to(BF16)


def lora_add(x_main, xa, b):
    """x_main + x_lora_a @ w_lora_b in bf16, product rounded before the add
    (models/utils/compute_utils.py:21-24; the same expression rebuilds q, k, v in backward,
    models/llama/fused_llama_layer_intra_inter_full_fuse.py:417,441,449)."""
    return x_main.to(BF16) + _lora_term(xa, b)


def lora_products(x, u=None, v=None):
    """The rank-R products of lora_forward / lora_backward over a wide operand x [T, N]
    (models/utils/compute_utils.py:22, :30-33), accumulated in float64 and rounded once:
    u^T x [R, N] (xa^T @ grad_y, x^T @ grad_medium) and x v^T [T, R] (x @ A, grad_y @ B^T)."""
    x2 = x.reshape(-1, x.shape[-1]).double()
    p1 = None if u is None else (u.reshape(-1, u.shape[-1]).double().t() @ x2).to(BF16)
    p2 = None if v is None else (x2 @ v.double().t()).to(BF16).reshape(*x.shape[:-1], v.shape[0])
    return p1, p2


def fused_fwd(xa1, b1, x1, s1, xa2, b2, x2, s2, q_bit):
    """triton_fuse_silu_forward (…forward_kernels.py:104-146,152-182) -> (q1, q2, o)."""
    x1 = x1.to(BF16); x2 = x2.to(BF16)
    q1 = compress(x1, s1, q_bit)
    q2 = compress(x2, s2, q_bit)
    y1 = x1 + _lora_term(xa1, b1)
    y1 = y1 * _sig_bf16(y1)
    y2 = x2 + _lora_term(xa2, b2)
    return q1, q2, y1 * y2


def fused_bwd(xa1, b1, q1, s1, xa2, b2, q2, s2, grad_o, q_bit):
    """triton_fuse_silu_backward (…backward_kernels.py:106-149,152-178)
    -> (o, grad_gate, grad_up)."""
    return fused_bwd_dense(xa1, b1, decompress(q1, s1, q_bit), xa2, b2, decompress(q2, s2, q_bit), grad_o)


def fused_bwd_dense(xa1, b1, x1, xa2, b2, x2, grad_o):
    """The arithmetic of fused_bwd after its two dequantisations (…backward_kernels.py:124-149): x1, x2 are the
    frozen-weight parts of gate and up as the kernel holds them at that point."""
    g = grad_o.to(BF16)
    x1 = x1.to(BF16); x2 = x2.to(BF16)
    y1 = x1 + _lora_term(xa1, b1)
    y2 = x2 + _lora_term(xa2, b2)
    sig = _sig_bf16(y1)
    sil = y1 * sig
    o = sil * y2
    gh1 = g * y2
    gh2 = g * sil
    grad_gate = gh1 * (sig * (1.0 + y1 * (1.0 - sig)))
    return o, grad_gate, gh2


# --------------------------------------------------------------------------------------
# NF4 frozen weights (bitsandbytes 0.43.2 is not importable here: its published format is restated)
# --------------------------------------------------------------------------------------
NF4_TABLE = torch.tensor([-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635,
                          -0.18477343022823334, -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725,
                          0.24611230194568634, 0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
                          0.7229568362236023, 1.0], dtype=F32)


def nf4_absmax(absmax, nested=None):
    """fp32 block statistics; nested = (code2 fp32 [256], absmax2 fp32, blocksize2, offset) for double
    quantisation: code2[absmax] * absmax2[block / blocksize2] + offset
    (bitsandbytes functional.py dequantize_4bit: dequantize_blockwise(absmax, state2) + offset)."""
    if nested is None:
        return absmax.float()
    code2, absmax2, bs2, offset = nested
    idx = torch.arange(absmax.numel()) // bs2
    return code2.float()[absmax.long()] * absmax2.float()[idx] + float(offset)


def nf4_dequant(packed, absmax, shape, blocksize=64, nested=None, table=NF4_TABLE):
    """bf16 weight of `shape`: element 2i from the HIGH nibble of byte i, 2i+1 from the low one
    (bitsandbytes csrc/kernels.cu kDequantizeBlockwise, NF4 branch); value = table[code] * absmax[i / blocksize]
    in fp32, rounded to bf16 (what models/utils/compute_utils.py:19 gets from BF.dequantize_nf4)."""
    p = packed.reshape(-1).long()
    codes = torch.stack([p >> 4, p & 15], dim=1).reshape(-1)
    am = nf4_absmax(absmax.reshape(-1), nested)
    vals = table.float()[codes] * am[torch.arange(codes.numel()) // blocksize]
    return vals.to(BF16).reshape(shape)


def nf4_quantize(w, blocksize=64, code2=None, blocksize2=256):
    """Test-data generator (not a restatement of bitsandbytes' quantiser): nearest NF4 level of
    w / absmax per block; with code2, the statistics are themselves quantised to 8 bits around their
    mean.  -> (packed uint8 [n/2], absmax fp32 [nblocks] or uint8 codes, nested tuple or None)."""
    flat = w.float().reshape(-1)
    n = flat.numel()
    nb = -(-n // blocksize)
    pad = torch.zeros(nb * blocksize)
    pad[:n] = flat
    blocks = pad.reshape(nb, blocksize)
    absmax = blocks.abs().amax(dim=1).clamp_min(1e-12)
    codes = ((blocks / absmax[:, None])[..., None] - NF4_TABLE).abs().argmin(dim=-1).reshape(-1)[:n]
    packed = ((codes[0::2] << 4) | codes[1::2]).to(torch.uint8)
    if code2 is None:
        return packed, absmax, None
    offset = absmax.mean()
    rest = absmax - offset
    nb2 = -(-nb // blocksize2)
    pad2 = torch.zeros(nb2 * blocksize2)
    pad2[:nb] = rest
    b2 = pad2.reshape(nb2, blocksize2)
    absmax2 = b2.abs().amax(dim=1).clamp_min(1e-12)
    c2 = ((b2 / absmax2[:, None])[..., None] - code2.float()).abs().argmin(dim=-1).reshape(-1)[:nb]
    return packed, c2.to(torch.uint8), (code2, absmax2, blocksize2, offset)
