"""Compress / decompress operators with the reference's Python API
(operators/compress_function.py), running on hand-written gfx950 kernels.

Function names, argument order and return values follow the reference so that the fused
decoder layers can call either implementation.  Differences, all deliberate:
  * `outlier_subtraction_fuse_compression_quantization` does not modify its input
    unless `zero_input=True` is passed (the reference zeroes the outlier columns of `x`
    in place, which is why its callers hand it a clone);
  * 4-D `[B, H, S, D]` inputs are read in place through their strides instead of being
    transposed into a temporary `[B, S, H*D]` copy;
  * outlier channels are chosen with a defined tie rule (norm descending, then channel
    index ascending) where `torch.topk` leaves the order open.
"""
from __future__ import annotations

import torch

from .. import _lib

BF16 = torch.bfloat16


# ---------------------------------------------------------------------------------------
# shape helpers (reference: operators/compress_function.py:6-13)
# ---------------------------------------------------------------------------------------
def hidden_to_head_shape(x: torch.Tensor, num_heads: int):
    bsz, seq_len, hidden = x.shape
    return x.reshape(bsz, seq_len, num_heads, hidden // num_heads).transpose(1, 2)


def head_to_hidden_shape(x: torch.Tensor):
    bsz, _, seq_len, _ = x.shape
    return x.transpose(1, 2).reshape(bsz, seq_len, -1)


def update_dict(old_dict, new_dict, iteration):
    """Running mean of calibration statistics; the outlier channel list is replaced
    (reference: operators/compress_function.py:15-27)."""
    for name in old_dict:
        fresh = new_dict[name]
        if name == 'outlier_channel_index' or old_dict[name] is None:
            old_dict[name] = fresh
        else:
            old_dict[name] = (iteration * old_dict[name] + fresh) / (iteration + 1)
    return old_dict


# ---------------------------------------------------------------------------------------
# addressing of the activation tensor handed to the kernels
# ---------------------------------------------------------------------------------------
class _Addr:
    """Logical [B, M, N] view of a 3-D or 4-D ([B, H, S, D]) bf16 tensor as the kernels
    address it: element (b, m, c) at b*sb + m*sm + (c // hd)*sh + c % hd."""
    __slots__ = ("t", "B", "M", "N", "sb", "sm", "hd", "sh")

    def __init__(self, x: torch.Tensor):
        if x.dim() == 4:
            ok = (x.stride(3) == 1 and x.shape[3] % 8 == 0 and x.data_ptr() % 16 == 0
                  and all(s % 8 == 0 for s in x.stride()[:3]))
            if not ok:
                x = x.contiguous()
            B, H, S, D = x.shape
            self.t, self.B, self.M, self.N = x, B, S, H * D
            self.sb, self.sm, self.hd, self.sh = x.stride(0), x.stride(2), D, x.stride(1)
        elif x.dim() == 3:
            ok = (x.stride(2) == 1 and x.data_ptr() % 16 == 0 and x.stride(0) % 8 == 0 and x.stride(1) % 8 == 0)
            if not ok:
                x = x.contiguous()
            B, M, N = x.shape
            self.t, self.B, self.M, self.N = x, B, M, N
            self.sb, self.sm, self.hd, self.sh = x.stride(0), x.stride(1), N, 0
        else:
            raise ValueError(f"expected a 3-D or 4-D activation tensor, got shape {tuple(x.shape)}")


def _vec(t: torch.Tensor, n: int, name: str) -> torch.Tensor:
    """A per-channel vector ([1, N], [N], ...) as contiguous, aligned bf16 [N]."""
    t = t.to(BF16).reshape(-1)
    if t.numel() != n:
        raise ValueError(f"{name} must have {n} elements (one per channel), got {t.numel()}")
    if not t.is_contiguous() or t.data_ptr() % 16:
        t = t.clone(memory_format=torch.contiguous_format)
    return t


def _check_bits(quantize_bit: int) -> int:
    if quantize_bit not in (2, 4, 8):
        raise ValueError(f"quantize_bit must be 2, 4 or 8, got {quantize_bit}")
    return 8 // quantize_bit


def _quantize(x, s, z, channel, quantize_bit, dtype, zero_input=False):
    if dtype != BF16:
        raise NotImplementedError("the gfx950 kernels compute in bfloat16 only")
    epp = _check_bits(quantize_bit)
    _lib.require_gpu(x, s, z, channel)
    if x.dtype != BF16:
        x = x.to(BF16)
    a = _Addr(x)
    if a.N % 32:
        raise ValueError(f"channel count must be a multiple of 32, got {a.N}")
    s = _vec(s, a.N, "scale")
    z = None if z is None else _vec(z, a.N, "zero point")
    q = torch.empty((a.B, a.M, a.N // epp), device=x.device, dtype=torch.uint8)
    k = 0
    x_outlier = None
    if channel is not None:
        channel = channel.to(torch.int64).contiguous()
        k = channel.numel()
        x_outlier = torch.empty((a.B, a.M, k), device=x.device, dtype=BF16)
    _lib.call("hyc_quant_pack", a.t.data_ptr(), s.data_ptr(), _lib.ptr(z), q.data_ptr(),
              _lib.ptr(channel) if k else None, k, _lib.ptr(x_outlier) if k else None, int(bool(zero_input)),
              a.B, a.M, a.N, a.sb, a.sm, a.hd, a.sh, quantize_bit, _lib.stream_of(x))
    return x_outlier, q


def _dequantize(q, s, z, x_outlier, channel, quantize_bit, is_head, num_heads, dtype):
    if dtype != BF16:
        raise NotImplementedError("the gfx950 kernels compute in bfloat16 only")
    epp = _check_bits(quantize_bit)
    _lib.require_gpu(q, s, z, x_outlier, channel)
    B, M, nbytes = q.shape
    N = s.shape[-1]
    if nbytes * epp != N:
        raise ValueError(f"packed width {nbytes} does not match {N} channels at {quantize_bit} bits")
    if N % 32:
        raise ValueError(f"channel count must be a multiple of 32, got {N}")
    if q.dtype != torch.uint8:
        raise ValueError("packed codes must be uint8")
    q = q.contiguous()
    s = _vec(s, N, "scale")
    z = None if z is None else _vec(z, N, "zero point")
    x = torch.empty((B, M, N), device=q.device, dtype=BF16)
    k = 0
    if channel is not None:
        channel = channel.to(torch.int64).contiguous()
        k = channel.numel()
        x_outlier = x_outlier.to(BF16).contiguous()
        if tuple(x_outlier.shape) != (B, M, k):
            raise ValueError(f"x_outlier must have shape {(B, M, k)}, got {tuple(x_outlier.shape)}")
    _lib.call("hyc_unpack_dequant", q.data_ptr(), s.data_ptr(), _lib.ptr(z), x.data_ptr(),
              _lib.ptr(channel) if k else None, k, _lib.ptr(x_outlier) if k else None,
              B, M, N, M * N, N, N, 0, quantize_bit, _lib.stream_of(q))
    if is_head:
        x = hidden_to_head_shape(x, num_heads=num_heads)
    return x


# ---------------------------------------------------------------------------------------
# compress / decompress interface (reference: operators/compress_function.py:111-306)
# ---------------------------------------------------------------------------------------
def outlier_subtraction_fuse_compression_quantization(x, s, channel, quantize_bit=8, dtype=BF16, zero_input=False):
    """-> (x_outlier [B,M,k] bf16, q [B,M,N*bits/8] uint8).  Reference :111-143."""
    return _quantize(x, s, None, channel, quantize_bit, dtype, zero_input)


def outlier_addition_fuse_decompression_dequantization(q, s, x_outlier, channel, quantize_bit=8, is_head=False,
                                                       num_heads=1, dtype=BF16):
    """Inverse of the above.  Reference :147-174."""
    return _dequantize(q, s, None, x_outlier, channel, quantize_bit, is_head, num_heads, dtype)


def compression_quantization(x, s, quantize_bit=8, dtype=BF16):
    """Reference :178-210."""
    return _quantize(x, s, None, None, quantize_bit, dtype)[1]


def decompression_dequantization(q, s, quantize_bit=8, is_head=False, num_heads=1, dtype=BF16):
    """Reference :214-241."""
    return _dequantize(q, s, None, None, None, quantize_bit, is_head, num_heads, dtype)


def compression_quantization_with_zero_point(x, s, z, quantize_bit=8, dtype=BF16):
    """Reference :245-274."""
    return _quantize(x, s, z, None, quantize_bit, dtype)[1]


def decompression_dequantization_with_zero_point(q, s, z, quantize_bit=8, is_head=False, num_heads=1, dtype=BF16):
    """Reference :278-306."""
    return _dequantize(q, s, z, None, None, quantize_bit, is_head, num_heads, dtype)
