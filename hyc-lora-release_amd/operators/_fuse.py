"""Launchers of the fused LoRA-SiLU-Hadamard kernels."""
import torch

from .. import _lib

BF16 = torch.bfloat16


def _prep(t, name):
    if t.dtype != BF16:
        t = t.to(BF16)
    t = t.contiguous()
    if t.data_ptr() % 16:
        t = t.clone()
    return t


def _validate(xa1, b1, s1, xa2, b2, s2, quantize_bit, rows, n):
    """Everything the kernels take on trust: they read xa[row, 0..R) for each of `rows` rows,
    B[0..R, 0..N) and s[0..N), so a short operand would be read out of bounds on the device."""
    if quantize_bit not in (2, 4, 8):
        raise ValueError(f"quantize_bit must be 2, 4 or 8, got {quantize_bit}")
    if b1.dim() != 2 or b2.dim() != 2:
        raise ValueError("LoRA-B operands must be matrices [R, N]")
    r = b1.shape[0]
    if b2.shape[0] != r or xa1.shape[-1] != r or xa2.shape[-1] != r:
        raise ValueError("LoRA rank mismatch between xa1/b1/xa2/b2")
    if r % 4 or not 4 <= r <= 64:
        raise ValueError(f"LoRA rank must be a multiple of 4 in 4..64, got {r}")
    if b1.shape[1] != n or b2.shape[1] != n:
        raise ValueError("LoRA-B width does not match the activation width")
    if n % 32:
        raise ValueError(f"channel count must be a multiple of 32, got {n}")
    for xa, name in ((xa1, "xa1"), (xa2, "xa2")):
        if xa.numel() != rows * r:
            raise ValueError(f"{name} must hold one row of {r} values per activation row ({rows} rows), "
                             f"got shape {tuple(xa.shape)}")
    for s, name in ((s1, "s1"), (s2, "s2")):
        if s.numel() != n:
            raise ValueError(f"{name} must have {n} elements (one per channel), got {s.numel()}")
    return r


def _common(xa1, b1, s1, xa2, b2, s2, quantize_bit, n):
    r = b1.shape[0]
    # [R, N] views of [N, R] contiguous weights (lora_B.weight.T) are read as they lie in memory
    bt = int(all(b.dtype == BF16 and not b.is_contiguous() and b.mT.is_contiguous() and b.data_ptr() % 8 == 0
                 for b in (b1, b2)))
    if not bt:
        b1, b2 = _prep(b1, "b1"), _prep(b2, "b2")
    return (_prep(xa1, "xa1"), b1, _prep(s1.reshape(-1), "s1"),
            _prep(xa2, "xa2"), b2, _prep(s2.reshape(-1), "s2"), r, bt)


def fuse_forward(xa1, b1, x1, s1, xa2, b2, x2, s2, quantize_bit=8):
    if x1.dim() != 3 or x2.shape != x1.shape:
        raise ValueError(f"x1 and x2 must be [B, M, N] of one shape, got {tuple(x1.shape)} and {tuple(x2.shape)}")
    B, M, N = x1.shape
    _validate(xa1, b1, s1, xa2, b2, s2, quantize_bit, B * M, N)
    _lib.require_gpu(xa1, b1, x1, s1, xa2, b2, x2, s2)
    xa1, b1, s1, xa2, b2, s2, R, bt = _common(xa1, b1, s1, xa2, b2, s2, quantize_bit, N)
    x1 = _prep(x1, "x1")
    x2 = _prep(x2, "x2")
    epp = 8 // quantize_bit
    q1 = torch.empty((B, M, N // epp), device=x1.device, dtype=torch.uint8)
    q2 = torch.empty((B, M, N // epp), device=x1.device, dtype=torch.uint8)
    o = torch.empty((B, M, N), device=x1.device, dtype=BF16)
    _lib.call("hyc_lora_silu_mul_fwd", xa1.data_ptr(), b1.data_ptr(), x1.data_ptr(), s1.data_ptr(),
              xa2.data_ptr(), b2.data_ptr(), x2.data_ptr(), s2.data_ptr(), q1.data_ptr(), q2.data_ptr(),
              o.data_ptr(), B * M, N, R, quantize_bit, bt, _lib.stream_of(x1))
    return q1, q2, o


def fuse_backward(xa1, b1, q1, s1, xa2, b2, q2, s2, grad_o, quantize_bit=8):
    if grad_o.dim() != 3:
        raise ValueError(f"grad_o must be [B, M, N], got shape {tuple(grad_o.shape)}")
    B, M, N = grad_o.shape
    _validate(xa1, b1, s1, xa2, b2, s2, quantize_bit, B * M, N)
    want = (B, M, N * quantize_bit // 8)
    if tuple(q1.shape) != want or tuple(q2.shape) != want or q1.dtype != torch.uint8 or q2.dtype != torch.uint8:
        raise ValueError(f"packed codes must be uint8 of shape {want}")
    _lib.require_gpu(xa1, b1, q1, s1, xa2, b2, q2, s2, grad_o)
    xa1, b1, s1, xa2, b2, s2, R, bt = _common(xa1, b1, s1, xa2, b2, s2, quantize_bit, N)
    grad_o = _prep(grad_o, "grad_o")
    q1 = q1.contiguous()
    q2 = q2.contiguous()
    o = torch.empty((B, M, N), device=grad_o.device, dtype=BF16)
    gg = torch.empty_like(o)
    gu = torch.empty_like(o)
    _lib.call("hyc_lora_silu_mul_bwd", xa1.data_ptr(), b1.data_ptr(), q1.data_ptr(), s1.data_ptr(),
              xa2.data_ptr(), b2.data_ptr(), q2.data_ptr(), s2.data_ptr(), grad_o.data_ptr(), o.data_ptr(),
              gg.data_ptr(), gu.data_ptr(), B * M, N, R, quantize_bit, bt, _lib.stream_of(grad_o))
    return o, gg, gu
