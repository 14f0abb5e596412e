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


def _common(xa1, b1, s1, xa2, b2, s2, quantize_bit, n):
    if quantize_bit not in (2, 4, 8):
        raise ValueError(f"quantize_bit must be 2, 4 or 8, got {quantize_bit}")
    r = b1.shape[0]
    if b2.shape[0] != r or xa1.shape[-1] != r or xa2.shape[-1] != r:
        raise ValueError("LoRA rank mismatch between xa1/b1/xa2/b2")
    if b1.shape[1] != n or b2.shape[1] != n:
        raise ValueError("LoRA-B width does not match the activation width")
    if n % 32:
        raise ValueError(f"channel count must be a multiple of 32, got {n}")
    # [R, N] views of [N, R] contiguous weights (lora_B.weight.T) are read as they lie in memory
    bt = int(all(b.dtype == BF16 and not b.is_contiguous() and b.mT.is_contiguous() and b.data_ptr() % 8 == 0
                 for b in (b1, b2)))
    if not bt:
        b1, b2 = _prep(b1, "b1"), _prep(b2, "b2")
    return (_prep(xa1, "xa1"), b1, _prep(s1.reshape(-1), "s1"),
            _prep(xa2, "xa2"), b2, _prep(s2.reshape(-1), "s2"), r, bt)


def fuse_forward(xa1, b1, x1, s1, xa2, b2, x2, s2, quantize_bit=8):
    _lib.require_gpu(xa1, b1, x1, s1, xa2, b2, x2, s2)
    B, M, N = x1.shape
    assert x2.shape == x1.shape
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
    _lib.require_gpu(xa1, b1, q1, s1, xa2, b2, q2, s2, grad_o)
    B, M, N = grad_o.shape
    xa1, b1, s1, xa2, b2, s2, R, bt = _common(xa1, b1, s1, xa2, b2, s2, quantize_bit, N)
    grad_o = _prep(grad_o, "grad_o")
    q1 = q1.contiguous()
    q2 = q2.contiguous()
    want = (B, M, N * quantize_bit // 8)
    if tuple(q1.shape) != want or tuple(q2.shape) != want or q1.dtype != torch.uint8 or q2.dtype != torch.uint8:
        raise ValueError(f"packed codes must be uint8 of shape {want}")
    o = torch.empty((B, M, N), device=grad_o.device, dtype=BF16)
    gg = torch.empty_like(o)
    gu = torch.empty_like(o)
    _lib.call("hyc_lora_silu_mul_bwd", xa1.data_ptr(), b1.data_ptr(), q1.data_ptr(), s1.data_ptr(),
              xa2.data_ptr(), b2.data_ptr(), q2.data_ptr(), s2.data_ptr(), grad_o.data_ptr(), o.data_ptr(),
              gg.data_ptr(), gu.data_ptr(), B * M, N, R, quantize_bit, bt, _lib.stream_of(grad_o))
    return o, gg, gu
