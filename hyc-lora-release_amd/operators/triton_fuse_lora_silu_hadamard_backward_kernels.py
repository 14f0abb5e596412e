"""Fused LoRA-SiLU-Hadamard backward (reference:
operators/triton_fuse_lora_silu_hadamard_backward_kernels.py:152-178); see the forward module."""
from ._fuse import fuse_backward


def triton_fuse_silu_backward(xa1, b1, q1, s1, xa2, b2, q2, s2, grad_o, quantize_bit=8):
    """-> (o, grad_gate, grad_up)."""
    return fuse_backward(xa1, b1, q1, s1, xa2, b2, q2, s2, grad_o, quantize_bit)
