"""Fused LoRA-SiLU-Hadamard forward.  The module and function keep the reference's names
(operators/triton_fuse_lora_silu_hadamard_forward_kernels.py:152-182) so that the fused layers
import them unchanged; the implementation is an MFMA kernel for gfx950, not Triton."""
from ._fuse import fuse_forward


def triton_fuse_silu_forward(xa1, b1, x1, s1, xa2, b2, x2, s2, quantize_bit=8):
    """-> (q1, q2, o): packed codes of x1 and x2, and silu(x1 + xa1@b1) * (x2 + xa2@b2)."""
    return fuse_forward(xa1, b1, x1, s1, xa2, b2, x2, s2, quantize_bit)
