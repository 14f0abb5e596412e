"""SiLU backward and SiLU*x2 on gfx950 (reference API: operators/silu_kernels.py:48-63,110-125)."""
import torch

from .. import _lib
from ._elementwise import binary


def silu_backward(x, g):
    """g * d/dx[x * sigmoid(x)], bf16 after every operation."""
    return binary("hyc_silu_bwd", x, g)


def silu_hadamard(x, g):
    """(sigmoid(x) * x) * g — SiLU of the first argument times the second."""
    return binary("hyc_silu_mul", x, g)


def silu_once_hadamard(x, u):
    """u * F.silu(x): SiLU evaluated in fp32 and rounded to bf16 once, then the product - the form in which
    the reference's backward recomputes the gated product
    (models/llama/fused_llama_layer_intra_inter.py:362,370), one pass instead of two."""
    return binary("hyc_silu_once_mul", x, u)


def silu_hadamard_backward(x, u, g):
    """Backward of the gated product silu(x) * u for an upstream gradient g, in one pass over the three
    tensors: -> (grad_x, grad_u) = (silu_backward(x, g * u), g * F.silu(x)).  No counterpart in the
    reference, whose layers compose exactly this from F.silu, two products and silu_backward
    (models/llama/fused_llama_layer_intra_inter.py:362-381)."""
    assert x.shape == u.shape == g.shape
    _lib.require_gpu(x, u, g)
    if not (x.dtype == u.dtype == g.dtype == torch.bfloat16):
        raise NotImplementedError("silu_hadamard_backward computes in bfloat16")
    x, u, g = x.contiguous(), u.contiguous(), g.contiguous()
    gx, gu = torch.empty_like(x), torch.empty_like(x)
    _lib.call("hyc_silu_mul_bwd", x.data_ptr(), u.data_ptr(), g.data_ptr(), gx.data_ptr(), gu.data_ptr(), x.numel(),
              _lib.stream_of(x))
    return gx, gu
