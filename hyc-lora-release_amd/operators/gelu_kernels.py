"""tanh-GELU backward on gfx950 (reference API: operators/gelu_kernels.py:61-76)."""
from ._elementwise import binary


def gelu_backward(x, g):
    return binary("hyc_gelu_bwd", x, g)
