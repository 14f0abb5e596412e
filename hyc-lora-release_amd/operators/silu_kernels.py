"""SiLU backward and SiLU*x2 on gfx950 (reference API: operators/silu_kernels.py:48-63,110-125)."""
from ._elementwise import binary


def silu_backward(x, g):
    """g * d/dx[x * sigmoid(x)], bf16 after every operation."""
    return binary("hyc_silu_bwd", x, g)


def silu_hadamard(x, g):
    """(sigmoid(x) * x) * g — SiLU of the first argument times the second."""
    return binary("hyc_silu_mul", x, g)
