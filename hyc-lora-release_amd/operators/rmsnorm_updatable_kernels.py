"""RMSNorm with a weight gradient (reference API: operators/rmsnorm_updatable_kernels.py:140-220)."""
from .rmsnorm_kernels import _backward, rmsnorm_forward  # noqa: F401


def rmsnorm_backward(dy, x, w, m, v, eps, num_warps, BLOCK_SIZE):
    """-> (dx, dw)."""
    return _backward(dy, x, w, v, want_dw=True)
