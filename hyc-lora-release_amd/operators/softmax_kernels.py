"""Softmax backward on gfx950 (reference API: operators/softmax_kernels.py:43-57)."""
import torch

from .. import _lib


def softmax_backward(y: torch.Tensor, grad_y: torch.Tensor) -> torch.Tensor:
    """o = (grad_y - sum_row(y * grad_y)) * y over the last dimension of a [b, h, n, n] map
    (any [..., n] shape is accepted), bf16."""
    assert grad_y.shape == y.shape
    _lib.require_gpu(y, grad_y)
    if y.dtype != torch.bfloat16 or grad_y.dtype != torch.bfloat16:
        raise NotImplementedError("softmax_backward computes in bfloat16")
    y = y.contiguous()
    grad_y = grad_y.contiguous()
    o = torch.empty_like(y)
    n = y.shape[-1]
    rows = y.numel() // n if n else 0
    _lib.call("hyc_softmax_bwd", y.data_ptr(), grad_y.data_ptr(), o.data_ptr(), rows, n, _lib.stream_of(y))
    return o
