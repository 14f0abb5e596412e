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


FUSED_ROW_LENGTHS = (512, 1024, 2048, 4096)


def softmax_backward_from_compressed(idx, val, seg_offsets, grad_y, want_map=True):
    """(restored map or None, softmax backward) straight from a compressed attention map
    (`compress_attention_map`) and the upstream gradient `grad_y` of the map's shape [..., n].
    One pass instead of restore + backward when n is 512, 1024, 2048 or 4096; other row lengths
    take the two-kernel route."""
    from .compress_function import restore_attention_map
    _lib.require_gpu(idx, val, seg_offsets, grad_y)
    if grad_y.dtype != torch.bfloat16:
        raise NotImplementedError("softmax backward computes in bfloat16")
    shape = tuple(grad_y.shape)
    n = shape[-1]
    numel = grad_y.numel()
    if n not in FUSED_ROW_LENGTHS or numel % 4096 or numel == 0:
        a = restore_attention_map(idx, val, seg_offsets, shape)
        return (a if want_map else None), softmax_backward(a, grad_y)
    grad_y = grad_y.contiguous()
    idx = idx.reshape(-1).contiguous()
    val = val.reshape(-1).contiguous()
    o = torch.empty(shape, device=grad_y.device, dtype=torch.bfloat16)
    a = torch.empty(shape, device=grad_y.device, dtype=torch.bfloat16) if want_map else None
    _lib.call("hyc_softmax_bwd_restore", _lib.ptr(idx) if idx.numel() else None, _lib.ptr(val) if val.numel() else None,
              seg_offsets.data_ptr(), grad_y.data_ptr(), _lib.ptr(a), o.data_ptr(), numel // n, n,
              _lib.stream_of(grad_y))
    return a, o
