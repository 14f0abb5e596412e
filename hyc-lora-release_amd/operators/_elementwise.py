"""Shared launcher of the flat element-wise kernels."""
import torch

from .. import _lib


def binary(name: str, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    assert a.shape == b.shape
    _lib.require_gpu(a, b)
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise NotImplementedError(f"{name} computes in bfloat16")
    a = a.contiguous()
    b = b.contiguous()
    o = torch.empty_like(a)
    _lib.call(name, a.data_ptr(), b.data_ptr(), o.data_ptr(), a.numel(), _lib.stream_of(a))
    return o
