"""RMSNorm forward / backward on gfx950 (reference API: operators/rmsnorm_kernels.py:116-185).

`rmsnorm_forward` returns the reference's 5-tuple; BLOCK_SIZE and num_warps are launch
parameters of the reference's Triton kernels and are carried only so that callers can hand
them back to `rmsnorm_backward` unchanged.  `mean` is an uninitialised placeholder there as
well."""
import torch

from .. import _lib

MAX_FUSED_BYTES = 65536


def _weight(weight: torch.Tensor):
    if weight.dtype == torch.float32:
        return weight.contiguous(), 1
    if weight.dtype == torch.bfloat16:
        return weight.contiguous(), 0
    return weight.to(torch.bfloat16).contiguous(), 0


def rmsnorm_forward(x, weight, eps):
    _lib.require_gpu(x, weight)
    if x.dtype != torch.bfloat16:
        raise NotImplementedError("rmsnorm_forward computes on bfloat16 activations")
    x = x.contiguous()
    n = x.shape[-1]
    if n * x.element_size() > MAX_FUSED_BYTES:
        raise RuntimeError("This layer norm doesn't support feature dim >= 64KB.")
    if n % 8:
        raise ValueError(f"feature dimension must be a multiple of 8, got {n}")
    rows = x.numel() // n if n else 0
    y = torch.empty_like(x)
    mean = torch.empty((rows,), dtype=torch.float32, device=x.device)
    rstd = torch.empty((rows,), dtype=torch.float32, device=x.device)
    w, w32 = _weight(weight)
    _lib.call("hyc_rmsnorm_fwd", x.data_ptr(), w.data_ptr(), w32, y.data_ptr(), rstd.data_ptr(), rows, n,
              float(eps), _lib.stream_of(x))
    block_size = 1 << max(n - 1, 0).bit_length()
    num_warps = min(max(block_size // 256, 1), 8)
    return y, mean, rstd, block_size, num_warps


def _backward(dy, x, w, rstd, want_dw):
    _lib.require_gpu(dy, x, w, rstd)
    if dy.dtype != torch.bfloat16 or x.dtype != torch.bfloat16:
        raise NotImplementedError("rmsnorm_backward computes on bfloat16 activations")
    n = x.shape[-1]
    if n > 8192 or n % 8:
        raise RuntimeError(f"rmsnorm_backward supports feature dims that are multiples of 8 up to 8192, got {n}")
    dy = dy.contiguous()
    x = x.contiguous()
    rows = x.numel() // n if n else 0
    dx = torch.empty_like(dy)
    wt, w32 = _weight(w)
    dw = ws = None
    ws_bytes = 0
    if want_dw:
        dw = torch.empty((n,), dtype=wt.dtype, device=x.device)
        ws_bytes = _lib.lib().hyc_rmsnorm_bwd_workspace(rows, n)
        ws = torch.empty((max(ws_bytes, 4) // 4,), dtype=torch.float32, device=x.device)
    _lib.call("hyc_rmsnorm_bwd", dy.data_ptr(), x.data_ptr(), wt.data_ptr(), w32,
              rstd.to(torch.float32).contiguous().data_ptr(), dx.data_ptr(), _lib.ptr(dw), _lib.ptr(ws), ws_bytes,
              rows, n, _lib.stream_of(x))
    if want_dw and dw.dtype != w.dtype:
        dw = dw.to(w.dtype)
    return dx, dw


def rmsnorm_backward(dy, x, w, m, v, needs_inputs_grad, eps, num_warps, BLOCK_SIZE):
    """-> (dx, None); `v` is the rstd returned by rmsnorm_forward.  Reference :149-185."""
    if not needs_inputs_grad:
        return None, None
    dx, _ = _backward(dy, x, w, v, want_dw=False)
    return dx, None
