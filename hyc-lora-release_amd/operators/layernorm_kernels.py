"""LayerNorm forward / backward on gfx950 (reference API: operators/layernorm_kernels.py:125-198).

`layernorm_forward` returns the reference's 5-tuple; BLOCK_SIZE and num_warps are launch parameters
of the reference's Triton kernels, carried only so that callers can hand them back to
`layernorm_backward` unchanged."""
import torch

from .. import _lib

HAS_APEX = False


def _params(weight, bias):
    if weight.dtype == torch.float32 and bias.dtype == torch.float32:
        return weight.contiguous(), bias.contiguous(), 1
    return weight.to(torch.bfloat16).contiguous(), bias.to(torch.bfloat16).contiguous(), 0


def _check(x):
    if x.dtype != torch.bfloat16:
        raise NotImplementedError("layernorm computes on bfloat16 activations")
    n = x.shape[-1]
    if n * x.element_size() > 65536:
        raise RuntimeError("This layer norm doesn't support feature dim >= 64KB.")
    if n % 8 or n > 8192:
        raise RuntimeError(f"layernorm supports feature dims that are multiples of 8 up to 8192, got {n}")
    return n


def layernorm_forward(x, weight, bias, eps):
    """-> (y, mean fp32 [rows], rstd fp32 [rows], BLOCK_SIZE, num_warps).  Reference :125-147."""
    _lib.require_gpu(x, weight, bias)
    n = _check(x)
    x = x.contiguous()
    rows = x.numel() // n if n else 0
    y = torch.empty_like(x)
    mean = torch.empty((rows,), dtype=torch.float32, device=x.device)
    rstd = torch.empty((rows,), dtype=torch.float32, device=x.device)
    w, b, p32 = _params(weight, bias)
    _lib.call("hyc_layernorm_fwd", x.data_ptr(), w.data_ptr(), b.data_ptr(), p32, y.data_ptr(), mean.data_ptr(),
              rstd.data_ptr(), rows, n, float(eps), _lib.stream_of(x))
    block_size = 1 << max(n - 1, 0).bit_length()
    num_warps = min(max(block_size // 256, 1), 8)
    return y, mean, rstd, block_size, num_warps


def layernorm_backward(dy, x, w, b, m, v, needs_inputs_grad, eps, num_warps, BLOCK_SIZE):
    """-> (dx, None, None); m, v are the mean and rstd of layernorm_forward.  Reference :150-198
    (which computes weight / bias gradient partials and discards them)."""
    if not needs_inputs_grad:
        return None, None, None
    _lib.require_gpu(dy, x, w, m, v)
    n = _check(x)
    if dy.dtype != torch.bfloat16:
        raise NotImplementedError("layernorm computes on bfloat16 activations")
    dy, x = dy.contiguous(), x.contiguous()
    rows = x.numel() // n if n else 0
    dx = torch.empty_like(dy)
    wt, _, p32 = _params(w, w if b is None else b)
    _lib.call("hyc_layernorm_bwd", dy.data_ptr(), x.data_ptr(), wt.data_ptr(), p32,
              m.to(torch.float32).contiguous().data_ptr(), v.to(torch.float32).contiguous().data_ptr(), dx.data_ptr(),
              rows, n, _lib.stream_of(x))
    return dx, None, None
