"""RMSNorm forward / backward on gfx950 (reference API: operators/rmsnorm_kernels.py:116-185).

`rmsnorm_forward` returns the reference's 5-tuple; BLOCK_SIZE and num_warps are launch
parameters of the reference's Triton kernels and are carried only so that callers can hand
them back to `rmsnorm_backward` unchanged.  `mean` is an uninitialised placeholder there as
well."""
import weakref

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


def _backward(dy, x, w, rstd, want_dw, residual=None):
    """-> (dx, dw or None).  With `residual` (bf16, dy's shape) dx is bf16(dx + residual): the
    gradient of the residual connection added in the same pass, same bits as adding it afterwards."""
    _lib.require_gpu(dy, x, w, rstd, residual)
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
    rstd = rstd.to(torch.float32).contiguous()
    if residual is None:
        _lib.call("hyc_rmsnorm_bwd", dy.data_ptr(), x.data_ptr(), wt.data_ptr(), w32, rstd.data_ptr(), dx.data_ptr(),
                  _lib.ptr(dw), _lib.ptr(ws), ws_bytes, rows, n, _lib.stream_of(x))
    else:
        if residual.shape != dy.shape or residual.dtype != torch.bfloat16:
            raise ValueError(f"residual must be bfloat16 of shape {tuple(dy.shape)}")
        residual = residual.contiguous()
        _lib.call("hyc_rmsnorm_bwd_add", dy.data_ptr(), x.data_ptr(), wt.data_ptr(), w32, rstd.data_ptr(),
                  residual.data_ptr(), dx.data_ptr(), _lib.ptr(dw), _lib.ptr(ws), ws_bytes, rows, n, _lib.stream_of(x))
    if want_dw and dw.dtype != w.dtype:
        dw = dw.to(w.dtype)
    return dx, dw


def rmsnorm_backward_into(dy, x, w, rstd, dx, dw):
    """rmsnorm_backward with the weight gradient, written into the caller's `dx` (bf16, dy's shape) and
    `dw` ([N], w's dtype), through the entry point that allocates nothing: its fp32 partial rows live
    in a fixed device array of the library (16 MiB per GPU), not in a workspace.  For callers that
    must not allocate device memory (graph capture, serving loops).  All tensors must already be
    contiguous, bf16 activations, fp32 rstd; calls that overlap in time on one GPU race on that array.
    Same bits as rmsnorm_updatable_kernels.rmsnorm_backward."""
    _lib.require_gpu(dy, x, w, rstd, dx, dw)
    n = x.shape[-1]
    rows = x.numel() // n if n else 0
    ok = (dy.dtype == x.dtype == dx.dtype == torch.bfloat16 and dy.shape == x.shape == dx.shape
          and rstd.dtype == torch.float32 and rstd.numel() == rows and w.numel() == n and dw.shape == w.shape
          and dw.dtype == w.dtype and w.dtype in (torch.bfloat16, torch.float32)
          and all(t.is_contiguous() for t in (dy, x, w, rstd, dx, dw)))
    if not ok:
        raise ValueError("rmsnorm_backward_into takes contiguous bf16 dy / x / dx of one shape, fp32 rstd [rows], "
                         "and w / dw [N] of one dtype (bf16 or fp32); nothing is converted or copied")
    _lib.call("hyc_rmsnorm_bwd_static", dy.data_ptr(), x.data_ptr(), w.data_ptr(), int(w.dtype == torch.float32),
              rstd.data_ptr(), dx.data_ptr(), dw.data_ptr(), rows, n, _lib.stream_of(x))
    return dx, dw


def backward_from_codes_supported(dy, n, want_dw):
    """Whether rmsnorm_backward_from_codes takes this case (whole 512-column slabs, an even number of
    rows, bf16 gradient, no weight gradient)."""
    return (not want_dw and dy.is_cuda and dy.dtype == torch.bfloat16 and n % 512 == 0 and 0 < n <= 8192
            and dy.numel() > 0 and (dy.numel() // n) % 2 == 0)


def rmsnorm_backward_from_codes(dy, q_x, scale_x, x_outlier, outlier_idx, q_bit, w, rstd, residual=None, table=None):
    """dx of rmsnorm_backward with the norm's input given as its channel-base compressed copy
    (q_x, scale_x, x_outlier, outlier_idx) - the same bits as
    outlier_addition_fuse_decompression_dequantization followed by rmsnorm_backward
    (fused_llama_layer_intra_inter_full_fuse.py:386-393), with `residual` added like there."""
    _lib.require_gpu(dy, q_x, scale_x, w, rstd, residual)
    n = dy.shape[-1]
    if not backward_from_codes_supported(dy, n, False):
        raise NotImplementedError("rmsnorm_backward_from_codes: bfloat16 gradient, N a multiple of 512 up to 8192, even row count")
    dy = dy.contiguous()
    rows = dy.numel() // n
    k = 0 if outlier_idx is None else int(outlier_idx.numel())
    if k and table is None:
        table = outlier_table(outlier_idx, n, cached=True)
    _check_table(table, n, k)
    if q_x.dtype != torch.uint8 or q_x.numel() != rows * n * q_bit // 8:
        raise ValueError("q_x does not hold the packed codes of a tensor of dy's shape")
    q_x = q_x.contiguous()
    sx = scale_x.to(torch.bfloat16).reshape(-1).contiguous()
    xo = None
    if k:
        xo = x_outlier.to(torch.bfloat16).contiguous()
        if xo.numel() != rows * k:
            raise ValueError("x_outlier does not match the outlier list")
    wt, w32 = _weight(w)
    rstd = rstd.to(torch.float32).contiguous()
    if sx.numel() != n or wt.numel() != n or rstd.numel() != rows:
        raise ValueError(f"steps and weight must have {n} entries and rstd {rows}, got {sx.numel()}, {wt.numel()}, {rstd.numel()}")
    if residual is not None:
        if residual.shape != dy.shape or residual.dtype != torch.bfloat16:
            raise ValueError(f"residual must be bfloat16 of shape {tuple(dy.shape)}")
        residual = residual.contiguous()
    dx = torch.empty_like(dy)
    _lib.call("hyc_rmsnorm_bwd_codes", dy.data_ptr(), q_x.data_ptr(), sx.data_ptr(), _lib.ptr(table) if k else None, k,
              _lib.ptr(xo), q_bit, wt.data_ptr(), w32, rstd.data_ptr(), _lib.ptr(residual), dx.data_ptr(), rows, n,
              _lib.stream_of(dy))
    return dx


def rmsnorm_backward(dy, x, w, m, v, needs_inputs_grad, eps, num_warps, BLOCK_SIZE, residual=None):
    """-> (dx, None); `v` is the rstd returned by rmsnorm_forward.  Reference :149-185.
    `residual` (not in the reference's signature): a tensor added to dx in the same pass."""
    if not needs_inputs_grad:
        return None, None
    dx, _ = _backward(dy, x, w, v, want_dw=False, residual=residual)
    return dx, None


def _check_table(table, n, k):
    """A table handed in by the caller is read with one entry per channel."""
    if k and (table.dtype != torch.int16 or table.numel() != n or not table.is_contiguous()):
        raise ValueError(f"outlier table must be a contiguous int16 [{n}] (outlier_table(idx, {n})), got "
                         f"{table.dtype} {tuple(table.shape)}")


_TABLES = {}          # id(channel-list tensor) -> (weak reference to it, its version, n, table)


def outlier_table(outlier_idx, n, cached=False):
    """uint16 [n] lookup for the fused norm kernels: 1 + list position for an outlier channel, else 0.
    cached=True keeps the table with the channel-list tensor (weakly, and only while the tensor is
    not modified in place): a frozen list is the same tensor object step after step."""
    _lib.require_gpu(outlier_idx)
    if cached:
        key = id(outlier_idx)
        hit = _TABLES.get(key)
        if hit is not None and hit[0]() is outlier_idx and hit[1] == outlier_idx._version and hit[2] == n:
            return hit[3]
        table = outlier_table(outlier_idx, n)
        _TABLES[key] = (weakref.ref(outlier_idx, lambda _r, k=key: _TABLES.pop(k, None)), outlier_idx._version, n, table)
        return table
    idx = outlier_idx.reshape(-1).to(torch.int64).contiguous()
    table = torch.empty((n,), dtype=torch.int16, device=idx.device)
    _lib.call("hyc_outlier_table", idx.data_ptr() if idx.numel() else None, idx.numel(), n, table.data_ptr(),
              _lib.stream_of(idx))
    return table


MAX_LORA_BLOCKS = 4          # 16-row blocks of adapter weights the fused norm kernel contracts with


def _adapter_weight(a):
    """lora_A as the kernel reads it: bf16 [R, N] row-major.  The layers pass the `[N, R]` view
    `lora_A.weight.T`, whose transpose is that weight as it lies in memory."""
    if a.dim() != 2:
        raise ValueError(f"a LoRA-A operand must be a matrix, got shape {tuple(a.shape)}")
    w = a.t()
    if w.dtype != torch.bfloat16:
        w = w.to(torch.bfloat16)
    if not w.is_contiguous():
        w = w.contiguous()
    if w.data_ptr() % 16:
        w = w.clone()
    return w


def lora_a_supported(x, weight, lora_a):
    """Whether rmsnorm_forward_compress(..., lora_a=lora_a) takes this case: bf16 [B, M, N] activations
    whose rows are whole 512-column slabs (N <= 8192), an even row count, a bf16 norm weight and
    adapters `[N, R]` whose ranks, rounded up to multiples of 16, add up to at most 64."""
    if not (x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 3 and weight.dtype == torch.bfloat16):
        return False
    n = x.shape[-1]
    if n % 512 or n > 8192 or x.numel() == 0 or (x.numel() // n) % 2:
        return False
    if not lora_a or any(a.dim() != 2 or a.shape[0] != n or not 1 <= a.shape[1] <= 64 or a.dtype != torch.bfloat16
                         for a in lora_a):
        return False
    return sum(-(-a.shape[1] // 16) for a in lora_a) <= MAX_LORA_BLOCKS


def rmsnorm_forward_compress(x, weight, eps, q_bit, scale_y=None, scale_x=None, outlier_idx=None, table=None, lora_a=None):
    """RMSNorm forward that also produces, from the same read of x, the packed codes of the
    normalised output (steps `scale_y`) and the channel-base compressed input (steps `scale_x`,
    outlier channels `outlier_idx`): what rmsnorm_forward + compression_pack_quant_base(y) +
    compression_pack_channel_base(x) produce with frozen statistics, bit for bit
    (fused_llama_layer_intra_inter_full_fuse.py:97-126).

    -> (y, rstd, q_y or None, q_x or None, x_outlier or None).

    lora_a: a list of LoRA-A operands `[N, R]` (the `lora_A.weight.T` views the layers pass around) of
    the projections that consume y.  Then a sixth result is returned, the list of `y @ a` as
    [B, M, R] bf16 - lora_forward's `x @ w_lora_a` (models/utils/compute_utils.py:22) for each of them,
    formed while y is still on the chip instead of by one library GEMM each over y in memory
    (see lora_a_supported for the shapes this takes)."""
    _lib.require_gpu(x, weight)
    if x.dtype != torch.bfloat16 or x.dim() != 3:
        raise NotImplementedError("rmsnorm_forward_compress takes bfloat16 [batch, seq, hidden] activations")
    if q_bit not in (2, 4, 8):
        raise ValueError(f"q_bit must be 2, 4 or 8, got {q_bit}")
    x = x.contiguous()
    b, m, n = x.shape
    if n % 32 or n > 8192:
        raise ValueError(f"hidden size {n}: must be a multiple of 32, at most 8192")
    rows = b * m
    dev = x.device
    y = torch.empty_like(x)
    rstd = torch.empty((rows,), dtype=torch.float32, device=dev)
    w, w32 = _weight(weight)

    def steps(sc):
        sc = sc.reshape(-1).to(torch.bfloat16).contiguous()
        if sc.numel() != n:
            raise ValueError(f"{sc.numel()} steps for {n} channels")
        return sc
    q_y = q_x = x_out = None
    k = 0
    if scale_y is not None:
        scale_y = steps(scale_y)
        q_y = torch.empty((b, m, n * q_bit // 8), dtype=torch.uint8, device=dev)
    if scale_x is not None:
        scale_x = steps(scale_x)
        q_x = torch.empty((b, m, n * q_bit // 8), dtype=torch.uint8, device=dev)
        k = 0 if outlier_idx is None else outlier_idx.numel()
        x_out = torch.empty((b, m, k), dtype=torch.bfloat16, device=dev)
        if k and table is None:
            table = outlier_table(outlier_idx, n, cached=True)
        _check_table(table, n, k)
    if lora_a is not None:
        import ctypes
        if not lora_a_supported(x, weight, lora_a):
            raise NotImplementedError("rmsnorm_forward_compress(lora_a=...): see lora_a_supported for the shapes it takes")
        ws = [_adapter_weight(a) for a in lora_a]
        outs = [torch.empty((b, m, a.shape[1]), dtype=torch.bfloat16, device=dev) for a in lora_a]
        g = len(ws)
        _lib.call("hyc_rmsnorm_fwd_compress_lora", x.data_ptr(), w.data_ptr(), y.data_ptr(), rstd.data_ptr(), rows, n,
                  float(eps), q_bit, _lib.ptr(scale_y), _lib.ptr(q_y), _lib.ptr(scale_x), _lib.ptr(q_x),
                  _lib.ptr(table) if k else None, k, _lib.ptr(x_out) if k else None, g,
                  (ctypes.c_void_p * g)(*[t.data_ptr() for t in ws]), (ctypes.c_int64 * g)(*[t.shape[0] for t in ws]),
                  (ctypes.c_void_p * g)(*[t.data_ptr() for t in outs]), _lib.stream_of(x))
        return y, rstd, q_y, q_x, x_out, outs
    _lib.call("hyc_rmsnorm_fwd_compress", x.data_ptr(), w.data_ptr(), w32, y.data_ptr(), rstd.data_ptr(), rows, n,
              float(eps), q_bit, _lib.ptr(scale_y), _lib.ptr(q_y), _lib.ptr(scale_x), _lib.ptr(q_x),
              _lib.ptr(table) if k else None, k, _lib.ptr(x_out) if k else None, _lib.stream_of(x))
    return y, rstd, q_y, q_x, x_out
