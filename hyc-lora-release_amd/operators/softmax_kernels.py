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


def fused_row_length(n: int) -> bool:
    """Row lengths the one-pass kernels take (the kept-entry count inside softmax_forward, restore +
    backward in softmax_backward_from_compressed): multiples of 8 up to 4096.  512, 1024, 2048 and
    4096 tile the 4096-element segments of the compressed map and run the tuned forms."""
    return 8 <= n <= 4096 and n % 8 == 0


def softmax_backward_from_compressed(idx, val, seg_offsets, grad_y, want_map=True, out_scale=1.0):
    """(restored map or None, softmax backward) straight from a compressed attention map
    (`compress_attention_map`) and the upstream gradient `grad_y` of the map's shape [..., n].
    One pass instead of restore + backward when n is a multiple of 8 up to 4096; other row lengths
    take the two-kernel route.  `out_scale` multiplies the bf16 gradient (and rounds again), which
    is what the layers' `grad_s = grad_s / math.sqrt(head_dim)` does on the device."""
    from .compress_function import check_map_lists, restore_attention_map
    shape = tuple(grad_y.shape)
    n = shape[-1]
    numel = grad_y.numel()
    check_map_lists(idx, val, seg_offsets, numel)
    _lib.require_gpu(idx, val, seg_offsets, grad_y)
    if grad_y.dtype != torch.bfloat16:
        raise NotImplementedError("softmax backward computes in bfloat16")
    if not fused_row_length(n) or numel == 0:
        a = restore_attention_map(idx, val, seg_offsets, shape)
        o = softmax_backward(a, grad_y)
        return (a if want_map else None), (o if out_scale == 1.0 else o * out_scale)
    grad_y = grad_y.contiguous()
    idx = idx.reshape(-1).contiguous()
    val = val.reshape(-1).contiguous()
    o = torch.empty(shape, device=grad_y.device, dtype=torch.bfloat16)
    a = torch.empty(shape, device=grad_y.device, dtype=torch.bfloat16) if want_map else None
    _lib.call("hyc_softmax_bwd_restore", _lib.ptr(idx) if idx.numel() else None, _lib.ptr(val) if val.numel() else None,
              seg_offsets.data_ptr(), grad_y.data_ptr(), _lib.ptr(a), o.data_ptr(), numel // n, n,
              float(out_scale), _lib.stream_of(grad_y))
    return a, o


def softmax_forward(s, scale, mask=None, threshold=None, inplace=False):
    """bf16 softmax over the last dimension of  bf16(bf16(s * scale) + mask)  in one pass: what the
    reference computes with three torch kernels (q @ k^T / sqrt(d), + attention_mask, softmax;
    fused_llama_layer_intra_inter_full_fuse.py:159-167).

    s: bf16 [..., rows, n] scores straight from the matmul; scale: Python float (1 / sqrt(head_dim));
    mask: None or an additive bf16 mask broadcastable as [B or 1, 1, S, n] against s [B, H, S, n];
    inplace: overwrite s.  With `threshold` (0-d tensor, the frozen keep-threshold) the per-segment
    offsets of the compaction are produced in the same pass and returned as the second value (None
    when the row length does not allow it); pass them to compress_attention_map."""
    _lib.require_gpu(s)
    if s.dtype != torch.bfloat16:
        raise NotImplementedError("softmax_forward computes on bfloat16 scores")
    n = s.shape[-1]
    if n % 8 or n > 8192:
        raise ValueError(f"row length {n}: must be a multiple of 8, at most 8192")
    if not s.is_contiguous() or s.data_ptr() % 16:
        s, inplace = s.contiguous(), True                     # a private copy may be overwritten
    out = s if inplace else torch.empty_like(s)
    rows = s.numel() // n if n else 0
    mptr, mask_rows, rows_per_batch, msb, msr = None, 1, 1, 0, 0
    if mask is not None:
        _lib.require_gpu(mask)
        if s.dim() != 4 or mask.dim() != 4 or mask.shape[1] != 1 or mask.shape[-1] != n or \
                mask.shape[2] != s.shape[2] or mask.shape[0] not in (1, s.shape[0]):
            raise ValueError(f"mask {tuple(mask.shape)} is not [B or 1, 1, S, n] for scores {tuple(s.shape)}")
        if mask.dtype != torch.bfloat16:
            mask = mask.to(torch.bfloat16)
        if mask.stride(-1) != 1 or mask.stride(2) % 8 or mask.stride(0) % 8 or mask.data_ptr() % 16:
            mask = mask.contiguous()
        mptr, mask_rows, rows_per_batch = mask.data_ptr(), s.shape[2], s.shape[1] * s.shape[2]
        msb, msr = (mask.stride(0) if mask.shape[0] > 1 else 0), mask.stride(2)
    counts = offsets = thr = None
    if threshold is not None and fused_row_length(n) and s.numel():
        from .compress_function import _threshold_tensor
        thr = _threshold_tensor(threshold, s.device)
        nseg = -(-s.numel() // 4096)
        counts = torch.empty(nseg, device=s.device, dtype=torch.int32)
        offsets = torch.empty(nseg + 1, device=s.device, dtype=torch.int64)
    _lib.call("hyc_softmax_fwd", s.data_ptr(), mptr, out.data_ptr(), rows, n, float(scale), mask_rows, rows_per_batch,
              msb, msr, _lib.ptr(thr), _lib.ptr(counts), _lib.ptr(offsets), _lib.stream_of(s))
    if threshold is not None:
        return out, offsets
    return out
