"""Compress / decompress operators with the reference's Python API
(operators/compress_function.py), running on hand-written gfx950 kernels.

Function names, argument order and return values follow the reference so that the fused
decoder layers can call either implementation.  Differences, all deliberate:
  * `outlier_subtraction_fuse_compression_quantization` does not modify its input
    unless `zero_input=True` is passed (the reference zeroes the outlier columns of `x`
    in place, which is why its callers hand it a clone); `zero_input=True` needs a bf16 tensor
    the kernels can address in place and raises otherwise;
  * 4-D `[B, H, S, D]` inputs are read in place through their strides instead of being
    transposed into a temporary `[B, S, H*D]` copy;
  * outlier channels are chosen with a defined tie rule (norm descending, then channel
    index ascending) where `torch.topk` leaves the order open.
"""
from __future__ import annotations

import torch

from .. import _lib

BF16 = torch.bfloat16


# ---------------------------------------------------------------------------------------
# shape helpers (reference: operators/compress_function.py:6-13)
# ---------------------------------------------------------------------------------------
def hidden_to_head_shape(x: torch.Tensor, num_heads: int):
    bsz, seq_len, hidden = x.shape
    return x.reshape(bsz, seq_len, num_heads, hidden // num_heads).transpose(1, 2)


def head_to_hidden_shape(x: torch.Tensor):
    bsz, _, seq_len, _ = x.shape
    return x.transpose(1, 2).reshape(bsz, seq_len, -1)


def update_dict(old_dict, new_dict, iteration):
    """Running mean of calibration statistics; the outlier channel list is replaced
    (reference: operators/compress_function.py:15-27)."""
    for name in old_dict:
        fresh = new_dict[name]
        if name == 'outlier_channel_index' or old_dict[name] is None:
            old_dict[name] = fresh
        else:
            old_dict[name] = (iteration * old_dict[name] + fresh) / (iteration + 1)
    return old_dict


# ---------------------------------------------------------------------------------------
# addressing of the activation tensor handed to the kernels
# ---------------------------------------------------------------------------------------
class _Addr:
    """Logical [B, M, N] view of a 3-D or 4-D ([B, H, S, D]) bf16 tensor as the kernels
    address it: element (b, m, c) at b*sb + m*sm + (c // hd)*sh + c % hd."""
    __slots__ = ("t", "B", "M", "N", "sb", "sm", "hd", "sh")

    def __init__(self, x: torch.Tensor):
        if x.dim() == 4:
            ok = (x.stride(3) == 1 and x.shape[3] % 8 == 0 and x.data_ptr() % 16 == 0
                  and all(s % 8 == 0 for s in x.stride()[:3]))
            if not ok:
                x = x.contiguous()
            B, H, S, D = x.shape
            self.t, self.B, self.M, self.N = x, B, S, H * D
            self.sb, self.sm, self.hd, self.sh = x.stride(0), x.stride(2), D, x.stride(1)
        elif x.dim() == 3:
            ok = (x.stride(2) == 1 and x.data_ptr() % 16 == 0 and x.stride(0) % 8 == 0 and x.stride(1) % 8 == 0)
            if not ok:
                x = x.contiguous()
            B, M, N = x.shape
            self.t, self.B, self.M, self.N = x, B, M, N
            self.sb, self.sm, self.hd, self.sh = x.stride(0), x.stride(1), N, 0
        else:
            raise ValueError(f"expected a 3-D or 4-D activation tensor, got shape {tuple(x.shape)}")


def _vec(t: torch.Tensor, n: int, name: str) -> torch.Tensor:
    """A per-channel vector ([1, N], [N], ...) as contiguous, aligned bf16 [N]."""
    t = _lib.bf16_vector(t)
    if t.numel() != n:
        raise ValueError(f"{name} must have {n} elements (one per channel), got {t.numel()}")
    if not t.is_contiguous() or t.data_ptr() % 16:
        t = t.clone(memory_format=torch.contiguous_format)
    return t


def _require_per_channel(q_method: str) -> None:
    if q_method == 'per-channel':
        return
    if q_method == 'per-tensor':
        # The reference computes a 0-d step for 'per-tensor' and then fails inside its own
        # kernel wrapper (s.stride(1) on a 0-d tensor); no layer ever asks for it.
        raise NotImplementedError("q_method='per-tensor' is not supported; the layers use 'per-channel'")
    raise ValueError(f"Unsupport Quantize Method: {q_method!r}")


def _batch0_stats(x: torch.Tensor):
    """(stats, strips, N): per-strip min / max / sum of squares per channel over batch element 0, fp32
    [strips*3 + 1, N] as hyc_channel_select takes it."""
    _lib.require_gpu(x)
    if x.dtype != BF16:
        x = x.to(BF16)
    a = _Addr(x)
    if a.N % 32:
        raise ValueError(f"channel count must be a multiple of 32, got {a.N}")
    if a.B == 0:
        raise ValueError("statistics need at least one batch element")
    strips = int(_lib.lib().hyc_channel_stats_strips(a.M, a.N))
    stats = torch.empty((strips * 3 + 1, a.N), device=x.device, dtype=torch.float32)
    _lib.call("hyc_channel_stats", a.t.data_ptr(), a.M, a.N, a.sm, a.hd, a.sh, stats.data_ptr(),
              stats.numel() * 4, _lib.stream_of(x))
    return stats, strips, a.N


# ---------------------------------------------------------------------------------------
# statistics (reference: operators/compress_function.py:30-105)
# ---------------------------------------------------------------------------------------
def _kth_value(x: torch.Tensor, kth: int) -> torch.Tensor:
    """Exact kth-smallest (1-based) value of a bf16 tensor as a 0-d fp32 tensor."""
    _lib.require_gpu(x)
    n = x.numel()
    if not 1 <= kth <= n:
        raise RuntimeError(f"kthvalue(): selected number k out of range: k={kth}, numel={n}")
    flat = x.reshape(-1)
    if not flat.is_contiguous() or flat.data_ptr() % 16:
        flat = flat.clone(memory_format=torch.contiguous_format)
    hist = torch.empty(65536, device=x.device, dtype=torch.int32)
    thr = torch.empty((), device=x.device, dtype=torch.float32)
    st = _lib.stream_of(x)
    _lib.call("hyc_hist16", flat.data_ptr(), n, hist.data_ptr(), st)
    _lib.call("hyc_hist_select", hist.data_ptr(), kth, thr.data_ptr(), st)
    return thr


def get_statistics_softmax(x: torch.Tensor, outlier_ratio: float):
    """Keep-threshold of an attention map: the int(numel*(1-ratio))-th smallest value,
    0-d fp32.  Reference :30-32 (torch.kthvalue on an fp32 copy)."""
    if x.dtype != BF16:
        x = x.to(BF16)
    return _kth_value(x, int(x.numel() * (1 - outlier_ratio)))


def get_statistics_outlier(x: torch.Tensor, outlier_ratio: float):
    """Same order statistic on |x|.  Reference :34-36 (not called by any layer)."""
    return _kth_value(x.to(BF16).abs(), int(x.numel() * (1 - outlier_ratio)))


def get_statistics_only_quant(x: torch.Tensor, q_bit: int = 8, q_method: str = 'per-tensor'):
    """Per-channel step bf16 [1, N] from batch element 0.  Reference :45-59."""
    _require_per_channel(q_method)
    _check_bits(q_bit)
    stats, strips, n = _batch0_stats(x)
    scale = torch.empty((1, n), device=x.device, dtype=BF16)
    _lib.call("hyc_channel_select", stats.data_ptr(), strips, n, 0, q_bit, 0, None, scale.data_ptr(), None,
              _lib.stream_of(x))
    return scale


def get_statistics_only_quant_zero_point(x: torch.Tensor, q_bit: int = 8, q_method: str = 'per-tensor'):
    """(step bf16 [1, N], zero point int8 [1, N]).  Reference :62-77."""
    _require_per_channel(q_method)
    _check_bits(q_bit)
    stats, strips, n = _batch0_stats(x)
    scale = torch.empty((1, n), device=x.device, dtype=BF16)
    zp = torch.empty((1, n), device=x.device, dtype=torch.int8)
    _lib.call("hyc_channel_select", stats.data_ptr(), strips, n, 0, q_bit, 0, None, scale.data_ptr(), zp.data_ptr(),
              _lib.stream_of(x))
    return scale, zp


def get_statistics_channel_base(x: torch.Tensor, outlier_ratio: float, q_bit: int = 8, q_method: str = 'per-tensor'):
    """(outlier channel indices int64 [k], step bf16 [1, N]) with k = int(N * ratio); the
    step is that of the tensor with the outlier channels zeroed.  Reference :80-105.
    No clone of x is made: the statistics of the zeroed tensor follow from those of x."""
    _require_per_channel(q_method)
    _check_bits(q_bit)
    stats, strips, n = _batch0_stats(x)
    k = int(n * outlier_ratio)
    idx = torch.empty((k,), device=x.device, dtype=torch.int64)
    scale = torch.empty((1, n), device=x.device, dtype=BF16)
    _lib.call("hyc_channel_select", stats.data_ptr(), strips, n, k, q_bit, 1, idx.data_ptr() if k else None,
              scale.data_ptr(), None, _lib.stream_of(x))
    return idx, scale


def validate_channel_list(channel: torch.Tensor, n: int) -> None:
    """An outlier channel list must name distinct channels inside [0, n): the kernels skip an index
    outside the tensor and keep one position of a repeated one, where `x[:, :, channel]` of the
    reference (:125) raises / gathers.  Reads the list back to the host, so it is meant for the
    places where a list enters from outside (a checkpoint), not for the per-step path."""
    if channel is None or channel.numel() == 0:
        return
    c = channel.detach().reshape(-1).to("cpu", torch.int64)
    if int(c.min()) < 0 or int(c.max()) >= n:
        raise ValueError(f"outlier channel index out of range for {n} channels: "
                         f"[{int(c.min())}, {int(c.max())}]")
    if torch.unique(c).numel() != c.numel():
        raise ValueError("outlier channel list names a channel twice")


def _check_bits(quantize_bit: int) -> int:
    if quantize_bit not in (2, 4, 8):
        raise ValueError(f"quantize_bit must be 2, 4 or 8, got {quantize_bit}")
    return 8 // quantize_bit


def _quantize(x, s, z, channel, quantize_bit, dtype, zero_input=False):
    if dtype != BF16:
        raise NotImplementedError("the gfx950 kernels compute in bfloat16 only")
    epp = _check_bits(quantize_bit)
    _lib.require_gpu(x, s, z, channel)
    if x.dtype != BF16:
        x = x.to(BF16)
    a = _Addr(x)
    if zero_input and a.t is not x:
        # the kernel would zero a private bf16 / contiguous copy and leave the caller's tensor as it was
        raise ValueError("zero_input=True needs a bfloat16 activation whose channel dimension is contiguous "
                         "and 16-byte aligned: it is zeroed in place")
    if a.N % 32:
        raise ValueError(f"channel count must be a multiple of 32, got {a.N}")
    s = _vec(s, a.N, "scale")
    z = None if z is None else _vec(z, a.N, "zero point")
    q = torch.empty((a.B, a.M, a.N // epp), device=x.device, dtype=torch.uint8)
    k = 0
    x_outlier = None
    if channel is not None:
        channel = channel.to(torch.int64).contiguous()
        k = channel.numel()
        # zero-filled (a few hundred KB): a list position the kernel finds no column for - an index
        # outside the tensor, the earlier copies of a repeated one - then reads as zeros, not as
        # whatever the allocator handed out
        x_outlier = torch.zeros((a.B, a.M, k), device=x.device, dtype=BF16)
    _lib.call("hyc_quant_pack", a.t.data_ptr(), s.data_ptr(), _lib.ptr(z), q.data_ptr(),
              _lib.ptr(channel) if k else None, k, _lib.ptr(x_outlier) if k else None, int(bool(zero_input)),
              a.B, a.M, a.N, a.sb, a.sm, a.hd, a.sh, quantize_bit, _lib.stream_of(x))
    return x_outlier, q


def _dequantize(q, s, z, x_outlier, channel, quantize_bit, is_head, num_heads, dtype):
    if dtype != BF16:
        raise NotImplementedError("the gfx950 kernels compute in bfloat16 only")
    epp = _check_bits(quantize_bit)
    _lib.require_gpu(q, s, z, x_outlier, channel)
    B, M, nbytes = q.shape
    N = s.shape[-1]
    if nbytes * epp != N:
        raise ValueError(f"packed width {nbytes} does not match {N} channels at {quantize_bit} bits")
    if N % 32:
        raise ValueError(f"channel count must be a multiple of 32, got {N}")
    if q.dtype != torch.uint8:
        raise ValueError("packed codes must be uint8")
    q = q.contiguous()
    s = _vec(s, N, "scale")
    z = None if z is None else _vec(z, N, "zero point")
    x = torch.empty((B, M, N), device=q.device, dtype=BF16)
    k = 0
    if channel is not None:
        channel = channel.to(torch.int64).contiguous()
        k = channel.numel()
        x_outlier = x_outlier.to(BF16).contiguous()
        if tuple(x_outlier.shape) != (B, M, k):
            raise ValueError(f"x_outlier must have shape {(B, M, k)}, got {tuple(x_outlier.shape)}")
    _lib.call("hyc_unpack_dequant", q.data_ptr(), s.data_ptr(), _lib.ptr(z), x.data_ptr(),
              _lib.ptr(channel) if k else None, k, _lib.ptr(x_outlier) if k else None,
              B, M, N, M * N, N, N, 0, quantize_bit, _lib.stream_of(q))
    if is_head:
        x = hidden_to_head_shape(x, num_heads=num_heads)
    return x


# ---------------------------------------------------------------------------------------
# compress / decompress interface (reference: operators/compress_function.py:111-306)
# ---------------------------------------------------------------------------------------
def outlier_subtraction_fuse_compression_quantization(x, s, channel, quantize_bit=8, dtype=BF16, zero_input=False):
    """-> (x_outlier [B,M,k] bf16, q [B,M,N*bits/8] uint8).  Reference :111-143."""
    return _quantize(x, s, None, channel, quantize_bit, dtype, zero_input)


def outlier_addition_fuse_decompression_dequantization(q, s, x_outlier, channel, quantize_bit=8, is_head=False,
                                                       num_heads=1, dtype=BF16):
    """Inverse of the above.  Reference :147-174."""
    return _dequantize(q, s, None, x_outlier, channel, quantize_bit, is_head, num_heads, dtype)


def compression_quantization(x, s, quantize_bit=8, dtype=BF16):
    """Reference :178-210."""
    return _quantize(x, s, None, None, quantize_bit, dtype)[1]


def decompression_dequantization(q, s, quantize_bit=8, is_head=False, num_heads=1, dtype=BF16):
    """Reference :214-241."""
    return _dequantize(q, s, None, None, None, quantize_bit, is_head, num_heads, dtype)


def compression_quantization_with_zero_point(x, s, z, quantize_bit=8, dtype=BF16):
    """Reference :245-274."""
    return _quantize(x, s, z, None, quantize_bit, dtype)[1]


def decompression_dequantization_with_zero_point(q, s, z, quantize_bit=8, is_head=False, num_heads=1, dtype=BF16):
    """Reference :278-306."""
    return _dequantize(q, s, z, None, None, quantize_bit, is_head, num_heads, dtype)


# ---------------------------------------------------------------------------------------
# attention-map compression (reference: operators/compress_function.py:309-317)
# ---------------------------------------------------------------------------------------
def _threshold_tensor(outlier, device) -> torch.Tensor:
    if torch.is_tensor(outlier):
        return outlier.to(device=device, dtype=torch.float32).reshape(())
    return torch.tensor(float(outlier), device=device, dtype=torch.float32)


_PINNED = {}          # device index -> [pinned int64 ring, next slot]
_PINNED_SLOTS = 256


class PendingCount:
    """A device-side element count on its way to the host without a stream synchronisation: an
    asynchronous copy into pinned memory followed by an event.  `value()` waits for that event only
    (the device keeps executing whatever has been enqueued since)."""

    def __init__(self, count: torch.Tensor):
        ring = _PINNED.get(count.device.index)
        if ring is None:
            ring = _PINNED[count.device.index] = [torch.empty(_PINNED_SLOTS, dtype=torch.int64, pin_memory=True), 0]
        slot = ring[1]
        ring[1] = (slot + 1) % _PINNED_SLOTS          # a slot is read long before the ring comes round again
        self._host = ring[0][slot:slot + 1]
        self._host.copy_(count.reshape(1), non_blocking=True)
        self._event = torch.cuda.Event()
        self._event.record(torch.cuda.current_stream(count.device))

    def value(self) -> int:
        self._event.synchronize()
        return int(self._host[0])


def compress_attention_map(x: torch.Tensor, outlier, seg_offsets=None, compare_abs=False, capacity=None):
    """Kept entries of the flattened map: (indices int64 [nnz] ascending, values bf16 [nnz],
    seg_offsets int64 [nseg + 1]).  An entry is kept when x > outlier (compared in bf16, as
    torch does) and x != 0.  seg_offsets lets restore_attention_map skip the index search.
    `seg_offsets` may be passed in when the producer of x already counted (softmax_forward with a
    threshold): the counting pass is skipped.  compare_abs: keep by magnitude, |x| > outlier.

    `capacity` (an int): no read-back of nnz.  The outputs are sized `capacity`, entries that do not
    fit are not written, and a fourth result - a PendingCount - tells later how many entries there
    were; the caller must check `pending.value() <= capacity` before the lists are consumed and call
    again without `capacity` (passing the same seg_offsets) when they did not fit.  Entries past nnz
    in the outputs are uninitialised; seg_offsets bounds what the restore kernels read."""
    _lib.require_gpu(x)
    if x.dtype != BF16:
        x = x.to(BF16)
    flat = x.reshape(-1)
    if not flat.is_contiguous() or flat.data_ptr() % 16:
        flat = flat.clone(memory_format=torch.contiguous_format)
    n = flat.numel()
    thr = _threshold_tensor(outlier, x.device)
    nseg = _lib.lib().hyc_sparse_num_segments(n)
    st = _lib.stream_of(x)
    if seg_offsets is not None:
        if seg_offsets.numel() != nseg + 1 or seg_offsets.dtype != torch.int64:
            raise ValueError("seg_offsets does not belong to a map of this size")
        offsets = seg_offsets
    else:
        counts = torch.empty(max(nseg, 1), device=x.device, dtype=torch.int32)
        offsets = torch.empty(nseg + 1, device=x.device, dtype=torch.int64)
        _lib.call("hyc_sparse_count", flat.data_ptr(), n, thr.data_ptr(), int(compare_abs), counts.data_ptr(),
                  offsets.data_ptr(), st)
    if capacity is not None:
        capacity = int(capacity)
        idx = torch.empty(capacity, device=x.device, dtype=torch.int64)
        val = torch.empty(capacity, device=x.device, dtype=BF16)
        _lib.call("hyc_sparse_write_bounded", flat.data_ptr(), n, thr.data_ptr(), int(compare_abs), offsets.data_ptr(),
                  capacity, idx.data_ptr(), val.data_ptr(), st)
        return idx, val, offsets, PendingCount(offsets[-1:])
    nnz = int(offsets[-1].item())      # the one host sync; to_sparse() has the same one
    idx = torch.empty(nnz, device=x.device, dtype=torch.int64)
    val = torch.empty(nnz, device=x.device, dtype=BF16)
    if nnz:
        _lib.call("hyc_sparse_write", flat.data_ptr(), n, thr.data_ptr(), int(compare_abs), offsets.data_ptr(),
                  idx.data_ptr(), val.data_ptr(), st)
    return idx, val, offsets


def check_map_lists(idx, val, seg_offsets, numel: int) -> None:
    """The kernels that rebuild a map read idx / val up to seg_offsets' last entry and seg_offsets up to
    the map's last 4096-element segment: lists of another map would be read out of bounds on the device."""
    if idx.dtype != torch.int64 or idx.numel() != val.numel():
        raise ValueError(f"compressed map: int64 indices and as many values expected, got {idx.dtype} "
                         f"x {idx.numel()} and {val.numel()} values")
    if seg_offsets is not None:
        nseg = -(-numel // 4096)
        if seg_offsets.dtype != torch.int64 or seg_offsets.numel() != nseg + 1:
            raise ValueError(f"seg_offsets must be int64 [{nseg + 1}] for a map of {numel} elements, got "
                             f"{seg_offsets.dtype} [{seg_offsets.numel()}]")


def restore_attention_map(idx, val, seg_offsets, shape):
    """Dense bf16 tensor of `shape`: zeros with val[i] at flat position idx[i]."""
    n = 1
    for d in shape:
        n *= int(d)
    check_map_lists(idx, val, seg_offsets, n)
    _lib.require_gpu(idx, val)
    idx = idx.reshape(-1).contiguous()
    val = val.to(BF16).reshape(-1).contiguous()
    st = _lib.stream_of(val)
    if seg_offsets is None:
        nseg = _lib.lib().hyc_sparse_num_segments(n)
        seg_offsets = torch.empty(nseg + 1, device=val.device, dtype=torch.int64)
        _lib.call("hyc_sparse_segment_offsets", idx.data_ptr(), idx.numel(), n, seg_offsets.data_ptr(), st)
    out = torch.empty(n, device=val.device, dtype=BF16)
    _lib.call("hyc_sparse_restore", idx.data_ptr(), val.data_ptr(), seg_offsets.data_ptr(), n, out.data_ptr(), st)
    return out.reshape(tuple(shape))


def compression_softmax(x: torch.Tensor, outlier):
    """Sparse COO tensor of the flattened map, like (x * (x > outlier)).flatten().to_sparse().
    Reference :309-313."""
    idx, val, _ = compress_attention_map(x, outlier)
    return torch.sparse_coo_tensor(idx.unsqueeze(0), val, (x.numel(),), is_coalesced=True)


def decompression_softmax(x_sparse: torch.Tensor):
    """Dense 1-D tensor, like x_sparse.to_dense().  Reference :316-317."""
    if not x_sparse.is_coalesced():
        x_sparse = x_sparse.coalesce()
    return restore_attention_map(x_sparse.indices()[0], x_sparse.values(), None, x_sparse.shape)


# ---------------------------------------------------------------------------------------
# pruning forms of the reference that none of its layers call (operators/compress_function.py:39-42,
# :320-341); kept so that the module is a complete stand-in
# ---------------------------------------------------------------------------------------
def get_statistics_structed_pruning(x: torch.Tensor, outlier_ratio: float):
    """Indices of the int(N * ratio) channels with the largest norm over dim -2, per leading index
    (x.abs().norm(dim=-2) then topk; reference :39-42).  Ties: larger norm first, then lower channel."""
    _lib.require_gpu(x)
    if x.dim() < 2:
        raise ValueError("needs at least [rows, channels]")
    xb = x.to(BF16)
    n = xb.shape[-1]
    k = int(n * outlier_ratio)
    lead = xb.shape[:-2]
    flat = xb.reshape(-1, xb.shape[-2], n)
    out = torch.empty((flat.shape[0], k), device=x.device, dtype=torch.int64)
    scale = torch.empty((1, n), device=x.device, dtype=BF16)
    for b in range(flat.shape[0]):
        stats, strips, _ = _batch0_stats(flat[b:b + 1])
        _lib.call("hyc_channel_select", stats.data_ptr(), strips, n, k, 8, 0, out[b].data_ptr() if k else None,
                  scale.data_ptr(), None, _lib.stream_of(x))
    return out.reshape(*lead, k)


def _unravel(flat_idx, shape):
    idx = []
    rem = flat_idx
    for d in reversed(shape):
        idx.append(rem % d)
        rem = torch.div(rem, d, rounding_mode="floor")
    return torch.stack(idx[::-1], dim=0)


def compression_unstructed_pruning_coo(x: torch.Tensor, outlier):
    """Sparse COO tensor of x's own shape holding the elements with |x| > outlier, like
    (x * (x.abs() > outlier)).to_sparse().  Reference :320-324."""
    idx, val, _ = compress_attention_map(x, outlier, compare_abs=True)
    return torch.sparse_coo_tensor(_unravel(idx, tuple(x.shape)), val, tuple(x.shape), is_coalesced=True)


def decompression_unstructed_pruning_coo(x_sparse: torch.Tensor):
    """x_sparse.to_dense().  Reference :327-328."""
    if not x_sparse.is_coalesced():
        x_sparse = x_sparse.coalesce()
    shape = tuple(x_sparse.shape)
    flat = torch.zeros((), device=x_sparse.device, dtype=torch.int64)
    for d, row in zip(shape, x_sparse.indices()):
        flat = flat * d + row
    return restore_attention_map(flat, x_sparse.values(), None, shape)


def compression_unstructed_pruning_bitmap(x: torch.Tensor, outlier):
    """(kept values in flat order, boolean mask |x| > outlier).  Reference :331-335: the values are
    (x * mask)[mask], so a kept element is any with |x| > outlier (zeros cannot qualify for
    outlier >= 0; NaN never does)."""
    _lib.require_gpu(x)
    thr = _threshold_tensor(outlier, x.device)
    mask = x.to(BF16).abs() > thr.to(BF16)
    idx, val, _ = compress_attention_map(x, outlier, compare_abs=True)
    if idx.numel() != int(mask.sum()):                        # outlier < 0 keeps exact zeros, which the compaction drops
        return (x.to(BF16) * mask)[mask], mask
    return val, mask


def decompression_unstructed_pruning_bitmap(x_sparse: torch.Tensor, mask: torch.Tensor):
    """Dense tensor of mask's shape with x_sparse at the True positions.  Reference :338-341 (which
    leaves the other positions uninitialised; here they are zero)."""
    _lib.require_gpu(x_sparse, mask)
    flat = torch.nonzero(mask.reshape(-1)).reshape(-1)
    return restore_attention_map(flat, x_sparse, None, tuple(mask.shape))


# ---------------------------------------------------------------------------------------
# statistics + compress in one call (reference: operators/compress_function.py:346-368)
# ---------------------------------------------------------------------------------------
def compression_pack_channel_base(x, o_ratio, q_bit, q_method, it_num, it_num_thd, static_value):
    """Outlier-channel extraction + quantisation; calibrates while it_num < it_num_thd."""
    if it_num < it_num_thd:
        o_channel_idx, scale = get_statistics_channel_base(x, o_ratio, q_bit, q_method)
    else:
        o_channel_idx, scale = static_value['outlier_channel_index'], static_value['scale']
    o, q = outlier_subtraction_fuse_compression_quantization(x, scale, o_channel_idx, q_bit)
    return o, q, o_channel_idx, scale


def compression_pack_quant_base(x, q_bit, q_method, it_num, it_num_thd, static_value):
    if it_num < it_num_thd:
        scale = get_statistics_only_quant(x, q_bit, q_method)
    else:
        scale = static_value['scale']
    return compression_quantization(x, scale, q_bit), scale


def compression_pack_quant_zp_base(x, q_bit, q_method, it_num, it_num_thd, static_value):
    if it_num < it_num_thd:
        scale, zero_point = get_statistics_only_quant_zero_point(x, q_bit, q_method)
    else:
        scale, zero_point = static_value['scale'], static_value['zero_point']
    return compression_quantization_with_zero_point(x, scale, zero_point, q_bit), scale, zero_point


def compression_pack_softmax_base(x, o_ratio, it_num, it_num_thd, static_value):
    """Attention-map compression -> (sparse COO tensor, threshold).  Reference :371-379."""
    if it_num < it_num_thd:
        outlier = get_statistics_softmax(x, o_ratio)
    else:
        outlier = static_value['outlier']
    return compression_softmax(x, outlier), outlier


def compression_pack_unstructed_pruning_coo(x, o_ratio, it_num, it_num_thd, static_value):
    """Reference :382-388."""
    outlier = get_statistics_outlier(x, o_ratio) if it_num < it_num_thd else static_value['outlier']
    return compression_unstructed_pruning_coo(x, outlier), outlier


def compression_pack_unstructed_pruning_bitmap(x, o_ratio, it_num, it_num_thd, static_value):
    """Reference :391-397."""
    outlier = get_statistics_outlier(x, o_ratio) if it_num < it_num_thd else static_value['outlier']
    x_outlier, mask = compression_unstructed_pruning_bitmap(x, outlier)
    return x_outlier, outlier, mask
