"""LoRA add fused with the compression of a projection's frozen part (gfx950 MFMA kernels).

No counterpart module in the reference: it computes `x_main + x_lora_a @ w_lora_b`
(models/utils/compute_utils.py:21-24), quantises `x_main` with a separate call
(models/llama/fused_llama_layer_intra_inter_full_fuse.py:128-140) and in backward dequantises and
adds again (:416-417, :439-441, :447-449), each step a pass over the tensor.  The functions here give
the same tensors, bit for bit, from one pass each.

`lora_products` / `lora_product_from_codes` are the rank-R GEMMs of lora_forward / lora_backward
(compute_utils.py:22, :30-33) as one streaming pass over the wide operand."""
import torch

from .. import _lib
from ._fuse import _prep

BF16 = torch.bfloat16


def _check(xa, b, n, rows):
    """Shapes the kernels rely on: they read xa[row, 0..R) for every row of the activation and
    B[0..R, 0..N), so a short operand would be read out of bounds on the device."""
    if b.dim() != 2:
        raise ValueError(f"LoRA-B must be a matrix [R, N], got shape {tuple(b.shape)}")
    r = b.shape[0]
    if xa.dim() < 1 or xa.shape[-1] != r:
        raise ValueError(f"LoRA rank mismatch: x@A has shape {tuple(xa.shape)}, B has {r} rows")
    if xa.numel() != rows * r:
        raise ValueError(f"x@A must hold one row of {r} values per activation row ({rows} rows), "
                         f"got shape {tuple(xa.shape)}")
    if b.shape[1] != n:
        raise ValueError(f"LoRA-B width {b.shape[1]} does not match the activation width {n}")
    if n % 32:
        raise ValueError(f"channel count must be a multiple of 32, got {n}")
    if r % 4 or not 4 <= r <= 64:
        raise ValueError(f"LoRA rank must be a multiple of 4 in 4..64, got {r}")
    return r


def _operands_ok(xa, b):
    n, r = b.shape[1], b.shape[0]
    return (xa.is_cuda and xa.dtype == BF16 and b.dtype == BF16 and xa.shape[-1] == r
            and n % 32 == 0 and r % 4 == 0 and 4 <= r <= 64 and xa.numel() > 0)


def supported(x_main, xa, b):
    """Whether lora_add / lora_add_quant take these operands (bf16, rank and width within the
    kernels' limits)."""
    return x_main.is_cuda and x_main.dtype == BF16 and x_main.shape[-1] == b.shape[1] and _operands_ok(xa, b)


def supported_restore(q, xa, b):
    """The same for lora_add_restore (q: packed codes uint8 [B, M, N*bits/8])."""
    return q.is_cuda and q.dtype == torch.uint8 and q.dim() == 3 and _operands_ok(xa, b)


def _lora_b(b):
    """-> (tensor to pass, b_transposed flag).  A [R, N] view of an [N, R] contiguous weight (what
    `lora_B.weight.T` is) is handed over as it lies in memory."""
    if b.dtype == BF16 and not b.is_contiguous() and b.mT.is_contiguous() and b.data_ptr() % 8 == 0:
        return b, 1
    return _prep(b, "b"), 0


def lora_add(x_main, xa, b, inplace=False, residual=None):
    """bf16(x_main + bf16(xa @ b)), then - with a residual of x_main's shape - bf16(residual + that);
    `inplace` overwrites x_main (contiguous bf16) and returns it."""
    n = x_main.shape[-1]
    r = _check(xa, b, n, x_main.numel() // max(n, 1))
    if residual is not None and residual.shape != x_main.shape:
        raise ValueError(f"residual must have the shape of x_main {tuple(x_main.shape)}, got {tuple(residual.shape)}")
    _lib.require_gpu(x_main, xa, b, residual)
    x = x_main if (inplace and x_main.dtype == BF16 and x_main.is_contiguous() and x_main.data_ptr() % 16 == 0) \
        else _prep(x_main, "x_main")
    y = x if inplace else torch.empty_like(x)
    xa, (b, bt) = _prep(xa, "xa"), _lora_b(b)
    if residual is not None:
        residual = _prep(residual, "residual")
    _lib.call("hyc_lora_add", xa.data_ptr(), b.data_ptr(), bt, x.data_ptr(), _lib.ptr(residual), y.data_ptr(),
              x.numel() // n, n, r, _lib.stream_of(x))
    if inplace and y is not x_main:
        x_main.copy_(y)
        return x_main
    return y


SUM_MAX_RANK = 16          # hyc_lora_add_sum holds the LoRA-B operands of all its terms in registers


def supported_sum(terms):
    """Whether lora_add_sum takes these (x_main, xa, b) terms: two or three, one shape, rank <= SUM_MAX_RANK."""
    if not 2 <= len(terms) <= 3:
        return False
    shape = terms[0][0].shape
    return all(x.shape == shape and x.dtype == BF16 and supported(x, xa, b) and b.shape[0] <= SUM_MAX_RANK and
               b.shape[0] == terms[0][2].shape[0] for x, xa, b in terms)


def lora_add_sum(terms):
    """t_0 (+) t_1 [(+) t_2] with t_i = bf16(x_i + bf16(xa_i @ b_i)) and (+) the bf16 addition, in that order: the
    bits of lora_add(x_0, ...), lora_add(x_1, ..., residual=that), lora_add(x_2, ..., residual=that), in one
    pass.  terms: (x_main, xa, b) triples of one shape; the result overwrites the first x_main when that is a
    contiguous bf16 tensor, and is returned."""
    if not 2 <= len(terms) <= 3:
        raise ValueError(f"lora_add_sum takes two or three terms, got {len(terms)}")
    shape = terms[0][0].shape
    n = shape[-1]
    rows = terms[0][0].numel() // max(n, 1)
    members, keep, rank = [], [], None
    for x_main, xa, b in terms:
        if x_main.shape != shape:
            raise ValueError(f"every term must have the shape {tuple(shape)}, got {tuple(x_main.shape)}")
        r = _check(xa, b, n, rows)
        if rank not in (None, r):
            raise ValueError("the terms share one LoRA rank")
        rank = r
        _lib.require_gpu(x_main, xa, b)
        x = x_main if (x_main.dtype == BF16 and x_main.is_contiguous() and x_main.data_ptr() % 16 == 0) else _prep(x_main, "x_main")
        xa, (b, bt) = _prep(xa, "xa"), _lora_b(b)
        members.append(_lib.LoraSumMember(xa.data_ptr(), b.data_ptr(), bt, x.data_ptr()))
        keep.append((x, xa, b))
    if rank > SUM_MAX_RANK:
        raise ValueError(f"lora_add_sum takes ranks up to {SUM_MAX_RANK}, got {rank}")
    y = keep[0][0]
    arr = (_lib.LoraSumMember * len(members))(*members)
    _lib.call("hyc_lora_add_sum", arr, len(members), y.data_ptr(), rows, n, rank, _lib.stream_of(y))
    return y


def _vec_ok(t, n, name):
    if t is not None and t.numel() != n:
        raise ValueError(f"{name} must have {n} elements (one per channel), got {t.numel()}")


def _vec(t, n, name):
    _vec_ok(t, n, name)
    return _prep(_lib.bf16_vector(t), name)


ROPE_HEAD_DIM = 128          # the fused rotation needs heads as wide as a column tile


def _rope_tables(rope, seq_len):
    from .rope_kernels import _table
    cos, sin = rope
    cos, sin = _table(cos, seq_len, ROPE_HEAD_DIM // 2), _table(sin, seq_len, ROPE_HEAD_DIM // 2)
    if cos.dtype != sin.dtype or cos.dtype not in (BF16, torch.float32):
        raise NotImplementedError("cos/sin tables must both be bfloat16 or both float32")
    return cos, sin


def lora_add_quant(x_main, xa, b, scale, zero_point=None, quantize_bit=8, inplace=False, rope=None):
    """-> (q, y): q = the packed codes compression_quantization[_with_zero_point](x_main, scale[, zero_point])
    returns, y = bf16(x_main + bf16(xa @ b)); x_main [B, M, N] is read once.  rope=(cos, sin) also
    rotates y as rope_forward would on its [B, M, N / 128, 128] view (heads of 128 dims only)."""
    if quantize_bit not in (2, 4, 8):
        raise ValueError(f"quantize_bit must be 2, 4 or 8, got {quantize_bit}")
    if x_main.dim() != 3:
        raise ValueError(f"x_main must be [B, M, N], got shape {tuple(x_main.shape)}")
    B, M, n = x_main.shape
    r = _check(xa, b, n, B * M)
    _vec_ok(scale, n, "scale")
    _vec_ok(zero_point, n, "zero point")
    _lib.require_gpu(x_main, xa, b, scale, zero_point)
    x = _prep(x_main, "x_main")
    y = x if (inplace and x is x_main) else torch.empty_like(x)
    xa, (b, bt) = _prep(xa, "xa"), _lora_b(b)
    s = _vec(scale, n, "scale")
    z = None if zero_point is None else _vec(zero_point, n, "zero point")
    q = torch.empty((B, M, n * quantize_bit // 8), device=x.device, dtype=torch.uint8)
    if rope is not None:
        if n % ROPE_HEAD_DIM:
            raise ValueError(f"the fused rotation needs a width that is a multiple of {ROPE_HEAD_DIM}, got {n}")
        cos, sin = _rope_tables(rope, M)
        _lib.call("hyc_lora_add_quant_rope", xa.data_ptr(), b.data_ptr(), bt, x.data_ptr(), s.data_ptr(), _lib.ptr(z),
                  q.data_ptr(), y.data_ptr(), cos.data_ptr(), sin.data_ptr(), int(cos.dtype == torch.float32), M,
                  cos.stride(0), sin.stride(0), B * M, n, r, quantize_bit, _lib.stream_of(x))
        return q, y
    _lib.call("hyc_lora_add_quant", xa.data_ptr(), b.data_ptr(), bt, x.data_ptr(), s.data_ptr(), _lib.ptr(z),
              q.data_ptr(), y.data_ptr(), B * M, n, r, quantize_bit, _lib.stream_of(x))
    return q, y


def lora_add_restore(q, scale, xa, b, zero_point=None, quantize_bit=8, rope=None):
    """bf16(decompression_dequantization[_with_zero_point](q, scale[, zero_point]) + bf16(xa @ b)) without
    writing the dequantised tensor; rope=(cos, sin) rotates the result like lora_add_quant's."""
    if quantize_bit not in (2, 4, 8):
        raise ValueError(f"quantize_bit must be 2, 4 or 8, got {quantize_bit}")
    if q.dim() != 3:
        raise ValueError(f"packed codes must be [B, M, N*bits/8], got shape {tuple(q.shape)}")
    B, M, nbytes = q.shape
    n = scale.numel()
    if nbytes * 8 != n * quantize_bit or q.dtype != torch.uint8:
        raise ValueError(f"packed codes must be uint8 of width {n * quantize_bit // 8}, got {q.dtype} {nbytes}")
    r = _check(xa, b, n, B * M)
    _vec_ok(zero_point, n, "zero point")
    _lib.require_gpu(q, scale, xa, b, zero_point)
    q = q.contiguous()
    xa, (b, bt) = _prep(xa, "xa"), _lora_b(b)
    s = _vec(scale, n, "scale")
    z = None if zero_point is None else _vec(zero_point, n, "zero point")
    y = torch.empty((B, M, n), device=q.device, dtype=BF16)
    if rope is not None:
        if n % ROPE_HEAD_DIM:
            raise ValueError(f"the fused rotation needs a width that is a multiple of {ROPE_HEAD_DIM}, got {n}")
        cos, sin = _rope_tables(rope, M)
        _lib.call("hyc_lora_add_restore_rope", xa.data_ptr(), b.data_ptr(), bt, q.data_ptr(), s.data_ptr(), _lib.ptr(z),
                  y.data_ptr(), cos.data_ptr(), sin.data_ptr(), int(cos.dtype == torch.float32), M,
                  cos.stride(0), sin.stride(0), B * M, n, r, quantize_bit, _lib.stream_of(q))
        return y
    _lib.call("hyc_lora_add_restore", xa.data_ptr(), b.data_ptr(), bt, q.data_ptr(), s.data_ptr(), _lib.ptr(z),
              y.data_ptr(), B * M, n, r, quantize_bit, _lib.stream_of(q))
    return y


GROUP_MAX = 4                # operand sets one grouped launch takes


def _member(xa, b, bt, x, s, z, q, y, rope_tables, n):
    m = _lib.LoraAddMember()
    m.xa, m.b, m.b_transposed, m.x = xa.data_ptr(), b.data_ptr(), bt, _lib.ptr(x)
    m.scale, m.zero_point, m.q, m.y, m.N = s.data_ptr(), _lib.ptr(z), q.data_ptr(), y.data_ptr(), n
    if rope_tables is not None:
        cos, sin, seq = rope_tables
        m.cos_t, m.sin_t, m.table_is_fp32 = cos.data_ptr(), sin.data_ptr(), int(cos.dtype == torch.float32)
        m.seq_len, m.stride_cos, m.stride_sin = seq, cos.stride(0), sin.stride(0)
    return m


def lora_add_quant_group(items, quantize_bit=8, inplace=False):
    """lora_add_quant for up to GROUP_MAX operand sets in one launch -> [(q, y), ...], each pair the same bits
    as its own call.  items: dicts with x_main [B, M, N_i], xa [B, M, R], b [R, N_i], scale, and optionally
    zero_point (all items or none) and rope=(cos, sin); B, M and R are shared."""
    if quantize_bit not in (2, 4, 8):
        raise ValueError(f"quantize_bit must be 2, 4 or 8, got {quantize_bit}")
    if not 1 <= len(items) <= GROUP_MAX:
        raise ValueError(f"a group holds 1 to {GROUP_MAX} operand sets, got {len(items)}")
    B, M = items[0]["x_main"].shape[:2]
    members, outs, keep = [], [], []
    rank = None
    for it in items:
        x_main, xa, b, scale, zp, rope = it["x_main"], it["xa"], it["b"], it["scale"], it.get("zero_point"), it.get("rope")
        if x_main.dim() != 3 or tuple(x_main.shape[:2]) != (B, M):
            raise ValueError(f"every x_main must be [{B}, {M}, N], got shape {tuple(x_main.shape)}")
        n = x_main.shape[-1]
        r = _check(xa, b, n, B * M)
        if rank not in (None, r):
            raise ValueError("the members of a group share one LoRA rank")
        rank = r
        if (zp is None) != (items[0].get("zero_point") is None):
            raise ValueError("either every member of a group has a zero point or none has")
        _vec_ok(scale, n, "scale")
        _vec_ok(zp, n, "zero point")
        _lib.require_gpu(x_main, xa, b, scale, zp)
        x = _prep(x_main, "x_main")
        y = x if (inplace and x is x_main) else torch.empty_like(x)
        xa, (b, bt) = _prep(xa, "xa"), _lora_b(b)
        s = _vec(scale, n, "scale")
        z = None if zp is None else _vec(zp, n, "zero point")
        q = torch.empty((B, M, n * quantize_bit // 8), device=x.device, dtype=torch.uint8)
        tables = None
        if rope is not None:
            if n % ROPE_HEAD_DIM:
                raise ValueError(f"the fused rotation needs a width that is a multiple of {ROPE_HEAD_DIM}, got {n}")
            tables = _rope_tables(rope, M) + (M,)
        members.append(_member(xa, b, bt, x, s, z, q, y, tables, n))
        keep.append((x, xa, b, s, z, tables))
        outs.append((q, y))
    arr = (_lib.LoraAddMember * len(members))(*members)
    _lib.call("hyc_lora_add_quant_group", arr, len(members), B * M, rank, quantize_bit, _lib.stream_of(outs[0][0]))
    return outs


def lora_add_restore_group(items, quantize_bit=8):
    """lora_add_restore for up to GROUP_MAX operand sets in one launch -> [y, ...].  items: dicts with q
    [B, M, N_i*bits/8], scale, xa, b and optionally zero_point (all or none) and rope=(cos, sin)."""
    if quantize_bit not in (2, 4, 8):
        raise ValueError(f"quantize_bit must be 2, 4 or 8, got {quantize_bit}")
    if not 1 <= len(items) <= GROUP_MAX:
        raise ValueError(f"a group holds 1 to {GROUP_MAX} operand sets, got {len(items)}")
    B, M = items[0]["q"].shape[:2]
    members, outs, keep = [], [], []
    rank = None
    for it in items:
        q, scale, xa, b, zp, rope = it["q"], it["scale"], it["xa"], it["b"], it.get("zero_point"), it.get("rope")
        n = scale.numel()
        if q.dim() != 3 or tuple(q.shape[:2]) != (B, M) or q.shape[2] * 8 != n * quantize_bit or q.dtype != torch.uint8:
            raise ValueError(f"packed codes must be uint8 [{B}, {M}, {n * quantize_bit // 8}], got {q.dtype} {tuple(q.shape)}")
        r = _check(xa, b, n, B * M)
        if rank not in (None, r):
            raise ValueError("the members of a group share one LoRA rank")
        rank = r
        if (zp is None) != (items[0].get("zero_point") is None):
            raise ValueError("either every member of a group has a zero point or none has")
        _vec_ok(zp, n, "zero point")
        _lib.require_gpu(q, scale, xa, b, zp)
        q = q.contiguous()
        xa, (b, bt) = _prep(xa, "xa"), _lora_b(b)
        s = _vec(scale, n, "scale")
        z = None if zp is None else _vec(zp, n, "zero point")
        y = torch.empty((B, M, n), device=q.device, dtype=BF16)
        tables = None
        if rope is not None:
            if n % ROPE_HEAD_DIM:
                raise ValueError(f"the fused rotation needs a width that is a multiple of {ROPE_HEAD_DIM}, got {n}")
            tables = _rope_tables(rope, M) + (M,)
        members.append(_member(xa, b, bt, None, s, z, q, y, tables, n))
        keep.append((q, xa, b, s, z, tables))
        outs.append(y)
    arr = (_lib.LoraAddMember * len(members))(*members)
    _lib.call("hyc_lora_add_restore_group", arr, len(members), B * M, rank, quantize_bit, _lib.stream_of(outs[0]))
    return outs


def contract_supported(x, n, r):
    """Whether lora_products takes a wide operand of this dtype / width and this rank."""
    return x.is_cuda and x.dtype == BF16 and n % 32 == 0 and 2 <= r <= 64 and r % 2 == 0 and x.numel() > 0


def _contract(x, codes, u, v, T, n, r, dev, p1_transposed=False):
    want1, want2 = u is not None, v is not None
    vt = 0
    if want1:
        u = _prep(u, "u")
        if u.shape[-1] != r or u.numel() != T * r:
            raise ValueError(f"u must be [T, {r}] with T = {T}, got {tuple(u.shape)}")
    if want2:
        if tuple(v.shape) != (r, n):
            raise ValueError(f"v must be [{r}, {n}], got {tuple(v.shape)}")
        v, vt = _lora_b(v)
    nbytes = _lib.lib().hyc_lora_contract_workspace(T, n, r, int(want1), int(want2))
    ws = torch.empty(max(nbytes, 16), device=dev, dtype=torch.uint8)
    p1 = torch.empty((n, r) if p1_transposed else (r, n), device=dev, dtype=BF16) if want1 else None
    p2 = torch.empty((T, r), device=dev, dtype=BF16) if want2 else None
    q, s, z, bits = codes if codes is not None else (None, None, None, 0)
    _lib.call("hyc_lora_contract", _lib.ptr(x), _lib.ptr(q), _lib.ptr(s), _lib.ptr(z), bits, _lib.ptr(u), _lib.ptr(v), vt,
              _lib.ptr(p1), int(p1_transposed), _lib.ptr(p2), ws.data_ptr(), ws.numel(), T, n, r, _lib.stream_of(ws))
    return p1, p2


def lora_products(x, u=None, v=None, p1_transposed=False):
    """x [..., N] bf16 read once -> (u^T x as [R, N] or None, x v^T as [..., R] or None), u [..., R], v [R, N]
    (a `weight.T` view of an [N, R] weight is read in place).  fp32 accumulation over the whole
    contraction, one bf16 rounding.  p1_transposed: the first result comes as x^T u, [N, R] contiguous - the
    layout of a lora_B weight, so that its gradient needs no copy on the way into `.grad`."""
    if u is None and v is None:
        raise ValueError("nothing to compute: pass u, v or both")
    n = x.shape[-1]
    r = u.shape[-1] if u is not None else v.shape[0]
    if n % 32 or r % 2 or not 2 <= r <= 64:
        raise ValueError(f"width must be a multiple of 32 and the rank even within 2..64, got {n}, {r}")
    if u is not None and u.numel() != x.numel() // n * r:
        raise ValueError(f"u must be [T, {r}] with T = {x.numel() // n}, got {tuple(u.shape)}")
    if v is not None and tuple(v.shape) != (r, n):
        raise ValueError(f"v must be [{r}, {n}], got {tuple(v.shape)}")
    _lib.require_gpu(x, u, v)
    lead = tuple(x.shape[:-1])
    x = _prep(x, "x")
    T = x.numel() // n
    p1, p2 = _contract(x, None, u, v, T, n, r, x.device, p1_transposed)
    return p1, (p2.reshape(*lead, r) if p2 is not None else None)


def lora_product_from_codes(q, scale, u, zero_point=None, quantize_bit=8):
    """u^T . DQ(q) as [R, N] straight from packed codes q [B, M, N*bits/8] (what
    decompression_dequantization[_with_zero_point](q, scale[, zero_point]) would expand first)."""
    if quantize_bit not in (2, 4, 8):
        raise ValueError(f"quantize_bit must be 2, 4 or 8, got {quantize_bit}")
    if q.dim() != 3:
        raise ValueError(f"packed codes must be [B, M, N*bits/8], got shape {tuple(q.shape)}")
    B, M, nbytes = q.shape
    n = scale.numel()
    if nbytes * 8 != n * quantize_bit or q.dtype != torch.uint8:
        raise ValueError(f"packed codes must be uint8 of width {n * quantize_bit // 8}, got {q.dtype} {nbytes}")
    r = u.shape[-1]
    if n % 32 or r % 2 or not 2 <= r <= 64:
        raise ValueError(f"width must be a multiple of 32 and the rank even within 2..64, got {n}, {r}")
    if u.numel() != B * M * r:
        raise ValueError(f"u must be [T, {r}] with T = {B * M}, got {tuple(u.shape)}")
    _vec_ok(zero_point, n, "zero point")
    _lib.require_gpu(q, scale, u, zero_point)
    s = _vec(scale, n, "scale")
    z = None if zero_point is None else _vec(zero_point, n, "zero point")
    p1, _ = _contract(None, (q.contiguous(), s, z, quantize_bit), u, None, B * M, n, r, q.device)
    return p1
