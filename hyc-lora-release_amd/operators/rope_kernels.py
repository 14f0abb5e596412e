"""In-place rotary position embedding on gfx950 (reference API: operators/rope_kernels.py:81-126)."""
import torch

from .. import _lib

ROPE_GROUP_SIZE = 4


def calculate_settings(n):
    """Launch settings of the reference's Triton kernel (rope_kernels.py:21-33).  The HIP kernel picks
    its own launch shape; the values are returned only so that callers which thread them through to
    rope_backward keep working."""
    block = 1 << max(0, (int(n) - 1).bit_length())
    if block > 65536:
        raise RuntimeError(f"n = {n} exceeds the maximum fused size 65536.")
    warps = 32 if block >= 32768 else 16 if block >= 8192 else 8 if block >= 2048 else 4
    return block, warps


def _table(t, seq_len, half):
    t = t.squeeze()
    if t.dim() != 2 or t.shape[0] < seq_len or t.shape[1] < half:
        raise ValueError(f"angle table of shape {tuple(t.shape)} does not cover seq_len {seq_len}, half head {half}")
    if t.stride(1) != 1 or t.stride(0) % 8 or t.data_ptr() % 16:
        t = t.contiguous()
    return t


def _rotate(x, cos, sin, backward):
    _lib.require_gpu(x, cos, sin)
    if x.dtype != torch.bfloat16 or x.dim() != 4:
        raise NotImplementedError("rope rotates a bfloat16 [batch, seq, heads, head_dim] tensor")
    b, s, h, d = x.shape
    if d % 16:
        raise ValueError(f"head_dim {d} is not a multiple of 16")
    cos, sin = _table(cos, s, d // 2), _table(sin, s, d // 2)
    if cos.dtype != sin.dtype or cos.dtype not in (torch.bfloat16, torch.float32):
        raise NotImplementedError("cos/sin tables must both be bfloat16 or both float32")
    _lib.call("hyc_rope", x.data_ptr(), cos.data_ptr(), sin.data_ptr(), int(cos.dtype == torch.float32),
              b, s, h, d, x.stride(0), x.stride(1), x.stride(2), cos.stride(0), sin.stride(0), int(backward),
              _lib.stream_of(x))
    return x


def _in_place_ok(x):
    return x.stride(-1) == 1 and all(st % 8 == 0 for st in x.stride()[:-1]) and x.data_ptr() % 16 == 0


def rope_forward(x, cos, sin):
    """Rotates x [batch, seq, heads, head_dim] IN PLACE and returns it (a contiguous input is the
    caller's own tensor, exactly as in the reference, rope_kernels.py:81-109).  A strided view whose
    last dimension is contiguous — e.g. the transpose of a [B,H,S,D] tensor — is rotated where it
    lies instead of being copied first; the reference copies such a view."""
    if not _in_place_ok(x):
        x = x.contiguous()
    return _rotate(x, cos, sin, False)


def rope_backward(dy, cos, sin, n_groups=None, BLOCK_SIZE=None, num_warps=None):
    """Same rotation with -sin (rope_kernels.py:112-126); the three launch arguments of the
    reference are accepted and ignored."""
    if not _in_place_ok(dy):
        dy = dy.contiguous()
    return _rotate(dy, cos, sin, True)
