"""GPU parity of the in-place rotary embedding against the oracle (bit-exact: the kernel performs
the same individually rounded operations) and against the rotate-half form."""
import pytest
import torch

from helpers import BF16, same_bits
from oracle import hyc_oracle as O
from test_oracle_rope import rotate_half, tables

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rk():
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import rope_kernels
    return rope_kernels


@pytest.mark.parametrize("shape", [(2, 64, 4, 128), (1, 100, 3, 64), (3, 7, 32, 128), (1, 1, 1, 16), (2, 33, 8, 96),
                                   (1, 5, 2, 256)])
@pytest.mark.parametrize("tdtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("backward", [False, True])
def test_rope_matches_oracle(rk, dev, shape, tdtype, backward):
    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(*shape, generator=g).to(BF16)
    cos, sin, _ = tables(shape[1] + 9, shape[-1], tdtype)
    want = O.rope(x, cos, sin, backward)
    xd = x.to(dev)
    fn = (lambda t, c, s: rk.rope_backward(t, c, s, 1, 64, 4)) if backward else rk.rope_forward
    got = fn(xd, cos.to(dev)[None, None], sin.to(dev)[None, None])      # [1,1,S,D] tables, as the rotary module returns
    assert got.data_ptr() == xd.data_ptr()                               # in place on a contiguous input
    assert same_bits(got, want)


def test_rope_in_place_on_head_major_layout(rk, dev):
    """A [B,H,S,D] tensor viewed as [B,S,H,D] is rotated where it lies (no transposed copy)."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 6, 40, 128, generator=g).to(BF16)               # [B,H,S,D]
    cos, sin, _ = tables(64, 128, torch.bfloat16)
    want = O.rope(x.transpose(1, 2), cos, sin).transpose(1, 2)
    xd = x.to(dev)
    out = rk.rope_forward(xd.transpose(1, 2), cos.to(dev), sin.to(dev))
    assert out.data_ptr() == xd.data_ptr() and same_bits(xd, want.contiguous())
    # a slice of a fused [B,S,3*H*D] projection: only the middle third is rotated
    qkv = torch.randn(2, 40, 3 * 4 * 64, generator=g).to(BF16)
    cos, sin, _ = tables(40, 64, torch.float32)
    qd = qkv.to(dev)
    k_view = qd[..., 256:512].unflatten(-1, (4, 64))
    rk.rope_forward(k_view, cos.to(dev), sin.to(dev))
    want = qkv.clone()
    want[..., 256:512] = O.rope(qkv[..., 256:512].unflatten(-1, (4, 64)), cos, sin).flatten(-2)
    assert same_bits(qd, want)


def test_rope_against_rotate_half_and_inverse(rk, dev):
    g = torch.Generator().manual_seed(6)
    x = torch.randn(2, 128, 8, 128, generator=g).to(BF16)
    cos, sin, _ = tables(128, 128, torch.float32)
    want = (x.float() * cos[None, :, None, :] + rotate_half(x.float()) * sin[None, :, None, :]).to(BF16)
    y = rk.rope_forward(x.to(dev), cos.to(dev), sin.to(dev))
    assert same_bits(y, want)
    back = rk.rope_backward(y.clone(), cos.to(dev), sin.to(dev), 2, 64, 4)
    assert (back.cpu().float() - x.float()).abs().max() <= 2 ** -6 * x.float().abs().max()


def test_rope_rejects_what_it_cannot_do(rk, dev):
    cos, sin, _ = tables(8, 24, torch.float32)
    with pytest.raises(ValueError):
        rk.rope_forward(torch.zeros(1, 4, 2, 24, device=dev, dtype=BF16), cos.to(dev), sin.to(dev))   # head_dim % 16
    cos, sin, _ = tables(4, 32, torch.float32)
    with pytest.raises(ValueError):
        rk.rope_forward(torch.zeros(1, 8, 2, 32, device=dev, dtype=BF16), cos.to(dev), sin.to(dev))   # table too short
    with pytest.raises(NotImplementedError):
        rk.rope_forward(torch.zeros(1, 4, 2, 32, device=dev), cos.to(dev), sin.to(dev))               # fp32 x
    with pytest.raises(Exception):
        rk.rope_forward(torch.zeros(1, 4, 2, 32, dtype=BF16), cos, sin)                               # CPU tensors
    assert rk.calculate_settings(64) == (64, 4) and rk.calculate_settings(3000) == (4096, 8)
