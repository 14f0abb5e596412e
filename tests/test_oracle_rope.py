"""Pins the oracle's rotary embedding (operators/rope_kernels.py:54-78) with checks that do not
retype its formula: the rotate-half form of the published RoPE, a complex rotation in float64,
and the invariants of a rotation."""
import torch

from oracle import hyc_oracle as O

BF16 = torch.bfloat16


def tables(S, D, dtype, base=10000.0):
    inv = 1.0 / base ** (torch.arange(0, D, 2, dtype=torch.float64) / D)
    ang = torch.arange(S, dtype=torch.float64)[:, None] * inv[None, :]        # [S, D/2]
    full = torch.cat([ang, ang], dim=-1)                                      # HF layout: halves repeated
    return full.cos().to(dtype), full.sin().to(dtype), ang


def rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat([-x[..., h:], x[..., :h]], dim=-1)


def test_matches_rotate_half_form_fp32_tables():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 12, 3, 32, generator=g).to(BF16)
    cos, sin, _ = tables(16, 32, torch.float32)
    want = (x.float() * cos[None, :12, None, :] + rotate_half(x.float()) * sin[None, :12, None, :]).to(BF16)
    assert torch.equal(O.rope(x, cos, sin), want)
    # the tables may carry singleton dimensions, as the reference's rotary module returns them
    assert torch.equal(O.rope(x, cos[None, None], sin[None, None]), want)


def test_is_the_complex_rotation():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, 9, 2, 16, generator=g).to(BF16)
    cos, sin, ang = tables(9, 16, torch.float32)
    z = torch.complex(x[..., :8].double(), x[..., 8:].double()) * torch.polar(torch.ones_like(ang), ang)[None, :, None, :]
    want = torch.cat([z.real, z.imag], dim=-1)
    got = O.rope(x, cos, sin).double()
    assert (got - want).abs().max() <= 2 ** -8 * want.abs().max()
    # backward is the inverse rotation
    zb = torch.complex(x[..., :8].double(), x[..., 8:].double()) * torch.polar(torch.ones_like(ang), -ang)[None, :, None, :]
    gotb = O.rope(x, cos, sin, backward=True).double()
    assert (gotb - torch.cat([zb.real, zb.imag], dim=-1)).abs().max() <= 2 ** -8 * want.abs().max()


def test_rotation_invariants():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, 33, 4, 64, generator=g).to(BF16)
    cos, sin, _ = tables(40, 64, torch.float32)
    y = O.rope(x, cos, sin)
    assert torch.equal(y[:, 0], x[:, 0])                                   # position 0: angle 0
    n_in = x.float()[..., :32] ** 2 + x.float()[..., 32:] ** 2
    n_out = y.float()[..., :32] ** 2 + y.float()[..., 32:] ** 2
    assert ((n_in - n_out).abs() <= 2 ** -6 * n_in + 1e-6).all()            # pair norms preserved
    back = O.rope(y, cos, sin, backward=True)
    assert (back.float() - x.float()).abs().max() <= 2 ** -6 * x.float().abs().max()


def test_bf16_tables_round_after_every_operation():
    # known answer by hand: x1=3, x2=5, c=0.7578125, s=0.65234375 (both exact in bf16)
    #   x1*c = 2.2734375  = 145.5 * 2^-6 -> tie to even 146 -> 2.28125
    #   x2*s = 3.26171875 = 208.75 * 2^-6 -> 209 -> 3.265625        x1' = 2.28125 - 3.265625 = -0.984375
    #   (rounding only once at the end would give -0.98828125)
    #   x2*c = 3.7890625  = 242.5 * 2^-6 -> 242 -> 3.78125
    #   x1*s = 1.95703125 = 250.5 * 2^-7 -> 250 -> 1.953125         x2' = 5.734375 = 183.5 * 2^-5 -> 184 -> 5.75
    x = torch.tensor([3.0, 5.0]).to(BF16).reshape(1, 1, 1, 2)
    cos = torch.tensor([[0.7578125, 0.0], [1.0, 0.0]]).to(BF16)     # two rows: squeeze() must keep it 2-D
    sin = torch.tensor([[0.65234375, 0.0], [0.0, 0.0]]).to(BF16)
    y = O.rope(x, cos, sin).float().flatten().tolist()
    assert y == [-0.984375, 5.75]
    yb = O.rope(x, cos, sin, backward=True).float().flatten().tolist()
    # x1' = 2.28125 + 3.265625 = 5.546875 = 177.5 * 2^-5 -> 178 -> 5.5625 ; x2' = 3.78125 - 1.953125 = 1.828125
    assert yb == [5.5625, 1.828125]
