"""Pins the torch oracle's quantise / pack / dequantise (oracle/hyc_oracle.py) with checks
that do not retype its formulas: an independently written scalar C implementation,
hand-computed known answers, round trips, the error bound and the q=8 identity layout."""
import numpy as np
import pytest
import torch

from oracle import hyc_oracle as O
from helpers import BF16, activation_with_outlier_channels, same_bits, scalar_quant_pack, scalar_unpack_dequant

QBITS = [2, 4, 8]


def bf(v):
    return torch.tensor(v, dtype=torch.float32).to(BF16)


@pytest.mark.parametrize("q_bit", QBITS)
def test_known_answers_exact_multiples_and_clamp(q_bit):
    # x = j*s exactly -> code j + 2^(q-1); beyond the range -> clamped ends
    half = 2 ** (q_bit - 1)
    s = bf([[0.25] * 32])
    js = torch.arange(-half - 3, half + 3)
    x = torch.zeros(1, js.numel(), 32)
    x[0, :, :] = (js * 0.25).unsqueeze(1)
    c = O.quant_codes(x.to(BF16), s, q_bit)
    expect = torch.clamp(js, -half, half - 1) + half
    assert torch.equal(c[0, :, 0].long(), expect)
    assert torch.equal(c[0, :, 31].long(), expect)


def test_ties_round_away_from_zero():
    # t = +-0.5, +-1.5, +-2.5 : roundf gives +-1, +-2, +-3 (half-even would give 0, 2, 2)
    s = bf([[1.0] * 32])
    t = torch.tensor([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.4375, -0.4375])
    x = t.reshape(1, -1, 1).repeat(1, 1, 32).to(BF16)
    c = O.quant_codes(x, s, 8)[0, :, 0].long() - 128
    assert c.tolist() == [1, -1, 2, -2, 3, -3, 0, 0]


def test_nan_inf_and_zero_scale():
    s = bf([[1.0] * 31 + [0.0]])
    x = torch.zeros(1, 4, 32)
    x[0, 0, 0] = float("nan"); x[0, 1, 0] = float("inf"); x[0, 2, 0] = float("-inf")
    x[0, 0, 31] = 1.0; x[0, 1, 31] = -1.0; x[0, 2, 31] = 0.0      # x/0: +inf, -inf, NaN
    c = O.quant_codes(x.to(BF16), s, 4)
    assert c[0, :3, 0].tolist() == [0, 15, 0]
    assert c[0, :3, 31].tolist() == [15, 0, 0]


def test_pack_layout_by_hand():
    # codes 0..31 in one 32-column block
    c = torch.arange(32, dtype=torch.uint8).reshape(1, 1, 32)
    assert torch.equal(O.pack_codes(c, 8), c)                                   # q=8: identity
    c4 = (c % 16)
    p4 = O.pack_codes(c4, 4)[0, 0]
    assert p4.tolist() == [(j % 16) | (((j + 16) % 16) << 4) for j in range(16)]  # byte j = c[j] | c[j+16]<<4
    c2 = (c % 4)
    p2 = O.pack_codes(c2, 2)[0, 0]
    assert p2.tolist() == [(j % 4) | (((j + 8) % 4) << 2) | (((j + 16) % 4) << 4) | (((j + 24) % 4) << 6)
                           for j in range(8)]
    # a single set code lands where the layout says: column 21 at q=4 -> byte 5, high nibble
    one = torch.zeros(1, 1, 64, dtype=torch.uint8); one[0, 0, 32 + 21] = 9
    p = O.pack_codes(one, 4)[0, 0]
    assert p[16 + 5].item() == 9 << 4 and p.sum().item() == 9 << 4
    # column 27 at q=2 -> byte 3, bits 6..7
    one = torch.zeros(1, 1, 32, dtype=torch.uint8); one[0, 0, 27] = 3
    p = O.pack_codes(one, 2)[0, 0]
    assert p[3].item() == 3 << 6 and p.sum().item() == 3 << 6


@pytest.mark.parametrize("q_bit", QBITS)
def test_pack_unpack_round_trip(q_bit):
    g = torch.Generator().manual_seed(q_bit)
    c = torch.randint(0, 2 ** q_bit, (2, 5, 96), generator=g, dtype=torch.uint8)
    assert torch.equal(O.unpack_codes(O.pack_codes(c, q_bit), q_bit), c)


@pytest.mark.parametrize("q_bit", QBITS)
@pytest.mark.parametrize("with_zp", [False, True])
def test_against_scalar_c(q_bit, with_zp):
    g = torch.Generator().manual_seed(100 + q_bit)
    x = (torch.randn(2, 37, 96, generator=g) * 3).to(BF16)
    x[1, 0, :8] = torch.tensor([0.0, -0.0, float("inf"), float("-inf"), float("nan"), 1e-40, 3e38, -3e38]).to(BF16)
    s = O.scale_only_quant(x, q_bit)      # from batch element 0, which holds ordinary values only
    s[0, 5] = 0.0            # a constant channel in the scale-only path
    z = None
    if with_zp:
        z = (torch.randn(1, 96, generator=g) * 3).to(BF16)      # non-integer after calibration averaging
    p_t = O.compress(x, s, q_bit, z)
    p_c = scalar_quant_pack(x, s, z, q_bit)
    assert torch.equal(p_t, p_c)
    s[0, 5] = 0.5
    d_t = O.decompress(p_t, s, q_bit, z)
    d_c = scalar_unpack_dequant(p_t, s, z, q_bit)
    assert same_bits(d_t, d_c)


@pytest.mark.parametrize("q_bit", QBITS)
def test_error_bound_and_outlier_columns_config1(q_bit):
    # benchmark configuration 1 (reduced in rows for CPU time): off-clamp error <= s/2,
    # outlier columns carry code 2^(q-1) and decode to exactly 0 before the scatter
    x, planted = activation_with_outlier_channels(seed=7, shape=(2, 64, 4096))
    idx, s = O.channel_stats(x, 0.005, q_bit)
    assert torch.equal(torch.sort(idx).values, planted)
    xo, p = O.compress_channel_base(x, s, idx, q_bit)
    assert torch.equal(xo, x[:, :, idx])
    codes = O.unpack_codes(p, q_bit)
    assert (codes[:, :, idx] == 2 ** (q_bit - 1)).all()
    d = O.decompress(p, s, q_bit)
    assert (d[:, :, idx] == 0).all()
    xz = x.clone(); xz[:, :, idx] = 0
    inside = (codes > 0) & (codes < 2 ** q_bit - 1)
    err = (xz.float() - d.float()).abs()
    # |x - c*s| <= s/2, plus one bf16 rounding (relative 2^-8) of the product c*s
    bound = s.float().reshape(1, 1, -1) * 0.5 + d.float().abs() * 2 ** -8
    assert (err[inside] <= bound[inside]).all()
    back = O.decompress_channel_base(p, s, xo, idx, q_bit)
    assert same_bits(back[:, :, idx], x[:, :, idx])


def test_scale_closed_forms():
    x = torch.zeros(2, 16, 64)
    x[0, :, 1] = torch.linspace(-7.5, 7.5, 16)       # max-min = 15 -> s = 1 at q=4
    x[0, 3, 2] = 255.0                                 # max-min = 255 -> s = 1 at q=8
    x[1, :, 3] = 1000.0                                # batch element 1 is ignored
    x = x.to(BF16)
    assert O.scale_only_quant(x, 4)[0, 1].item() == 1.0
    assert O.scale_only_quant(x, 8)[0, 2].item() == 1.0
    assert O.scale_only_quant(x, 4)[0, 3].item() == 0.0
    assert O.scale_only_quant(x, 4)[0, 0].item() == 0.0
    _, s = O.channel_stats(x, 0.0, 4)
    assert s[0, 0].item() == 0.00099945068359375      # bf16(1e-3) replaces a zero step
    assert s[0, 1].item() == 1.0


def test_outlier_tie_break_is_index_ascending():
    x = torch.zeros(1, 4, 64)
    x[0, :, [5, 9, 17, 40]] = 2.0                      # four equal norms
    x[0, :, 33] = 3.0
    idx = O.outlier_channels(x.to(BF16), 3 / 64)
    assert idx.tolist() == [33, 5, 9]


def test_zero_point_round_trip():
    g = torch.Generator().manual_seed(3)
    # asymmetric data; the zero point -round(min/s) - 128 must stay inside int8 as in the reference
    x = (torch.rand(1, 64, 64, generator=g) * 4 - 1).to(BF16)
    s, z = O.scale_zero_point(x, 8)
    p = O.compress(x, s, 8, z)
    d = O.decompress(p, s, 8, z)
    # one step of clamp/rounding slack plus the bf16 roundings of (code - z) and of the product
    assert ((d.float() - x.float()).abs() <= s.float().reshape(1, 1, -1) + x.float().abs() * 2 ** -6).all()


def test_update_dict_running_mean():
    old = {'scale': None, 'outlier_channel_index': None}
    for it, v in enumerate([2.0, 4.0, 6.0]):
        old = O.update_dict(old, {'scale': torch.tensor([v]), 'outlier_channel_index': torch.tensor([it])}, it)
    assert old['scale'].item() == 4.0 and old['outlier_channel_index'].item() == 2
