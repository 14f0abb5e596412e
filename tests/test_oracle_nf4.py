"""Pins the oracle's NF4 dequantisation with known answers: nibble order, the block statistic of each
element, the nested (double-quantised) statistics formula, and exact recovery of weights that lie on
the NF4 grid.  bitsandbytes itself is not installed, so its own outputs are not available."""
import torch

from oracle import hyc_oracle as O

BF16 = torch.bfloat16


def test_nibble_order_and_block_statistics():
    # bytes 0x1F, 0x70: elements = levels 1, 15, 7, 0  ->  -0.6962, 1.0, 0.0, -1.0
    packed = torch.tensor([0x1F, 0x70] * 4, dtype=torch.uint8)          # 16 elements, blocksize 8: two blocks
    absmax = torch.tensor([2.0, 0.5])
    w = O.nf4_dequant(packed, absmax, (16,), blocksize=8).float().tolist()
    lv = [-0.6961928009986877, 1.0, 0.0, -1.0]
    want = [torch.tensor(v * 2.0).to(BF16).item() for v in lv * 2] + [torch.tensor(v * 0.5).to(BF16).item() for v in lv * 2]
    assert w == want


def test_code_book_is_the_published_one():
    t = O.NF4_TABLE
    assert t.numel() == 16 and t[0] == -1 and t[7] == 0 and t[15] == 1
    assert bool((t[1:] > t[:-1]).all())
    # QLoRA's construction: quantiles of N(0,1) normalised to [-1, 1], asymmetric around an exact zero
    # (8 positive levels from 9 quantile points, 7 negative from 8); first positive and last negative level:
    nd = torch.distributions.Normal(0.0, 1.0)
    off = 0.9677083
    pos = nd.icdf(torch.linspace(off, 0.5, 9)[:-1])
    neg = -nd.icdf(torch.linspace(off, 0.5, 8)[:-1])
    grid = torch.cat([pos, torch.zeros(1), neg]).sort().values
    grid = grid / grid.max()
    assert torch.allclose(grid, t, atol=2e-6)


def test_nested_statistics_formula():
    code2 = torch.linspace(-1, 1, 256)
    packed = torch.tensor([0xFF] * 8, dtype=torch.uint8)                   # 16 elements of level 15 (= 1.0), blocksize 8
    absmax_codes = torch.tensor([255, 0], dtype=torch.uint8)               # code2 -> +1, -1
    nested = (code2, torch.tensor([0.25]), 256, 1.0)                        # absmax = +-0.25 + 1.0
    w = O.nf4_dequant(packed, absmax_codes, (2, 8), blocksize=8, nested=nested).float()
    assert w[0].tolist() == [1.25] * 8 and w[1].tolist() == [0.75] * 8


def test_on_grid_weights_round_trip_exactly():
    g = torch.Generator().manual_seed(0)
    codes = torch.randint(0, 16, (4, 128), generator=g)
    codes[:, 0] = 15                                                       # every block of 64 holds its maximum
    codes[:, 64] = 0
    scale = torch.tensor([0.5, 2.0, 0.125, 1.0])[:, None]
    w = O.NF4_TABLE[codes] * scale
    packed, absmax, _ = O.nf4_quantize(w, blocksize=64)
    assert torch.equal(O.nf4_dequant(packed, absmax, w.shape), w.to(BF16))
    # random weights: error bounded by half the widest gap of the grid times the block maximum
    w = torch.randn(8, 256, generator=g)
    packed, absmax, _ = O.nf4_quantize(w, blocksize=64)
    err = (O.nf4_dequant(packed, absmax, w.shape).float() - w).abs().reshape(-1, 64)
    gap = (O.NF4_TABLE[1:] - O.NF4_TABLE[:-1]).max() / 2
    assert bool((err <= (gap * absmax[:, None] * 1.01 + 1e-2)).all())
