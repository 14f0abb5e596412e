"""GPU checks of the pruning forms of the operator module that no layer of the reference calls
(compress_function.py:39-42, :320-341, :382-397), against the torch composites they are defined by."""
import pytest
import torch

from helpers import BF16, same_bits

pytestmark = pytest.mark.gpu


def same_bits_nan_ok(a, b):
    """Bit-equal, except that a NaN only has to be a NaN (torch's own CPU kernels return different NaN
    payloads for the same product depending on whether the vectorised or the scalar path ran)."""
    a, b = a.detach().cpu(), b.detach().cpu()
    return a.shape == b.shape and torch.equal(a.isnan(), b.isnan()) and same_bits(torch.nan_to_num(a), torch.nan_to_num(b))


@pytest.fixture(scope="module")
def cf():
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import compress_function
    return compress_function


@pytest.mark.parametrize("shape", [(2, 3, 64, 96), (1, 5000), (4, 128, 32)])
@pytest.mark.parametrize("ratio", [0.1, 0.5])
def test_unstructured_pruning_coo_and_bitmap(cf, dev, shape, ratio):
    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(*shape, generator=g).to(BF16)
    x.view(-1)[:3] = torch.tensor([0.0, float("nan"), -7.0]).to(BF16)
    thr = cf.get_statistics_outlier(x.to(dev), ratio)
    # the threshold is the exact order statistic of |x| (NaN sorts last in torch.kthvalue as well)
    k = int(x.numel() * (1 - ratio))
    assert thr.item() == torch.kthvalue(x.float().abs().flatten(), k).values.item()
    t = thr.cpu().to(BF16)
    want = (x * (x.abs() > t)).to_sparse()
    got = cf.compression_unstructed_pruning_coo(x.to(dev), thr)
    assert got.shape == x.shape and got.is_coalesced()
    assert torch.equal(got.indices().cpu(), want.indices()) and same_bits_nan_ok(got.values(), want.values())
    dense = cf.decompression_unstructed_pruning_coo(got)
    assert same_bits_nan_ok(dense, want.to_dense())
    vals, mask = cf.compression_unstructed_pruning_bitmap(x.to(dev), thr)
    wmask = x.abs() > t
    assert torch.equal(mask.cpu(), wmask) and same_bits_nan_ok(vals, (x * wmask)[wmask])
    back = cf.decompression_unstructed_pruning_bitmap(vals, mask)
    assert same_bits_nan_ok(back, torch.where(wmask, x, torch.zeros_like(x)))
    # the calib-or-static dispatchers
    sp, thr2 = cf.compression_pack_unstructed_pruning_coo(x.to(dev), ratio, 0, 5, {'outlier': None})
    assert thr2.item() == thr.item() and torch.equal(sp.indices(), got.indices())
    v3, thr3, m3 = cf.compression_pack_unstructed_pruning_bitmap(x.to(dev), ratio, 9, 5, {'outlier': thr})
    assert thr3 is thr and same_bits(v3, vals) and torch.equal(m3, mask)


def test_structured_pruning_channels(cf, dev):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(3, 200, 256, generator=g)
    x = (x * (1 + torch.arange(256) / 64.0)).to(BF16)          # distinct channel norms
    got = cf.get_statistics_structed_pruning(x.to(dev), 0.05).cpu()
    k = int(256 * 0.05)
    assert got.shape == (3, k)
    # the norms are bf16 numbers (x.abs().norm(dim=-2) of a bf16 tensor), so several channels can tie;
    # any top-k of the rounded norms is a right answer, and ties go to the lower channel here
    norms = x.float().pow(2).sum(dim=-2).sqrt().to(BF16).float()
    for b in range(3):
        sel = torch.zeros(256, dtype=torch.bool)
        sel[got[b]] = True
        assert int(sel.sum()) == k
        assert norms[b][sel].min() >= norms[b][~sel].max()
        order = sorted(range(256), key=lambda c: (-norms[b, c].item(), c))[:k]
        assert got[b].tolist() == order
