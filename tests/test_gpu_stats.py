"""GPU parity of the calibration statistics (hyc_channel_stats + hyc_channel_select) against
the CPU oracle: steps and zero points bit-exact, outlier channel lists equal with the defined
tie rule (and, for untied random data, equal up to channels whose bf16 norm equals the k-th)."""
import pytest
import torch

from helpers import BF16, activation_with_outlier_channels, same_bits
from oracle import hyc_oracle as O

pytestmark = pytest.mark.gpu
QBITS = [2, 4, 8]


@pytest.fixture(scope="module")
def cf():
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import compress_function
    return compress_function


def _rand(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(BF16)


@pytest.mark.parametrize("q_bit", QBITS)
@pytest.mark.parametrize("shape", [(2, 512, 4096), (3, 37, 96), (1, 1, 32), (2, 1000, 1024), (1, 300, 11008)])
def test_scale_only_bit_exact(cf, dev, q_bit, shape):
    x = _rand(shape, seed=shape[1] + q_bit, scale=1.5)
    x[-1] = x[-1] * 100                      # other batch elements must not matter
    s = cf.get_statistics_only_quant(x.to(dev), q_bit, 'per-channel')
    assert tuple(s.shape) == (1, shape[2]) and s.dtype == BF16
    assert same_bits(s.cpu(), O.scale_only_quant(x, q_bit))


@pytest.mark.parametrize("q_bit", QBITS)
def test_zero_point_bit_exact(cf, dev, q_bit):
    x = (_rand((2, 200, 256), seed=4).float() * torch.linspace(0.1, 3, 256) + torch.linspace(-2, 2, 256)).to(BF16)
    s, z = cf.get_statistics_only_quant_zero_point(x.to(dev), q_bit, 'per-channel')
    s_ref, z_ref = O.scale_zero_point(x, q_bit)
    assert same_bits(s.cpu(), s_ref)
    assert z.dtype == torch.int8 and torch.equal(z.cpu(), z_ref)


@pytest.mark.parametrize("q_bit", QBITS)
def test_head_layout_input(cf, dev, q_bit):
    xh = _rand((2, 8, 50, 64), seed=9)
    assert same_bits(cf.get_statistics_only_quant(xh.to(dev), q_bit, 'per-channel').cpu(), O.scale_only_quant(xh, q_bit))
    xv = _rand((2, 50, 8, 64), seed=10).transpose(1, 2)
    assert same_bits(cf.get_statistics_only_quant(xv.to(dev), q_bit, 'per-channel').cpu(), O.scale_only_quant(xv, q_bit))


@pytest.mark.parametrize("q_bit", QBITS)
def test_config1_channel_base(cf, dev, q_bit):
    x, planted = activation_with_outlier_channels(seed=99)
    idx, s = cf.get_statistics_channel_base(x.to(dev), 0.005, q_bit, 'per-channel')
    assert idx.dtype == torch.int64 and idx.numel() == 20
    idx_ref, s_ref = O.channel_stats(x, 0.005, q_bit)
    assert torch.equal(torch.sort(idx.cpu()).values, planted)
    assert torch.equal(idx.cpu(), idx_ref), "order must follow norm descending, index ascending"
    assert same_bits(s.cpu(), s_ref)
    assert (s.cpu()[0, planted].float() == 0.00099945068359375).all()


def test_tie_rule_and_constant_channels(cf, dev):
    x = torch.zeros(2, 16, 128)
    x[0, :, [5, 9, 17, 40, 100]] = 2.0          # five equal norms
    x[0, :, 33] = 3.0
    x[0, :8, 64] = 1.0                            # smaller norm, non-constant
    x = x.to(BF16)
    idx, s = cf.get_statistics_channel_base(x.to(dev), 4 / 128, 4, 'per-channel')
    assert idx.cpu().tolist() == [33, 5, 9, 17]
    idx_ref, s_ref = O.channel_stats(x, 4 / 128, 4)
    assert torch.equal(idx.cpu(), idx_ref) and same_bits(s.cpu(), s_ref)
    # channel 40 is constant but not chosen: max-min = 0 -> step bf16(1e-3); channel 64 spans 1 -> 1/15
    assert s.cpu()[0, 40].item() == 0.00099945068359375
    assert s.cpu()[0, 64].item() == torch.tensor(1 / 15).to(BF16).item()


def test_random_data_boundary_ties(cf, dev):
    # without planted outliers many bf16 norms coincide; the fp32 sum of squares is accumulated
    # in a different order on the GPU, so a channel may land on the other side of a bf16
    # rounding boundary.  Allowed difference: channels whose oracle norm equals the k-th norm
    # or is one bf16 step away from it.
    x = _rand((2, 2048, 4096), seed=5)
    k = 20
    idx, s = cf.get_statistics_channel_base(x.to(dev), 0.005, 4, 'per-channel')
    idx = idx.cpu()
    assert idx.numel() == k and torch.unique(idx).numel() == k
    nrm = O.channel_norms(x).float()
    kth = torch.sort(nrm, descending=True).values[k - 1]
    ref = set(O.outlier_channels(x, 0.005).tolist())
    for c in set(idx.tolist()) ^ ref:
        assert abs(nrm[c].item() - kth.item()) <= kth.item() * 2 ** -7, f"channel {c} is not a boundary tie"
    # given the GPU's own channel list, the step must be exact
    _, s_ref = O.channel_stats(x, 0.005, 4, idx=idx)
    assert same_bits(s.cpu(), s_ref)


def test_nan_propagates_like_torch(cf, dev):
    x = _rand((1, 64, 64), seed=8)
    x[0, 3, 7] = float("nan")
    s = cf.get_statistics_only_quant(x.to(dev), 8, 'per-channel').cpu()
    s_ref = O.scale_only_quant(x, 8)
    assert torch.isnan(s[0, 7]) and torch.isnan(s_ref[0, 7])
    keep = torch.ones(64, dtype=torch.bool); keep[7] = False
    assert same_bits(s[0, keep], s_ref[0, keep])


def test_calibration_dispatch_and_static_values(cf, dev):
    x, _ = activation_with_outlier_channels(seed=3, shape=(2, 64, 1024))
    xg = x.to(dev)
    o, q, idx, s = cf.compression_pack_channel_base(xg, 0.005, 4, 'per-channel', 0, 5, {})
    static = {'outlier_channel_index': idx, 'scale': s}
    o2, q2, idx2, s2 = cf.compression_pack_channel_base(xg, 0.005, 4, 'per-channel', 5, 5, static)
    assert idx2 is idx and s2 is s and torch.equal(q2, q) and torch.equal(o2, o)
    qq, ss = cf.compression_pack_quant_base(xg, 4, 'per-channel', 0, 5, {})
    assert torch.equal(qq.cpu(), O.compress(x, O.scale_only_quant(x, 4), 4))
    qz, sz, zz = cf.compression_pack_quant_zp_base(xg, 8, 'per-channel', 0, 5, {})
    s_ref, z_ref = O.scale_zero_point(x, 8)
    assert torch.equal(qz.cpu(), O.compress(x, s_ref, 8, z_ref))
    with pytest.raises(NotImplementedError):
        cf.get_statistics_only_quant(xg, 4, 'per-tensor')
    with pytest.raises(ValueError):
        cf.get_statistics_only_quant(xg, 4, 'per-row')


@pytest.mark.parametrize("shape", [(1, 2048, 14336), (2, 512, 4096), (1, 37, 96), (1, 7, 32), (1, 1000, 1024)])
def test_statistics_do_not_depend_on_the_strip_count(cf, dev, shape):
    """The rows are split into strips whose number follows the launch size aimed for ("stats_waves"); minimum
    and maximum cannot depend on it, the fp32 sum of squares only in its last bits - so steps and zero points
    must be the same bits for every setting and equal the oracle's, and a channel list may differ from the
    oracle's only in channels whose norm is within a bf16 step of the k-th (the order of the additions)."""
    from hyclora_amd import _lib
    x = _rand(shape, seed=shape[1], scale=1.5)
    x[0, :, 5] *= 40
    k = int(shape[2] * 0.02)
    got = []
    try:
        for waves in (4, 64, 2048, 1 << 16):
            _lib.set_tuning("stats_waves", waves)
            s, z = cf.get_statistics_only_quant_zero_point(x.to(dev), 4, 'per-channel')
            idx, sc = cf.get_statistics_channel_base(x.to(dev), 0.02, 4, 'per-channel')
            got.append((s.cpu(), z.cpu(), idx.cpu(), sc.cpu()))
    finally:
        _lib.set_tuning("stats_waves", 4096)
    s_ref, z_ref = O.scale_zero_point(x, 4)
    nrm = O.channel_norms(x).float()
    ref = set(O.outlier_channels(x, 0.02).tolist())
    kth = torch.sort(nrm, descending=True).values[k - 1] if k else None
    for s, z, idx, sc in got:
        assert same_bits(s, s_ref) and torch.equal(z, z_ref)
        assert idx.numel() == k and torch.unique(idx).numel() == k
        for c in set(idx.tolist()) ^ ref:
            assert abs(nrm[c].item() - kth.item()) <= kth.item() * 2 ** -7, f"channel {c} is not a boundary tie"
        if k:
            assert idx[0].item() == 5
            # descending norms, ties by ascending channel
            keys = [(-nrm[c].item(), c) for c in idx.tolist()]
            assert all(a[0] <= b[0] for a, b in zip(keys, keys[1:]))
        _, sc_ref = O.channel_stats(x, 0.02, 4, idx=idx)
        assert same_bits(sc, sc_ref)


@pytest.mark.parametrize("n,k", [(4096, 1024), (4096, 1025), (2048, 2048), (1024, 1), (32768, 163), (96, 95)])
def test_channel_lists_of_any_length(cf, dev, n, k):
    """Lists of up to 1024 channels are found by a radix select and ordered by counting, longer ones by rounds
    of a block-wide maximum; both must give `norm descending, channel ascending`.  Exactly representable norms
    (every channel constant, its value a small integer) make the expected list exact, ties included."""
    g = torch.Generator().manual_seed(n + k)
    level = torch.randint(0, 200, (n,), generator=g).float()          # many ties
    x = level.reshape(1, 1, n).expand(1, 4, n).to(BF16).contiguous()
    idx, _ = cf.get_statistics_channel_base(x.to(dev), k / n + 1e-9, 4, 'per-channel')
    assert idx.numel() == k
    order = sorted(range(n), key=lambda c: (-level[c].item(), c))[:k]
    assert idx.cpu().tolist() == order
