"""GPU parity of the attention-map path: exact threshold (k-th value), ordered compaction,
dense restore and softmax backward, against the CPU oracle / torch library routines."""
import pytest
import torch

from helpers import BF16, assert_close_bf16, same_bits
from oracle import hyc_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cf():
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import compress_function
    return compress_function


@pytest.fixture(scope="module")
def sk():
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import softmax_kernels
    return softmax_kernels


def attention_map(seed, shape=(2, 4, 128, 128), causal=True):
    """benchmark configuration 3 in small: softmax of N(0,1)*8/sqrt(128) logits with a causal mask."""
    g = torch.Generator().manual_seed(seed)
    b, h, n, _ = shape
    s = torch.randn(*shape, generator=g) * 8 / 128 ** 0.5
    if causal:
        s = s + torch.full((n, n), float("-inf")).triu(1)
    return torch.softmax(s, dim=-1, dtype=torch.float32).to(BF16)


@pytest.mark.parametrize("shape", [(2, 4, 128, 128), (1, 2, 100, 100), (1, 1, 8, 8), (2, 2, 256, 256)])
@pytest.mark.parametrize("ratio", [0.05, 0.5, 0.001])
def test_threshold_is_exact_order_statistic(cf, dev, shape, ratio):
    a = attention_map(seed=shape[2], shape=shape)
    thr = cf.get_statistics_softmax(a.to(dev), ratio)
    assert thr.dtype == torch.float32 and thr.dim() == 0
    assert thr.item() == O.softmax_threshold(a, ratio).item()
    # independent of kthvalue: the value at that rank of a full sort
    k = int(a.numel() * (1 - ratio))
    assert thr.item() == torch.sort(a.float().flatten()).values[k - 1].item()


def test_threshold_general_values(cf, dev):
    # negative values, values >= 2 (outside the LDS-binned range), -0, inf
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(3, 1000, generator=g) * 5).to(BF16)
    x[0, :5] = torch.tensor([float("inf"), -float("inf"), -0.0, 0.0, 300.0]).to(BF16)
    for k in (1, 2, 17, 1500, 2999, 3000):
        got = cf._kth_value(x.to(dev), k).item()
        assert got == torch.kthvalue(x.float().flatten(), k).values.item(), k
    with pytest.raises(RuntimeError):
        cf._kth_value(x.to(dev), 0)
    with pytest.raises(RuntimeError):
        cf._kth_value(x.to(dev), 3001)


@pytest.mark.parametrize("shape", [(2, 4, 128, 128), (1, 2, 100, 100), (1, 1, 8, 8), (1, 3, 77, 77)])
def test_compaction_and_restore(cf, dev, shape):
    a = attention_map(seed=5, shape=shape)
    thr = O.softmax_threshold(a, 0.05)
    idx_ref, val_ref = O.softmax_compress(a, thr)
    ag = a.to(dev)
    idx, val, seg = cf.compress_attention_map(ag, thr.to(dev))
    assert idx.dtype == torch.int64 and torch.equal(idx.cpu(), idx_ref)
    assert same_bits(val.cpu(), val_ref)
    dense_ref = O.softmax_restore(idx_ref, val_ref, a.shape)
    assert same_bits(cf.restore_attention_map(idx, val, seg, a.shape).cpu(), dense_ref)
    assert same_bits(cf.restore_attention_map(idx, val, None, a.shape).cpu(), dense_ref)
    # reference-shaped API: a sparse COO tensor of the flattened map, and to_dense()
    sp = cf.compression_softmax(ag, thr.to(dev))
    ref_sp = (a * (a > thr)).flatten().to_sparse()
    assert sp.layout == torch.sparse_coo and sp.shape == ref_sp.shape
    assert torch.equal(sp.indices().cpu(), ref_sp.indices()) and same_bits(sp.values().cpu(), ref_sp.values())
    assert same_bits(cf.decompression_softmax(sp).cpu(), ref_sp.to_dense())
    assert same_bits(sp.to_dense().cpu(), ref_sp.to_dense())
    # a sparse tensor that torch made restores through the same kernel
    assert same_bits(cf.decompression_softmax(ref_sp.to(dev)).cpu(), ref_sp.to_dense())


@pytest.mark.parametrize("shape,ratio", [((2, 4, 128, 128), 0.05), ((1, 2, 100, 100), 0.5), ((1, 1, 8, 8), 0.5),
                                         ((1, 2, 256, 256), 0.9)])         # the last: dense segments (direct stores)
def test_compaction_into_preallocated_lists(cf, dev, shape, ratio):
    """The compaction that sizes its outputs before the count is known: with room for everything the
    lists' first nnz entries are the exact lists and the deferred count is nnz; with too little room
    the first `capacity` entries are still right, nothing is written past them, and the count tells."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd import _lib as L
    a = attention_map(seed=3, shape=shape).to(dev)
    thr = cf.get_statistics_softmax(a, ratio)
    idx, val, seg = cf.compress_attention_map(a, thr)
    nnz = idx.numel()
    assert nnz > 8
    for capacity in (nnz + 100, nnz, nnz - 1, nnz // 2, 1):
        i2, v2, s2, count = cf.compress_attention_map(a, thr, capacity=capacity)
        assert count.value() == nnz and torch.equal(s2, seg)
        keep = min(capacity, nnz)
        assert i2.numel() == capacity and torch.equal(i2[:keep], idx[:keep]) and torch.equal(v2[:keep], val[:keep])
        # nothing past the capacity is touched: the C entry point on buffers with a guard zone
        gi = torch.full((capacity + 64,), -7, device=dev, dtype=torch.int64)
        gv = torch.full((capacity + 64,), 3.0, device=dev, dtype=BF16)
        flat = a.reshape(-1)
        L.call("hyc_sparse_write_bounded", flat.data_ptr(), flat.numel(), thr.data_ptr(), 0, seg.data_ptr(), capacity,
               gi.data_ptr(), gv.data_ptr(), L.stream_of(a))
        assert torch.equal(gi[:keep], idx[:keep]) and bool((gi[capacity:] == -7).all()) and bool((gv[capacity:] == 3.0).all())
    # the counting pass of the producer is reused in the same way
    i3, v3, s3, count = cf.compress_attention_map(a, thr, seg_offsets=seg, capacity=nnz + 5)
    assert count.value() == nnz and torch.equal(i3[:nnz], idx) and torch.equal(v3[:nnz], val) and s3 is seg
    # and the consumers read only what the segment offsets bound
    back = cf.restore_attention_map(i3, v3, s3, a.shape)
    assert torch.equal(back, cf.restore_attention_map(idx, val, seg, a.shape))


def test_threshold_is_compared_in_bf16_and_zeros_are_dropped(cf, dev):
    a = torch.tensor([1.0078125, 1.0, 0.0, -0.0, 0.5, float("nan"), 1.015625, 2.0] * 8, dtype=BF16)
    thr = torch.tensor(1.0058, dtype=torch.float32)        # rounds to bf16 1.0078125
    idx_ref, val_ref = O.softmax_compress(a, thr)
    idx, val, _ = cf.compress_attention_map(a.to(dev), thr.to(dev))
    assert torch.equal(idx.cpu(), idx_ref) and same_bits(val.cpu(), val_ref)
    assert idx_ref.numel() == 24                            # 1.015625, 2.0 - and NaN: NaN * False is NaN, which to_sparse keeps
    sp = (a * (a > thr)).flatten().to_sparse()              # the reference's own expression
    assert torch.equal(idx_ref, sp.indices()[0])
    assert torch.equal(val_ref.isnan(), sp.values().isnan()) and same_bits(torch.nan_to_num(val_ref), torch.nan_to_num(sp.values()))
    # negative threshold: zeros pass the comparison but to_sparse drops them
    thr = torch.tensor(-1.0)
    idx_ref, val_ref = O.softmax_compress(a, thr)
    idx, val, _ = cf.compress_attention_map(a.to(dev), -1.0)
    assert torch.equal(idx.cpu(), idx_ref) and same_bits(val.cpu(), val_ref)
    # nothing kept (a map without NaN) / only the NaNs kept
    idx, val, seg = cf.compress_attention_map(torch.nan_to_num(a).to(dev), 1e9)
    assert idx.numel() == 0 and (cf.restore_attention_map(idx, val, seg, a.shape) == 0).all()
    idx, val, seg = cf.compress_attention_map(a.to(dev), 1e9)
    assert idx.cpu().tolist() == list(range(5, 64, 8)) and bool(val.isnan().all())


def test_pack_softmax_base_dispatch(cf, dev):
    a = attention_map(seed=9).to(dev)
    sp, thr = cf.compression_pack_softmax_base(a, 0.05, 0, 5, {'outlier': None})
    sp2, thr2 = cf.compression_pack_softmax_base(a, 0.05, 5, 5, {'outlier': thr})
    assert thr2 is thr and torch.equal(sp.indices(), sp2.indices())
    nnz = sp.values().numel()
    assert nnz <= int(a.numel() * 0.05) + 1


@pytest.mark.parametrize("shape", [(2, 4, 128, 128), (1, 2, 100, 100), (1, 1, 1024, 1024), (1, 1, 8, 2048),
                                   (1, 1, 4, 4096), (1, 1, 3, 8192), (1, 2, 5, 36)])
def test_softmax_backward(sk, dev, shape):
    g = torch.Generator().manual_seed(shape[-1])
    y = torch.softmax(torch.randn(*shape, generator=g), dim=-1).to(BF16)
    gr = torch.randn(*shape, generator=g).to(BF16)
    o = sk.softmax_backward(y.to(dev), gr.to(dev))
    assert o.dtype == BF16 and o.shape == y.shape
    assert_close_bf16(o, O.softmax_bwd(y, gr), what="softmax_backward vs oracle")
    # independent: autograd of softmax in fp64 at the same y
    yf = y.double()
    ref = (gr.double() - (yf * gr.double()).sum(-1, keepdim=True)) * yf
    assert_close_bf16(o, ref, what="softmax_backward vs closed form")


@pytest.mark.parametrize("shape", [(1, 2, 16, 512), (2, 2, 8, 1024), (1, 1, 1024, 1024), (1, 3, 4, 2048), (1, 1, 5, 4096),
                                   (1, 2, 100, 100), (1, 1, 3, 8192), (1, 1, 7, 512),
                                   (1, 2, 1000, 1000), (2, 3, 50, 768), (1, 1, 33, 520), (1, 2, 9, 4088), (3, 1, 41, 24),
                                   (1, 1, 1, 8), (1, 2, 19, 3584), (1, 1, 600, 8)])
@pytest.mark.parametrize("ratio", [0.05, 0.0])
def test_softmax_backward_from_compressed(cf, sk, dev, shape, ratio):
    """restore + backward in one pass == the two separate kernels, bit for bit.  Row lengths 512 .. 4096
    that tile the map's 4096-element segments take the tuned kernel, other multiples of 8 up to 4096
    (and element counts that are not a multiple of 4096) the row-group kernel, the rest (100, 8192) the
    two-kernel route."""
    g = torch.Generator().manual_seed(shape[-1] + shape[-2])
    a = torch.softmax(torch.randn(*shape, generator=g) * 3, dim=-1).to(BF16)
    gr = torch.randn(*shape, generator=g).to(BF16)
    thr = cf.get_statistics_softmax(a.to(dev), ratio) if ratio else torch.tensor(2.0, device=dev)  # 2.0: keeps nothing
    idx, val, seg = cf.compress_attention_map(a.to(dev), thr)
    dense = cf.restore_attention_map(idx, val, seg, shape)
    want = sk.softmax_backward(dense, gr.to(dev))
    a_out, o = sk.softmax_backward_from_compressed(idx, val, seg, gr.to(dev))
    assert same_bits(a_out, dense) and same_bits(o, want)
    none, o2 = sk.softmax_backward_from_compressed(idx, val, seg, gr.to(dev), want_map=False)
    assert none is None and same_bits(o2, want)
    # the layers' grad_s / sqrt(head_dim) folded in: the bf16 result times the fp32 reciprocal, rounded again
    _, o3 = sk.softmax_backward_from_compressed(idx, val, seg, gr.to(dev), out_scale=1.0 / 128 ** 0.5)
    assert same_bits(o3, (want.float() * torch.tensor(1.0 / 128 ** 0.5, dtype=torch.float32)).to(BF16))
    # against the oracle, from the oracle's own compressed form
    i_o, v_o = O.softmax_compress(a, thr.cpu())
    ref = O.softmax_bwd(O.softmax_restore(i_o, v_o, a.shape), gr)
    if ratio:
        assert_close_bf16(o, ref, what="fused restore+bwd vs oracle")
    else:                                     # nothing kept: the gradient is exactly zero
        assert i_o.numel() == 0 and not bool(o.cpu().float().abs().max()) and not bool(ref.float().abs().max())


@pytest.mark.parametrize("shape", [(2, 4, 128, 128), (1, 2, 64, 1024), (2, 2, 24, 512), (1, 1, 8, 2048), (1, 1, 4, 4096),
                                   (1, 1, 3, 8192), (1, 3, 40, 40), (1, 2, 7, 1000)])
@pytest.mark.parametrize("masked", ["causal", "batch", None])
def test_softmax_forward(sk, dev, shape, masked):
    b, h, m, n = shape
    g = torch.Generator().manual_seed(n + m)
    s = (torch.randn(*shape, generator=g) * 20).to(BF16)
    mask = None
    if masked == "causal":                         # [1,1,S,n] additive, -inf above the diagonal band
        mask = torch.zeros(1, 1, m, n)
        mask[0, 0] = torch.full((m, n), float("-inf")).triu(n - m + 1)
        mask = mask.to(BF16)
    elif masked == "batch":                        # [B,1,S,n] with the dtype's minimum, as HF builds it
        mask = torch.where(torch.rand(b, 1, m, n, generator=g) < 0.3, torch.finfo(BF16).min, 0.0).to(BF16)
        mask[..., 0] = 0
    scale = 1.0 / 128 ** 0.5
    want = O.softmax_fwd(s, scale, mask)
    got = sk.softmax_forward(s.to(dev), scale, None if mask is None else mask.to(dev))
    assert got.dtype == BF16 and got.shape == s.shape
    assert_close_bf16(got, want, what="softmax_forward vs oracle")
    # independent: float64 softmax of the same bf16 logits; rows sum to one; masked entries are exactly zero
    t = (s.float() * torch.tensor(scale)).to(BF16)
    if mask is not None:
        t = t + mask
    ref = torch.softmax(t.double(), dim=-1)
    assert_close_bf16(got, ref, what="softmax_forward vs float64")
    assert (got.float().sum(-1).cpu() - 1).abs().max() < 2e-2
    if masked == "causal":
        assert not bool(got.cpu()[mask.expand_as(s) == float("-inf")].float().abs().max())
    # in place
    sd = s.to(dev)
    same = sk.softmax_forward(sd, scale, None if mask is None else mask.to(dev), inplace=True)
    assert same.data_ptr() == sd.data_ptr() and same_bits(same, got)


@pytest.mark.parametrize("shape", [(1, 2, 16, 512), (2, 2, 8, 1024), (1, 1, 6, 2048), (1, 3, 4, 4096), (1, 1, 3, 8192), (1, 2, 40, 40),
                                   (1, 2, 1000, 1000), (2, 3, 50, 768), (1, 1, 33, 520), (1, 2, 9, 4088), (3, 1, 41, 24),
                                   (1, 1, 1, 8), (1, 1, 7, 512), (1, 1, 600, 8)])
def test_softmax_forward_counts_for_the_compaction(cf, sk, dev, shape):
    """With a frozen threshold the forward pass hands the compaction its segment offsets: same
    compressed map as the separate counting pass (for row lengths that do not allow it the second
    value is None and the compaction counts by itself)."""
    g = torch.Generator().manual_seed(shape[-1])
    s = (torch.randn(*shape, generator=g) * 8).to(BF16).to(dev)
    a = sk.softmax_forward(s, 0.25)
    thr = cf.get_statistics_softmax(a, 0.05)
    a2, seg = sk.softmax_forward(s, 0.25, threshold=thr)
    assert same_bits(a2, a)
    idx, val, seg_ref = cf.compress_attention_map(a, thr)
    if shape[-1] % 8 == 0 and shape[-1] <= 4096:       # counted in the softmax pass itself
        assert seg is not None and torch.equal(seg, seg_ref)
    else:
        assert seg is None
    idx2, val2, seg2 = cf.compress_attention_map(a2, thr, seg)
    assert torch.equal(idx2, idx) and same_bits(val2, val) and torch.equal(seg2, seg_ref)


def test_full_size_config3_properties(cf, sk, dev):
    # benchmark configuration 3 at full size: [4,32,1024,1024], ratio 0.05
    g = torch.Generator(device=dev).manual_seed(1)
    s = torch.randn(4, 32, 1024, 1024, generator=g, device=dev, dtype=torch.float32) * (8 / 128 ** 0.5)
    s += torch.full((1024, 1024), float("-inf"), device=dev).triu(1)
    a = torch.softmax(s, dim=-1).to(BF16)
    del s
    n = a.numel()
    k = int(n * (1 - 0.05))
    assert k == 127506841
    thr = cf.get_statistics_softmax(a, 0.05)
    flat = a.flatten()
    # rank property of an exact k-th value: #(< thr) < k <= #(<= thr)
    below = int((flat < thr.to(BF16)).sum().item())
    upto = int((flat <= thr.to(BF16)).sum().item())
    assert below < k <= upto
    idx, val, seg = cf.compress_attention_map(a, thr)
    assert idx.numel() == n - upto and idx.numel() <= 6710887
    assert bool((idx[1:] > idx[:-1]).all())
    assert torch.equal(flat[idx], val)
    dense = cf.restore_attention_map(idx, val, seg, a.shape)
    assert torch.equal(dense, torch.where(a > thr.to(BF16), a, torch.zeros_like(a)))
    grad = torch.randn(a.shape, generator=g, device=dev, dtype=torch.float32).to(BF16)
    o = sk.softmax_backward(dense, grad)
    # row 700 of a few heads against the oracle
    rows = (slice(0, 4), slice(0, 2), slice(700, 704))
    assert_close_bf16(o[rows], O.softmax_bwd(dense[rows].cpu(), grad[rows].cpu()), what="softmax bwd rows")
    a2, o2 = sk.softmax_backward_from_compressed(idx, val, seg, grad)
    assert torch.equal(a2, dense) and torch.equal(o2, o)
