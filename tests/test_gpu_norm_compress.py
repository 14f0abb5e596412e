"""GPU parity of the fused RMSNorm-forward + compression kernel: its outputs must equal, bit for
bit, those of the separate operators (which are themselves checked against the oracle), and the
oracle's compressed forms directly."""
import pytest
import torch

from helpers import BF16, activation_with_outlier_channels, assert_close_bf16, same_bits
from oracle import hyc_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import compress_function, rmsnorm_kernels

    class Ops:
        cf = compress_function
        norm = rmsnorm_kernels
    return Ops


@pytest.mark.parametrize("q_bit", [2, 4, 8])
@pytest.mark.parametrize("shape", [(2, 37, 4096), (1, 5, 512), (3, 4, 96), (1, 9, 8192), (2, 3, 1024 + 32),
                                   # whole 512-column slabs and an even row count: the
                                   # column-slab kernel (1, 2, 8, 10 and 16 waves per workgroup)
                                   (2, 34, 4096), (1, 8, 512), (4, 1, 1024), (1, 20, 5120), (1, 12, 8192)])
@pytest.mark.parametrize("wdtype", [BF16, torch.float32])
def test_fused_equals_separate_operators(ops, dev, q_bit, shape, wdtype):
    x, planted = activation_with_outlier_channels(seed=shape[-1] + q_bit, shape=shape, frac=0.01)
    g = torch.Generator().manual_seed(1)
    w = (1 + 0.1 * torch.randn(shape[-1], generator=g)).to(wdtype)
    xd, wd = x.to(dev), w.to(dev)
    # frozen statistics, as after calibration
    idx, s_x = ops.cf.get_statistics_channel_base(xd, 0.01, q_bit, 'per-channel')
    y_ref, _, rstd_ref, _, _ = ops.norm.rmsnorm_forward(xd, wd, 1e-5)
    s_y = ops.cf.get_statistics_only_quant(y_ref, q_bit, 'per-channel')
    xo_ref, qx_ref = ops.cf.outlier_subtraction_fuse_compression_quantization(xd, s_x, idx, q_bit)
    qy_ref = ops.cf.compression_quantization(y_ref, s_y, q_bit)

    y, rstd, q_y, q_x, x_out = ops.norm.rmsnorm_forward_compress(xd, wd, 1e-5, q_bit, scale_y=s_y, scale_x=s_x, outlier_idx=idx)
    assert same_bits(y, y_ref) and torch.equal(rstd, rstd_ref)
    assert torch.equal(q_y, qy_ref) and torch.equal(q_x, qx_ref) and same_bits(x_out, xo_ref)
    # against the oracle's own forms of the two compressions
    xo_o, qx_o = O.compress_channel_base(x, s_x.cpu(), idx.cpu(), q_bit)
    assert torch.equal(q_x.cpu(), qx_o) and same_bits(x_out.cpu(), xo_o)
    assert torch.equal(q_y.cpu(), O.compress(y_ref.cpu(), s_y.cpu(), q_bit))
    y_o, _ = O.rmsnorm_fwd(x, w, 1e-5)
    assert_close_bf16(y, y_o, what="fused rmsnorm y vs oracle")
    # parts can be switched off
    y2, _, q_y2, q_x2, xo2 = ops.norm.rmsnorm_forward_compress(xd, wd, 1e-5, q_bit, scale_y=s_y)
    assert same_bits(y2, y_ref) and torch.equal(q_y2, qy_ref) and q_x2 is None and xo2 is None
    y3, _, q_y3, q_x3, xo3 = ops.norm.rmsnorm_forward_compress(xd, wd, 1e-5, q_bit, scale_x=s_x)   # no outlier channels
    assert q_y3 is None and xo3.shape[-1] == 0
    assert torch.equal(q_x3, ops.cf.compression_quantization(xd, s_x, q_bit))


@pytest.mark.parametrize("q_bit", [2, 4, 8])
@pytest.mark.parametrize("shape", [(1, 72, 4096), (1, 40, 8192), (2, 10, 1536)])
def test_both_kernel_forms_give_the_same_bits(ops, dev, q_bit, shape):
    # the row-per-wave kernel and the column-slab kernel, the latter at several strip heights
    # (one step per strip, two, several, a short last strip)
    from hyclora_amd import _lib
    x, _ = activation_with_outlier_channels(seed=3 + q_bit, shape=shape, frac=0.01)
    w = (1 + 0.1 * torch.randn(shape[-1], generator=torch.Generator().manual_seed(2))).to(BF16)
    xd, wd = x.to(dev), w.to(dev)
    idx, s_x = ops.cf.get_statistics_channel_base(xd, 0.01, q_bit, 'per-channel')
    y_ref = ops.norm.rmsnorm_forward(xd, wd, 1e-5)[0]
    s_y = ops.cf.get_statistics_only_quant(y_ref, q_bit, 'per-channel')
    run = lambda: ops.norm.rmsnorm_forward_compress(xd, wd, 1e-5, q_bit, scale_y=s_y, scale_x=s_x, outlier_idx=idx)
    try:
        _lib.set_tuning("norm_compress_slab", 0)
        base = run()
        _lib.set_tuning("norm_compress_slab", 1)
        for rows in (0, 2, 4, 6, 16, 128):             # 0: the library's own choice
            _lib.set_tuning("norm_compress_rows_per_group", rows)
            for got, want in zip(run(), base):
                assert torch.equal(got.view(torch.uint8) if got.dtype == BF16 else got,
                                   want.view(torch.uint8) if want.dtype == BF16 else want), f"strip height {rows}"
    finally:
        _lib.set_tuning("norm_compress_slab", 1)
        _lib.set_tuning("norm_compress_rows_per_group", 0)


@pytest.mark.parametrize("q_bit", [2, 4, 8])
@pytest.mark.parametrize("shape", [(2, 34, 4096), (1, 8, 512), (4, 1, 1024), (1, 20, 5120), (1, 12, 8192)])
@pytest.mark.parametrize("wdtype", [BF16, torch.float32])
def test_backward_from_codes_equals_restore_then_backward(ops, dev, q_bit, shape, wdtype):
    from hyclora_amd import _lib
    x, _ = activation_with_outlier_channels(seed=11 + q_bit, shape=shape, frac=0.01)
    g = torch.Generator().manual_seed(5)
    w = (1 + 0.1 * torch.randn(shape[-1], generator=g)).to(wdtype).to(dev)
    dy = torch.randn(*shape, generator=g).to(BF16).to(dev)
    res = torch.randn(*shape, generator=g).to(BF16).to(dev)
    xd = x.to(dev)
    idx, s_x = ops.cf.get_statistics_channel_base(xd, 0.01, q_bit, 'per-channel')
    rstd = ops.norm.rmsnorm_forward(xd, w, 1e-5)[2]
    xo, q_x = ops.cf.outlier_subtraction_fuse_compression_quantization(xd.clone(), s_x, idx, q_bit)
    restored = ops.cf.outlier_addition_fuse_decompression_dequantization(q_x, s_x, xo, idx, q_bit)
    want = ops.norm._backward(dy, restored, w, rstd, want_dw=False)[0]
    want_res = ops.norm._backward(dy, restored, w, rstd, want_dw=False, residual=res)[0]
    try:
        for rows in (0, 2, 6, 64):
            _lib.set_tuning("norm_compress_rows_per_group", rows)
            got = ops.norm.rmsnorm_backward_from_codes(dy, q_x, s_x, xo, idx, q_bit, w, rstd)
            got_res = ops.norm.rmsnorm_backward_from_codes(dy, q_x, s_x, xo, idx, q_bit, w, rstd, residual=res)
            assert same_bits(got, want) and same_bits(got_res, want_res), f"strip height {rows}"
    finally:
        _lib.set_tuning("norm_compress_rows_per_group", 0)
    # against the oracle's formula on the oracle's restored input
    x_o = O.decompress_channel_base(q_x.cpu(), s_x.cpu(), xo.cpu(), idx.cpu(), q_bit)
    dx_o, _ = O.rmsnorm_bwd(dy.cpu(), x_o, w.cpu(), rstd.cpu())
    assert_close_bf16(got, dx_o, what="backward from codes vs oracle")
    # no outlier channels at all
    q_plain = ops.cf.compression_quantization(xd, s_x, q_bit)
    plain = ops.cf.decompression_dequantization(q_plain, s_x, q_bit)
    got0 = ops.norm.rmsnorm_backward_from_codes(dy, q_plain, s_x, None, None, q_bit, w, rstd, residual=res)
    assert same_bits(got0, ops.norm._backward(dy, plain, w, rstd, want_dw=False, residual=res)[0])


def test_backward_from_codes_many_outliers_in_one_chunk_and_errors(ops, dev):
    # more than two outlier columns inside one lane's 8 columns: the third and later ones are read
    # when they are used instead of with the row
    shape, q_bit = (1, 6, 512), 4
    g = torch.Generator().manual_seed(9)
    x = torch.randn(*shape, generator=g).to(BF16).to(dev)
    idx = torch.tensor([16, 17, 19, 22, 23, 300, 8], device=dev)
    s_x = ops.cf.get_statistics_only_quant(x, q_bit, 'per-channel')
    w = torch.ones(512, dtype=BF16, device=dev)
    dy = torch.randn(*shape, generator=g).to(BF16).to(dev)
    rstd = ops.norm.rmsnorm_forward(x, w, 1e-5)[2]
    xo, q_x = ops.cf.outlier_subtraction_fuse_compression_quantization(x.clone(), s_x, idx, q_bit)
    restored = ops.cf.outlier_addition_fuse_decompression_dequantization(q_x, s_x, xo, idx, q_bit)
    got = ops.norm.rmsnorm_backward_from_codes(dy, q_x, s_x, xo, idx, q_bit, w, rstd)
    assert same_bits(got, ops.norm._backward(dy, restored, w, rstd, want_dw=False)[0])
    with pytest.raises(NotImplementedError):      # odd row count
        ops.norm.rmsnorm_backward_from_codes(dy[:, :5], q_x[:, :5], s_x, xo[:, :5], idx, q_bit, w, rstd[:5])
    with pytest.raises(ValueError):               # codes of another shape
        ops.norm.rmsnorm_backward_from_codes(dy, q_x[:, :4], s_x, xo, idx, q_bit, w, rstd)
    assert not ops.norm.backward_from_codes_supported(dy, 512, True)
    assert not ops.norm.backward_from_codes_supported(dy[..., :96], 96, False)


def test_outlier_table_and_errors(ops, dev):
    idx = torch.tensor([5, 0, 31, 7], device=dev)
    t = ops.norm.outlier_table(idx, 32).cpu().tolist()
    want = [0] * 32
    want[5], want[0], want[31], want[7] = 1, 2, 3, 4
    assert t == want
    x = torch.zeros(1, 2, 40, device=dev, dtype=BF16)
    w = torch.ones(40, device=dev, dtype=BF16)
    with pytest.raises(ValueError):
        ops.norm.rmsnorm_forward_compress(x, w, 1e-5, 4, scale_y=torch.ones(40, device=dev, dtype=BF16))   # N % 32
    x = torch.zeros(1, 2, 64, device=dev, dtype=BF16)
    w = torch.ones(64, device=dev, dtype=BF16)
    with pytest.raises(ValueError):
        ops.norm.rmsnorm_forward_compress(x, w, 1e-5, 3, scale_y=torch.ones(64, device=dev, dtype=BF16))
    with pytest.raises(ValueError):
        ops.norm.rmsnorm_forward_compress(x, w, 1e-5, 4, scale_y=torch.ones(32, device=dev, dtype=BF16))


@pytest.mark.parametrize("shape", [(2, 34, 4096), (1, 8, 512), (4, 1, 1024), (1, 20, 5120), (1, 12, 8192), (2, 513, 2048)])
@pytest.mark.parametrize("ranks", [(16, 16, 16), (16, 16), (8,), (64,), (32, 4), (12, 16, 16, 16)])
def test_lora_a_contraction_in_the_norm_pass(ops, dev, shape, ranks):
    """y @ lora_A^T for every adapter fed by the norm's output, formed inside the norm kernel
    (compute_utils.py:22 via ...full_fuse.py:111-117, :218-226): against the float64 product of the
    kernel's own y rounded once (the oracle's lora_products: >= 99 % of the values the same bits, all
    within tolerance), with every other output of the call unchanged bit for bit; row counts that do
    not fill the last 8-row tile, ranks that do not fill a 16-row block, 1 to 16 waves per workgroup."""
    q_bit = 4
    x, _ = activation_with_outlier_channels(seed=shape[1] + len(ranks), shape=shape, frac=0.01)
    g = torch.Generator().manual_seed(7)
    n = shape[-1]
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(BF16)
    weights = [(torch.randn(r, n, generator=g) / n ** 0.5).to(BF16).to(dev) for r in ranks]     # lora_A.weight: [R, N]
    views = [a.t() for a in weights]                                                             # what the layers pass: [N, R]
    xd, wd = x.to(dev), w.to(dev)
    idx, s_x = ops.cf.get_statistics_channel_base(xd, 0.01, q_bit, 'per-channel')
    y_ref, _, _, _, _ = ops.norm.rmsnorm_forward(xd, wd, 1e-5)
    s_y = ops.cf.get_statistics_only_quant(y_ref, q_bit, 'per-channel')
    assert ops.norm.lora_a_supported(xd, wd, views)
    base = ops.norm.rmsnorm_forward_compress(xd, wd, 1e-5, q_bit, scale_y=s_y, scale_x=s_x, outlier_idx=idx)
    got = ops.norm.rmsnorm_forward_compress(xd, wd, 1e-5, q_bit, scale_y=s_y, scale_x=s_x, outlier_idx=idx, lora_a=views)
    for a, b in zip(base, got[:5]):
        assert torch.equal(a, b), "an output of the norm changes when the contraction is switched on"
    plain = ops.norm.rmsnorm_forward_compress(xd, wd, 1e-5, q_bit, lora_a=views)                 # no compressed copies
    assert torch.equal(plain[0], base[0]) and torch.equal(plain[1], base[1]) and plain[2] is None and plain[3] is None
    y = got[0].cpu()
    for r, a, xa, xa2 in zip(ranks, weights, got[5], plain[5]):
        assert xa.shape == (*shape[:2], r) and xa.dtype == BF16 and xa.is_contiguous()
        assert torch.equal(xa, xa2)
        _, want = O.lora_products(y, v=a.cpu())
        assert_close_bf16(xa, want, what=f"rank {r} x@A vs float64 product")
        same = (xa.cpu().view(torch.int16) == want.view(torch.int16)).float().mean().item()
        assert same >= 0.99, f"rank {r}: only {same:.4f} of the values are the same bits as the float64 product"
        assert_close_bf16(xa, got[0] @ a.t(), what=f"rank {r} x@A vs the library GEMM")
    # repeated calls give the same bits (fixed summation order, no atomics)
    again = ops.norm.rmsnorm_forward_compress(xd, wd, 1e-5, q_bit, scale_y=s_y, scale_x=s_x, outlier_idx=idx, lora_a=views)
    for xa, xb in zip(got[5], again[5]):
        assert torch.equal(xa, xb)


def test_lora_a_contraction_limits(ops, dev):
    z = lambda *sh: torch.zeros(*sh, dtype=BF16, device=dev)
    w = torch.ones(1024, dtype=BF16, device=dev)
    ok = [z(1024, 16)]
    assert ops.norm.lora_a_supported(z(2, 4, 1024), w, ok)
    assert not ops.norm.lora_a_supported(z(2, 4, 1024), w.float(), ok)            # fp32 norm weight
    assert not ops.norm.lora_a_supported(z(1, 3, 1024), w, ok)                     # odd row count
    assert not ops.norm.lora_a_supported(z(2, 4, 1024 + 32), torch.ones(1056, dtype=BF16, device=dev), [z(1056, 16)])
    assert not ops.norm.lora_a_supported(z(2, 4, 1024), w, [z(1024, 16)] * 5)      # five blocks
    assert not ops.norm.lora_a_supported(z(2, 4, 1024), w, [z(1024, 48), z(1024, 32)])
    assert not ops.norm.lora_a_supported(z(2, 4, 1024), w, [z(512, 16)])           # adapter of another width
    with pytest.raises(NotImplementedError):
        ops.norm.rmsnorm_forward_compress(z(1, 3, 1024), w, 1e-5, 4, lora_a=ok)


@pytest.mark.parametrize("shape", [(1, 8, 512), (2, 34, 4096)])
def test_a_table_of_a_longer_list_does_not_reach_past_the_outlier_buffer(ops, dev, shape):
    """The kernels index x_outlier[row * k + position] with the positions of the caller's table.  A table built
    for a longer channel list than the one passed (k entries) has positions past k: those channels are treated
    as ordinary ones - the result is that of the list's first k channels - instead of being written or read
    past the [rows, k] buffer."""
    q_bit, n = 4, shape[-1]
    g = torch.Generator().manual_seed(3)
    x = torch.randn(*shape, generator=g).to(BF16).to(dev)
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(BF16).to(dev)
    dy = torch.randn(*shape, generator=g).to(BF16).to(dev)
    longer = torch.randperm(n, generator=g)[:12].to(dev)
    short = longer[:5].contiguous()
    s_x = ops.cf.get_statistics_only_quant(x, q_bit, 'per-channel')
    s_y = ops.cf.get_statistics_only_quant(ops.norm.rmsnorm_forward(x, w, 1e-5)[0], q_bit, 'per-channel')
    t_long, t_short = ops.norm.outlier_table(longer, n), ops.norm.outlier_table(short, n)
    want = ops.norm.rmsnorm_forward_compress(x, w, 1e-5, q_bit, scale_y=s_y, scale_x=s_x, outlier_idx=short, table=t_short)
    got = ops.norm.rmsnorm_forward_compress(x, w, 1e-5, q_bit, scale_y=s_y, scale_x=s_x, outlier_idx=short, table=t_long)
    for a, b in zip(want[:5], got[:5]):
        assert torch.equal(a, b)
    y, rstd, q_y, q_x, xo = want[:5]
    assert xo.shape[-1] == 5
    d_want = ops.norm.rmsnorm_backward_from_codes(dy, q_x, s_x, xo, short, q_bit, w, rstd, table=t_short)
    d_got = ops.norm.rmsnorm_backward_from_codes(dy, q_x, s_x, xo, short, q_bit, w, rstd, table=t_long)
    assert torch.equal(d_want, d_got)
