"""GPU parity of hyc_quant_pack / hyc_unpack_dequant (through the Python operator API and
the C ABI underneath) against the CPU oracle: packed codes, outlier values and the
dequantised tensor must be bit-exact."""
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
@pytest.mark.parametrize("shape", [(2, 64, 4096), (3, 37, 96), (1, 1, 32), (2, 130, 11008), (1, 5, 544)])
def test_quant_dequant_bit_exact(cf, dev, q_bit, shape):
    x = _rand(shape, seed=sum(shape) + q_bit, scale=2.0)
    s = O.scale_only_quant(x, q_bit)
    p_ref = O.compress(x, s, q_bit)
    p = cf.compression_quantization(x.to(dev), s.to(dev), q_bit)
    assert p.dtype == torch.uint8 and tuple(p.shape) == tuple(p_ref.shape)
    assert torch.equal(p.cpu(), p_ref)
    d = cf.decompression_dequantization(p, s.to(dev), q_bit)
    assert same_bits(d.cpu(), O.decompress(p_ref, s, q_bit))


@pytest.mark.parametrize("q_bit", QBITS)
def test_special_values_and_degenerate_scales(cf, dev, q_bit):
    x = _rand((2, 40, 128), seed=11, scale=3.0)
    x[1, 0, :8] = torch.tensor([0.0, -0.0, float("inf"), float("-inf"), float("nan"), 1e-40, 3e38, -3e38]).to(BF16)
    x[1, 1, 64:72] = torch.tensor([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 3.5, -3.5]).to(BF16)
    # signalling NaN bit patterns (0x7f81, 0xffa0): never produced by arithmetic, still code 0
    x[1, 2, :2] = torch.tensor([0x7f81, 0xffa0 - 0x10000], dtype=torch.int16).view(BF16)
    s = O.scale_only_quant(x, q_bit)
    s[0, 64:72] = 1.0                      # exact ties t = +-k.5
    s[0, 5] = 0.0                          # zero step (constant channel, scale-only path): x/0
    s[0, 6] = float("inf")
    s[0, 7] = 1e-38                        # subnormal in bf16 terms: reciprocal path must not be taken
    s[0, 9] = 3e38
    s[0, 10] = -0.25                       # negative step
    s[0, 11] = float("nan")
    p = cf.compression_quantization(x.to(dev), s.to(dev), q_bit)
    assert torch.equal(p.cpu(), O.compress(x, s, q_bit))


@pytest.mark.parametrize("q_bit", QBITS)
def test_every_bf16_pattern_against_a_spread_of_steps(cf, dev, q_bit):
    """All 65536 bf16 bit patterns (both NaN kinds, infinities, subnormals) as x, one per row, against
    64 steps per wave-width of columns: the reciprocal path's whole range, its edges, and steps outside
    it.  Covers on the device what the exhaustive CPU check covers for the shared arithmetic, plus the
    device-only clamp instruction."""
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(BF16)        # every pattern
    g = torch.Generator().manual_seed(q_bit)
    steps = torch.cat([
        torch.tensor([1e-18, 1.0001e-18, 9.9e17, 1e18, 1e-19, 2e18, 1.0, 0.5, 3.0, 0.1, 7.0, 1e-3, 0.0, -1.0,
                      float("inf"), 2 ** -126]),
        torch.exp(torch.rand(48, generator=g) * 80 - 40)]).to(BF16)                  # log-uniform 4e-18 .. 2e17
    x = pats[None, :, None].expand(1, 65536, 64).contiguous()
    p = cf.compression_quantization(x.to(dev), steps.to(dev), q_bit)
    want = O.compress(x, steps, q_bit)
    if not torch.equal(p.cpu(), want):
        bad = (O.unpack_codes(p.cpu(), q_bit) != O.unpack_codes(want, q_bit)).nonzero()
        r, c = bad[0, -2].item(), bad[0, -1].item()
        raise AssertionError(f"{bad.shape[0]} codes differ; first: x pattern {r:#06x}, step {steps[c].item()!r}")


@pytest.mark.parametrize("q_bit", QBITS)
def test_zero_point_path(cf, dev, q_bit):
    x = (_rand((2, 70, 256), seed=5).float() + 0.7).to(BF16)
    s, z8 = O.scale_zero_point(x, q_bit)
    # after calibration averaging the zero point is a non-integer float tensor
    z = (z8.float() + torch.linspace(-0.4, 0.4, 256)).to(BF16)
    p_ref = O.compress(x, s, q_bit, z)
    p = cf.compression_quantization_with_zero_point(x.to(dev), s.to(dev), z.to(dev), q_bit)
    assert torch.equal(p.cpu(), p_ref)
    d = cf.decompression_dequantization_with_zero_point(p, s.to(dev), z.to(dev), q_bit)
    assert same_bits(d.cpu(), O.decompress(p_ref, s, q_bit, z))


@pytest.mark.parametrize("q_bit", QBITS)
def test_config1_outlier_channels_round_trip(cf, dev, q_bit):
    # benchmark configuration 1 at full size: bf16 [2,512,4096], 0.5 % channels x50
    x, planted = activation_with_outlier_channels(seed=1234)
    idx, s = O.channel_stats(x, 0.005, q_bit)
    assert torch.equal(torch.sort(idx).values, planted)
    xo_ref, p_ref = O.compress_channel_base(x, s, idx, q_bit)
    xg = x.to(dev)
    xo, p = cf.outlier_subtraction_fuse_compression_quantization(xg, s.to(dev), idx.to(dev), q_bit)
    assert same_bits(xg.cpu(), x), "input must not be modified unless zero_input is set"
    assert same_bits(xo.cpu(), xo_ref)
    assert torch.equal(p.cpu(), p_ref)
    back = cf.outlier_addition_fuse_decompression_dequantization(p, s.to(dev), xo, idx.to(dev), q_bit)
    assert same_bits(back.cpu(), O.decompress_channel_base(p_ref, s, xo_ref, idx, q_bit))
    # reference side effect on request: the outlier columns of the input are zeroed
    xo2, p2 = cf.outlier_subtraction_fuse_compression_quantization(xg, s.to(dev), idx.to(dev), q_bit, zero_input=True)
    assert torch.equal(p2, p) and torch.equal(xo2, xo)
    xz = x.clone(); xz[:, :, idx] = 0
    assert same_bits(xg.cpu(), xz)


def test_outliers_many_unsorted_adjacent(cf, dev):
    # more than 64 outlier channels (two scan passes), unsorted, several inside one 8-column chunk
    x = _rand((2, 33, 2048), seed=21)
    g = torch.Generator().manual_seed(2)
    idx = torch.randperm(2048, generator=g)[:90]
    idx[:8] = torch.tensor([7, 0, 3, 1, 2, 6, 5, 4])
    idx = torch.unique(idx, sorted=False)[torch.randperm(torch.unique(idx).numel(), generator=g)]
    _, s = O.channel_stats(x, 0.0, 4, idx=idx)
    xo_ref, p_ref = O.compress_channel_base(x, s, idx, 4)
    xo, p = cf.outlier_subtraction_fuse_compression_quantization(x.to(dev), s.to(dev), idx.to(dev), 4)
    assert same_bits(xo.cpu(), xo_ref) and torch.equal(p.cpu(), p_ref)
    back = cf.outlier_addition_fuse_decompression_dequantization(p, s.to(dev), xo, idx.to(dev), 4)
    assert same_bits(back.cpu(), O.decompress_channel_base(p_ref, s, xo_ref, idx, 4))
    # the in-place zeroing with several outlier columns inside one lane's chunk
    xg = x.to(dev)
    xo2, p2 = cf.outlier_subtraction_fuse_compression_quantization(xg, s.to(dev), idx.to(dev), 4, zero_input=True)
    assert torch.equal(p2, p) and torch.equal(xo2, xo)
    xz = x.clone(); xz[:, :, idx] = 0
    assert same_bits(xg.cpu(), xz)


@pytest.mark.parametrize("q_bit", QBITS)
def test_head_layout_and_strided_rows(cf, dev, q_bit):
    # [B, H, S, D] input is read through its strides as [B, S, H*D]
    xh = _rand((2, 8, 50, 64), seed=9)
    s = O.scale_only_quant(xh, q_bit)
    p_ref = O.compress(xh, s, q_bit)
    p = cf.compression_quantization(xh.to(dev), s.to(dev), q_bit)
    assert torch.equal(p.cpu(), p_ref)
    d = cf.decompression_dequantization(p, s.to(dev), q_bit, is_head=True, num_heads=8)
    assert tuple(d.shape) == (2, 8, 50, 64)
    assert same_bits(d.cpu().contiguous(), O.decompress(p_ref, s, q_bit, is_head=True, num_heads=8).contiguous())
    # a transposed view of [B, S, H, D] storage (what hidden_to_head_shape yields)
    xv = _rand((2, 50, 8, 64), seed=10).to(dev).transpose(1, 2)
    s2 = O.scale_only_quant(xv.cpu(), q_bit)
    assert torch.equal(cf.compression_quantization(xv, s2.to(dev), q_bit).cpu(), O.compress(xv.cpu(), s2, q_bit))
    # every second row of a larger buffer
    big = _rand((2, 60, 256), seed=12).to(dev)
    view = big[:, ::2, :]
    s3 = O.scale_only_quant(view.cpu(), q_bit)
    assert torch.equal(cf.compression_quantization(view, s3.to(dev), q_bit).cpu(), O.compress(view.cpu(), s3, q_bit))


def test_empty_and_bad_arguments(cf, dev):
    s = torch.ones(1, 64, dtype=BF16, device=dev)
    q = cf.compression_quantization(torch.empty(0, 4, 64, dtype=BF16, device=dev), s, 4)
    assert tuple(q.shape) == (0, 4, 32)
    q = cf.compression_quantization(torch.empty(2, 0, 64, dtype=BF16, device=dev), s, 4)
    assert tuple(q.shape) == (2, 0, 32)
    with pytest.raises(ValueError):
        cf.compression_quantization(torch.zeros(1, 4, 48, dtype=BF16, device=dev), torch.ones(1, 48, dtype=BF16, device=dev), 4)
    with pytest.raises(ValueError):
        cf.compression_quantization(torch.zeros(1, 4, 64, dtype=BF16, device=dev), s, 3)
    with pytest.raises(RuntimeError):
        cf.compression_quantization(torch.zeros(1, 4, 64, dtype=BF16), torch.ones(1, 64, dtype=BF16), 4)


@pytest.mark.parametrize("q_bit", QBITS)
def test_full_size_properties_config2_shape(cf, dev, q_bit):
    # [4,1024,11008] (benchmark configuration 2's activation shape): properties that need no CPU pass
    g = torch.Generator(device=dev).manual_seed(q_bit)
    x = torch.randn(4, 1024, 11008, generator=g, device=dev, dtype=torch.float32).to(BF16)
    hi = x[0].max(dim=0, keepdim=True).values
    lo = x[0].min(dim=0, keepdim=True).values
    s = ((hi - lo) / (2 ** q_bit - 1)).to(BF16)
    p = cf.compression_quantization(x, s, q_bit)
    d = cf.decompression_dequantization(p, s, q_bit)
    # re-quantising the dequantised tensor reproduces the codes (idempotence)
    assert torch.equal(cf.compression_quantization(d, s, q_bit), p)
    # error bound off the clamp ends, evaluated on the GPU with torch
    err = (x.float() - d.float()).abs()
    inside = (x.float().abs() < (2 ** (q_bit - 1) - 1) * s.float())
    bound = 0.5 * s.float() + d.float().abs() * 2 ** -8
    assert bool((err <= bound)[inside].all())
    # a 64-row sample against the oracle
    rows = x[:, 100:116, :].cpu()
    assert torch.equal(p[:, 100:116, :].cpu(), O.compress(rows, s.cpu(), q_bit))


def test_wrappers_enqueue_on_torchs_current_stream(cf, dev):
    """Inside `with torch.cuda.stream(side)` the kernels go to `side`: its handle is what the wrappers
    hand to the library, and a result produced there is ordered after work queued on `side` before it."""
    from hyclora_amd import _lib
    side = torch.cuda.Stream(device=dev)
    x = torch.randn(2, 64, 512, device=dev).to(BF16)
    s = cf.get_statistics_only_quant(x, 4, 'per-channel')
    want = cf.compression_quantization(x, s, 4)
    assert _lib.stream_of(x) == torch.cuda.current_stream(dev).cuda_stream
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        assert _lib.stream_of(x) == side.cuda_stream != 0
        y = torch.zeros_like(x)
        torch.cuda._sleep(20_000_000)                  # keeps `side` busy while the next two calls are queued
        y.copy_(x)                                     # on `side`, after the sleep
        got = cf.compression_quantization(y, s, 4)     # must wait for that copy: same stream
    side.synchronize()
    assert torch.equal(got, want)
