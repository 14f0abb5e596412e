"""GPU checks of the element-wise backward operators and RMSNorm against the CPU oracle
(bf16 tolerance: max rel err <= 1e-2, cosine >= 0.9999) and against torch.autograd of the
fp32 composite."""
import pytest
import torch
import torch.nn.functional as F

from helpers import BF16, assert_close_bf16
from oracle import hyc_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import gelu_kernels, rmsnorm_kernels, rmsnorm_updatable_kernels, silu_kernels

    class Ops:
        silu = silu_kernels
        gelu = gelu_kernels
        norm = rmsnorm_kernels
        normu = rmsnorm_updatable_kernels
    return Ops


def _pair(shape, seed, scale=2.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(BF16), torch.randn(*shape, generator=g).to(BF16)


SHAPES = [(2, 64, 11008), (1, 7, 96), (3, 5, 41), (1, 1, 8)]


@pytest.mark.parametrize("shape", SHAPES)
def test_silu_backward(ops, dev, shape):
    x, g = _pair(shape, 1)
    o = ops.silu.silu_backward(x.to(dev), g.to(dev))
    assert_close_bf16(o, O.silu_bwd(x, g), what="silu_backward vs oracle")
    xf = x.float().requires_grad_()
    F.silu(xf).backward(g.float())
    # five bf16 roundings in a row (2^-8 each) separate the reference's expression from fp32 autograd
    assert_close_bf16(o, xf.grad, rel_tol=2e-2, what="silu_backward vs autograd")


@pytest.mark.parametrize("shape", SHAPES)
def test_silu_hadamard(ops, dev, shape):
    x1, x2 = _pair(shape, 2)
    o = ops.silu.silu_hadamard(x1.to(dev), x2.to(dev))
    assert_close_bf16(o, O.silu_mul(x1, x2), what="silu_hadamard vs oracle")
    assert_close_bf16(o, F.silu(x1.float()) * x2.float(), what="silu_hadamard vs torch")


@pytest.mark.parametrize("shape", SHAPES)
def test_silu_once_hadamard(ops, dev, shape):
    """u * F.silu(x) as the reference's backward recomputes the gated product
    (models/llama/fused_llama_layer_intra_inter.py:362,370): silu rounded once, then the product."""
    x, u = _pair(shape, 6)
    o = ops.silu.silu_once_hadamard(x.to(dev), u.to(dev))
    want = u * F.silu(x)                     # CPU torch, bf16 tensors
    assert_close_bf16(o, want, rel_tol=2.0 ** -7, what="silu_once_hadamard vs u * F.silu(x)")   # one bf16 step
    mismatched = (o.cpu() != want).float().mean().item()
    assert mismatched < 0.02, f"{mismatched:.3%} of the elements differ from torch's bits"
    assert_close_bf16(o, F.silu(x.float()) * u.float(), what="silu_once_hadamard vs fp32")


@pytest.mark.parametrize("shape", SHAPES)
def test_silu_hadamard_backward(ops, dev, shape):
    x, u = _pair(shape, 4)
    g = _pair(shape, 5)[0]
    gx, gu = ops.silu.silu_hadamard_backward(x.to(dev), u.to(dev), g.to(dev))
    # the composition it stands for, from the operators already checked: bit for bit
    gd, ud, xd = g.to(dev), u.to(dev), x.to(dev)
    assert torch.equal(gx, ops.silu.silu_backward(xd, gd * ud))
    assert torch.equal(gu, gd * ops.silu.silu_once_hadamard(xd, torch.ones_like(xd)))
    # F.silu itself (fp32 inside, one rounding): the kernel's sigmoid may differ from torch's in the last fp32
    # bit, which shows as a last bf16 bit on a few elements in a thousand
    assert_close_bf16(gu, gd * F.silu(xd), rel_tol=2.0 ** -7, what="grad_u vs g * F.silu(x)")   # one bf16 step
    gx_o, gu_o = O.silu_mul_bwd(x, u, g)
    assert_close_bf16(gx, gx_o, what="grad_x vs oracle")
    assert_close_bf16(gu, gu_o, what="grad_u vs oracle")
    xf, uf = x.float().requires_grad_(), u.float().requires_grad_()
    (F.silu(xf) * uf).backward(g.float())
    assert_close_bf16(gx, xf.grad, rel_tol=2e-2, what="grad_x vs autograd")
    assert_close_bf16(gu, uf.grad, what="grad_u vs autograd")


@pytest.mark.parametrize("shape", SHAPES)
def test_gelu_backward(ops, dev, shape):
    x, g = _pair(shape, 3)
    o = ops.gelu.gelu_backward(x.to(dev), g.to(dev))
    assert_close_bf16(o, O.gelu_bwd(x, g), what="gelu_backward vs oracle")
    xf = x.float().requires_grad_()
    F.gelu(xf, approximate="tanh").backward(g.float())
    assert_close_bf16(o, xf.grad, what="gelu_backward vs autograd of tanh-GELU")


def test_elementwise_extremes(ops, dev):
    # saturated sigmoid / tanh must give the limits 0 and 1, not NaN.  (The GELU formula itself
    # overflows to inf*0 beyond |x| ~ 1e19, in the reference as well, so it is probed up to 1e4.)
    for top, fn, ref in ((3e38, ops.silu.silu_backward, O.silu_bwd), (1e4, ops.gelu.gelu_backward, O.gelu_bwd)):
        x = torch.tensor([0.0, -0.0, 50.0, -50.0, 1e4, -1e4, top, -top] * 2, dtype=BF16).reshape(1, 2, 8)
        g = torch.ones_like(x)
        o = fn(x.to(dev), g.to(dev)).cpu().float()
        r = ref(x, g).float()
        assert torch.isfinite(o).all() and torch.allclose(o, r, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("n", [4096, 512, 96, 1024, 8192, 16384, 2048 + 64, 3072, 5120, 6144, 7168])
@pytest.mark.parametrize("wdtype", [BF16, torch.float32])
def test_rmsnorm_forward(ops, dev, n, wdtype):
    g = torch.Generator().manual_seed(n)
    x = (torch.randn(2, 33, n, generator=g) * 3).to(BF16)
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(wdtype)
    y, mean, rstd, block, warps = ops.norm.rmsnorm_forward(x.to(dev), w.to(dev), 1e-5)
    y_ref, rstd_ref = O.rmsnorm_fwd(x, w, 1e-5)
    assert y.shape == x.shape and y.dtype == BF16 and rstd.shape == (66,) and rstd.dtype == torch.float32
    assert block >= n and 1 <= warps <= 8 and mean.shape == (66,)
    assert torch.allclose(rstd.cpu(), rstd_ref, rtol=1e-5, atol=0)
    assert_close_bf16(y, y_ref, what="rmsnorm_forward vs oracle")
    # independent: the textbook formula in fp64
    xd = x.double()
    ref = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-5) * w.double()
    assert_close_bf16(y, ref, what="rmsnorm_forward vs fp64 formula")


@pytest.mark.parametrize("n", [4096, 512, 96, 1024, 8192, 3072, 5120, 7168, 6144 + 8])   # beyond 4096: even row counts take the column-slab kernel
@pytest.mark.parametrize("rows", [(2, 33), (1, 1), (4, 300)])
def test_rmsnorm_backward(ops, dev, n, rows):
    g = torch.Generator().manual_seed(n + rows[1])
    x = (torch.randn(*rows, n, generator=g) * 2).to(BF16)
    dy = torch.randn(*rows, n, generator=g).to(BF16)
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(BF16)
    xg, dyg, wg = x.to(dev), dy.to(dev), w.to(dev)
    _, mean, rstd, block, warps = ops.norm.rmsnorm_forward(xg, wg, 1e-5)
    dx, none = ops.norm.rmsnorm_backward(dyg, xg, wg, mean, rstd, True, 1e-5, warps, block)
    assert none is None
    dx_ref, dw_ref = O.rmsnorm_bwd(dy, x, w, rstd.cpu())
    assert_close_bf16(dx, dx_ref, what="rmsnorm_backward dx vs oracle")
    dx2, dw = ops.normu.rmsnorm_backward(dyg, xg, wg, mean, rstd, 1e-5, warps, block)
    assert torch.equal(dx2, dx)
    assert dw.dtype == w.dtype and dw.shape == (n,)
    assert_close_bf16(dw, dw_ref, what="rmsnorm_backward dw vs oracle")
    assert ops.norm.rmsnorm_backward(dyg, xg, wg, mean, rstd, False, 1e-5, warps, block) == (None, None)
    # the residual connection's gradient added in the same pass: the bits of dx + residual
    res = torch.randn(*rows, n, generator=g).to(BF16).to(dev)
    dx3, _ = ops.norm.rmsnorm_backward(dyg, xg, wg, mean, rstd, True, 1e-5, warps, block, residual=res)
    assert torch.equal(dx3, dx + res)
    dx4, dw4 = ops.norm._backward(dyg, xg, wg, rstd, want_dw=True, residual=res)
    assert torch.equal(dx4, dx3) and torch.equal(dw4, dw)
    with pytest.raises(ValueError):
        ops.norm.rmsnorm_backward(dyg, xg, wg, mean, rstd, True, 1e-5, warps, block, residual=res[..., :8])
    # independent check of dw and of dx's x^-dependent part: autograd of true RMSNorm, to
    # which the reference formula adds only the -mean(w*dy)*rstd term
    xf = x.double().requires_grad_()
    wf = w.double().requires_grad_()
    yf = xf / torch.sqrt((xf * xf).mean(-1, keepdim=True) + 1e-5) * wf
    yf.backward(dy.double())
    assert_close_bf16(dw, wf.grad, what="dw vs autograd")
    c2 = (w.double() * dy.double()).mean(-1, keepdim=True) * rstd.cpu().double().reshape(*rows, 1)
    assert_close_bf16(dx, xf.grad - c2, what="dx vs autograd minus the LayerNorm mean term")


@pytest.mark.parametrize("n,rows", [(512, 7), (4096, 64), (96, 33), (8192, 4)])
def test_rmsnorm_backward_mean_term_is_layernorms(ops, dev, n, rows):
    """The c2 = mean(w*dy) term of the reference's formula (rmsnorm_kernels.py:96-98) is not part of a
    true RMSNorm's derivative.  On rows whose mean is exactly zero the formula IS LayerNorm's backward
    (layernorm_kernels.py:92-104), so there the kernel must agree with autograd of F.layer_norm - an
    independent library routine - and must differ from autograd of RMSNorm by c2 * rstd."""
    from test_oracle_norm import layernorm_autograd_dx, rmsnorm_autograd_dx, zero_mean_case
    x, dy, w = zero_mean_case(n, rows, seed=n + rows)
    xg, dyg, wg = x.to(dev), dy.to(dev), w.to(dev)
    y, mean, rstd, block, warps = ops.norm.rmsnorm_forward(xg, wg, 1e-5)
    assert_close_bf16(y, F.layer_norm(x.double(), (n,), w.double(), None, 1e-5), what="rmsnorm_forward vs layer_norm")
    ln_dx = layernorm_autograd_dx(x, dy, w)
    rms_dx = rmsnorm_autograd_dx(x, dy, w)
    c2 = (w.double() * dy.double()).mean(-1, keepdim=True) * rstd.cpu().double().reshape(-1, 1)
    dx, _ = ops.norm.rmsnorm_backward(dyg, xg, wg, mean, rstd, True, 1e-5, warps, block)
    dxu, dw = ops.normu.rmsnorm_backward(dyg, xg, wg, mean, rstd, 1e-5, warps, block)
    res = torch.zeros_like(dyg)
    dxr, _ = ops.norm.rmsnorm_backward(dyg, xg, wg, mean, rstd, True, 1e-5, warps, block, residual=res)
    for got, what in ((dx, "rmsnorm_backward"), (dxu, "updatable rmsnorm_backward"), (dxr, "rmsnorm_backward + residual")):
        assert_close_bf16(got, ln_dx, what=what + " vs autograd of layer_norm")
        assert_close_bf16(got, rms_dx - c2, what=what + ": difference to true RMSNorm is c2 * rstd")
        assert (got.cpu().double() - rms_dx).abs().max() / rms_dx.abs().max() > 5e-2, "case does not exercise the mean term"
    assert_close_bf16(dx, O.rmsnorm_bwd(dy, x, w, rstd.cpu())[0], what="rmsnorm_backward vs oracle")
    wd = w.double().requires_grad_()
    F.layer_norm(x.double(), (n,), wd, None, 1e-5).backward(dy.double())
    assert_close_bf16(dw, wd.grad, what="dw vs autograd of layer_norm")


def test_rmsnorm_backward_from_codes_mean_term(ops, dev):
    """The same pin for the backward that reads the norm's input from its compressed copy.  The rows
    (v | -v) lie on the grid k/16, |k| <= 127, and every channel has the step 1/16, so the 8-bit
    codes decode to the rows themselves and these still sum to exactly zero."""
    from hyclora_amd.operators import compress_function as cf
    from test_oracle_norm import layernorm_autograd_dx
    n, rows = 1024, 16
    g = torch.Generator().manual_seed(11)
    v = (torch.randn(rows, n // 2, generator=g) * 32).round().clamp(-127, 127) / 16
    x = torch.cat([v, -v], dim=-1)[:, torch.randperm(n, generator=g)].to(BF16).contiguous()
    dy = (torch.randn(rows, n, generator=g) + 0.5).to(BF16)
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(BF16)
    x3, dy3, wg = x.reshape(1, rows, n).to(dev), dy.reshape(1, rows, n).to(dev), w.to(dev)
    scale = torch.full((1, n), 1 / 16, dtype=BF16, device=dev)
    q = cf.compression_quantization(x3, scale, 8)
    assert torch.equal(cf.decompression_dequantization(q, scale, 8), x3), "the codes do not decode to the rows"
    _, _, rstd, _, _ = ops.norm.rmsnorm_forward(x3, wg, 1e-5)
    dx = ops.norm.rmsnorm_backward_from_codes(dy3, q, scale, None, None, 8, wg, rstd)
    assert_close_bf16(dx.reshape(rows, n), layernorm_autograd_dx(x, dy, w),
                      what="rmsnorm_backward_from_codes vs autograd of layer_norm")
    dense, _ = ops.norm.rmsnorm_backward(dy3, x3, wg, None, rstd, True, 1e-5, 0, 0)
    assert torch.equal(dx, dense), "from-codes backward and dense backward differ"


def test_rmsnorm_errors(ops, dev):
    with pytest.raises(RuntimeError):
        ops.norm.rmsnorm_forward(torch.zeros(1, 1, 32776, dtype=BF16, device=dev), torch.ones(32776, dtype=BF16, device=dev), 1e-5)
    with pytest.raises(ValueError):
        ops.norm.rmsnorm_forward(torch.zeros(1, 1, 100, dtype=BF16, device=dev), torch.ones(100, dtype=BF16, device=dev), 1e-5)


@pytest.fixture(scope="module")
def ln():
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import layernorm_kernels
    return layernorm_kernels


@pytest.mark.parametrize("n", [768, 1024, 96, 4096, 8192, 2048 + 64])
@pytest.mark.parametrize("pdtype", [BF16, torch.float32])
def test_layernorm_forward_backward(ln, dev, n, pdtype):
    g = torch.Generator().manual_seed(n)
    shape = (3, 11, n)
    x = (torch.randn(*shape, generator=g) * 2 + 0.5).to(BF16)
    w = (1 + 0.2 * torch.randn(n, generator=g)).to(pdtype)
    b = (0.1 * torch.randn(n, generator=g)).to(pdtype)
    dy = torch.randn(*shape, generator=g).to(BF16)
    y, mean, rstd, bs, nw = ln.layernorm_forward(x.to(dev), w.to(dev), b.to(dev), 1e-5)
    y_o, mean_o, rstd_o = O.layernorm_fwd(x, w, b, 1e-5)
    assert y.dtype == BF16 and y.shape == x.shape and mean.shape == (33,) and bs >= n
    assert_close_bf16(y, y_o, what="layernorm_forward vs oracle")
    assert torch.allclose(mean.cpu(), mean_o, atol=1e-5) and torch.allclose(rstd.cpu(), rstd_o, rtol=1e-5)
    ref = F.layer_norm(x.double(), (n,), w.double(), b.double(), 1e-5)
    assert_close_bf16(y, ref, what="layernorm_forward vs torch layer_norm")
    dx, dw, db = ln.layernorm_backward(dy.to(dev), x.to(dev), w.to(dev), b.to(dev), mean, rstd, True, 1e-5, nw, bs)
    assert dw is None and db is None
    assert_close_bf16(dx, O.layernorm_bwd(dy, x, w, mean_o, rstd_o), what="layernorm_backward vs oracle")
    xd = x.double().requires_grad_()
    F.layer_norm(xd, (n,), w.double(), b.double(), 1e-5).backward(dy.double())
    assert_close_bf16(dx, xd.grad, what="layernorm_backward vs autograd")
    assert ln.layernorm_backward(dy.to(dev), x.to(dev), w.to(dev), b.to(dev), mean, rstd, False, 1e-5, nw, bs) == (None, None, None)


def test_layernorm_errors(ln, dev):
    w = torch.ones(20, device=dev, dtype=BF16)
    with pytest.raises(RuntimeError):
        ln.layernorm_forward(torch.zeros(2, 20, device=dev, dtype=BF16), w, w, 1e-5)             # N % 8
    with pytest.raises(NotImplementedError):
        ln.layernorm_forward(torch.zeros(2, 24, device=dev), torch.ones(24, device=dev), torch.ones(24, device=dev), 1e-5)
    with pytest.raises(Exception):
        ln.layernorm_forward(torch.zeros(2, 24, dtype=BF16), torch.ones(24, dtype=BF16), torch.ones(24, dtype=BF16), 1e-5)


@pytest.mark.parametrize("n", [5120, 6144, 8192])
@pytest.mark.parametrize("wdtype", [BF16, torch.float32])
def test_rmsnorm_backward_wide_rows_both_kernels_same_bits(ops, dev, n, wdtype):
    """Rows wider than 4096 channels: an even row count goes to the column-slab kernel, an odd one (or the
    "norm_compress_slab" switch off) to the row-per-wave kernel.  The same rows through both must be the same
    bits, with and without the residual add."""
    from hyclora_amd import _lib
    g = torch.Generator().manual_seed(n)
    rows = 64
    x = (torch.randn(1, rows, n, generator=g) * 2).to(BF16).to(dev)
    dy = torch.randn(1, rows, n, generator=g).to(BF16).to(dev)
    res = torch.randn(1, rows, n, generator=g).to(BF16).to(dev)
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(wdtype).to(dev)
    rstd = ops.norm.rmsnorm_forward(x, w, 1e-5)[2]
    got = {}
    try:
        for slab in (1, 0):
            _lib.set_tuning("norm_compress_slab", slab)
            got[slab] = (ops.norm._backward(dy, x, w, rstd, want_dw=False)[0],
                         ops.norm._backward(dy, x, w, rstd, want_dw=False, residual=res)[0])
    finally:
        _lib.set_tuning("norm_compress_slab", 1)
    assert torch.equal(got[1][0], got[0][0]) and torch.equal(got[1][1], got[0][1])
    # an odd row count takes the row-per-wave kernel whatever the switch says: the first 63 rows must agree too
    odd = ops.norm._backward(dy[:, :63], x[:, :63], w, rstd[:63], want_dw=False)[0]
    assert torch.equal(odd, got[1][0][:, :63])
    dx_ref, _ = O.rmsnorm_bwd(dy.cpu(), x.cpu(), w.cpu(), rstd.cpu())
    assert_close_bf16(got[1][0], dx_ref, what="wide-row backward vs oracle")
