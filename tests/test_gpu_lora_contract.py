"""GPU parity of the skinny LoRA products (u^T x and x v^T from one read of x, x dense or packed
codes) against the oracle's float64 products, across ragged shapes, ranks and operand layouts."""
import numpy as np
import pytest
import torch

from helpers import BF16, assert_close_bf16, bits
from oracle import hyc_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import compress_function, lora_kernels

    class Ns:
        products = staticmethod(lora_kernels.lora_products)
        from_codes = staticmethod(lora_kernels.lora_product_from_codes)
        dequant = staticmethod(compress_function.decompression_dequantization)
        dequant_zp = staticmethod(compress_function.decompression_dequantization_with_zero_point)
    return Ns


def inputs(seed, lead, N, R):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*lead, N, generator=g).to(BF16)
    u = torch.randn(*lead, R, generator=g).to(BF16)
    v = (torch.randn(R, N, generator=g) * 0.1).to(BF16)
    return x, u, v


def nearly_same_bits(a, b, what):
    """fp32 accumulation on the matrix cores against float64 on the host: the bf16 rounding lands
    on the neighbour for a few results that sit at a rounding boundary."""
    same = np.mean(bits(a) == bits(b))
    assert same >= 0.99, f"{what}: only {same:.5f} of the results bit-identical"
    assert_close_bf16(a, b, what=what)


SHAPES = [((2, 64), 256, 16), ((1, 37), 160, 16), ((300,), 11008, 16), ((2, 20), 256, 8), ((1, 33), 384, 32),
          ((1, 16), 128, 64), ((5,), 96, 4), ((3, 50), 4096, 16), ((2, 513), 512, 48), ((1, 1), 32, 2), ((700,), 1024, 12),
          ((520,), 8192, 64), ((300,), 4224, 40)]      # ranks past 32: several passes over several tiles per workgroup


@pytest.mark.parametrize("lead,N,R", SHAPES)
def test_both_products_from_one_pass(K, dev, lead, N, R):
    x, u, v = inputs(N + R, lead, N, R)
    want1, want2 = O.lora_products(x, u, v)
    d = lambda t: t.to(dev)
    p1, p2 = K.products(d(x), d(u), d(v))
    assert p1.shape == (R, N) and p2.shape == (*lead, R)
    nearly_same_bits(p1, want1, "u^T x")
    nearly_same_bits(p2, want2, "x v^T")
    # each product alone, and v handed over as the transposed view of an [N, R] weight
    a1, none = K.products(d(x), u=d(u))
    assert none is None and np.array_equal(bits(a1), bits(p1))
    none, a2 = K.products(d(x), v=d(v))
    assert none is None and np.array_equal(bits(a2), bits(p2))
    vt = d(v).t().contiguous().t()
    b1, b2 = K.products(d(x), d(u), vt)
    assert np.array_equal(bits(b1), bits(p1)) and np.array_equal(bits(b2), bits(p2))
    # the first product in the layout of a lora_B weight, [N, R]: the same values transposed
    t1, t2 = K.products(d(x), d(u), d(v), p1_transposed=True)
    assert t1.shape == (N, R) and t1.is_contiguous()
    assert torch.equal(t1.t(), p1) and np.array_equal(bits(t2), bits(p2))
    t1_alone, _ = K.products(d(x), u=d(u), p1_transposed=True)
    assert torch.equal(t1_alone, t1)


@pytest.mark.parametrize("q_bit", [2, 4, 8])
@pytest.mark.parametrize("zp", [False, True])
@pytest.mark.parametrize("B,M,N,R", [(2, 64, 256, 16), (1, 37, 160, 16), (1, 300, 11008, 16), (2, 50, 4096, 32), (3, 7, 96, 8),
                                     (1, 300, 1024, 64), (2, 40, 8192, 48)])
def test_row_product_straight_from_codes(K, dev, q_bit, zp, B, M, N, R):
    x, u, _ = inputs(q_bit + N, (B, M), N, R)
    if zp:
        x = x + 1.5
        s, z = O.scale_zero_point(x, q_bit)
    else:
        s, z = O.scale_only_quant(x, q_bit), None
    q = O.compress(x, s, q_bit, z)
    x_hat = O.decompress(q, s, q_bit, z)
    d = lambda t: None if t is None else t.to(dev)
    p1 = K.from_codes(d(q), d(s), d(u), d(z), q_bit)
    nearly_same_bits(p1, O.lora_products(x_hat, u)[0], "u^T DQ(q) vs oracle")
    dense = K.dequant_zp(d(q), d(s), d(z), q_bit) if zp else K.dequant(d(q), d(s), q_bit)
    assert np.array_equal(bits(p1), bits(K.products(dense, u=d(u))[0])), "same as dequantise, then multiply"


def test_results_do_not_depend_on_scheduling(K, dev):
    x, u, v = inputs(9, (4, 1024), 4096, 16)
    d = lambda t: t.to(dev)
    first = K.products(d(x), d(u), d(v))
    for _ in range(3):
        again = K.products(d(x), d(u), d(v))
        assert np.array_equal(bits(first[0]), bits(again[0])) and np.array_equal(bits(first[1]), bits(again[1]))


def test_argument_checks(K, dev):
    x, u, v = inputs(1, (8,), 64, 16)
    d = lambda t: t.to(dev)
    with pytest.raises(ValueError):
        K.products(d(x))
    with pytest.raises(ValueError):
        K.products(d(x)[..., :48], d(u), d(v)[:, :48])
    with pytest.raises(ValueError):
        K.products(d(x), d(u)[:4], None)
    with pytest.raises(ValueError):
        K.products(d(x), None, d(v)[:, :32])
    with pytest.raises(RuntimeError):
        K.products(x, u, v)


def test_lora_b_gradient_arrives_in_the_weights_layout(dev):
    """lora_backward returns grad lora_B as the [R, N] view of an [N, R] tensor: autograd's transpose on the way to
    the `weight.T` leaf is then contiguous and `.grad` takes it without the copy a strided gradient costs."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models.compute_utils import lora_backward
    g = torch.Generator().manual_seed(3)
    T, n_in, n_out, r = 64, 256, 384, 16
    w = torch.randn(n_out, n_in, generator=g).to(BF16).to(dev)
    la = torch.randn(r, n_in, generator=g).to(BF16).to(dev)
    lb = torch.randn(n_out, r, generator=g).to(BF16).to(dev)
    x = torch.randn(1, T, n_in, generator=g).to(BF16).to(dev)
    gy = torch.randn(1, T, n_out, generator=g).to(BF16).to(dev)
    xa = x @ la.t()
    grad_a, grad_b, grad_x = lora_backward(w, None, la.t(), lb.t(), x, xa, gy)
    assert grad_b.shape == (r, n_out) and grad_b.t().is_contiguous()
    assert grad_a.shape == (n_in, r) and grad_a.t().is_contiguous()
    want_b = (xa.float().reshape(T, r).t() @ gy.float().reshape(T, n_out))
    assert_close_bf16(grad_b.cpu(), want_b.to(BF16).cpu(), what="grad lora_B")
