"""GPU parity of the LoRA-add kernels (plain, with the quantiser, from packed codes): packed codes
bit-exact against the oracle's quantiser, the sum against the oracle's bf16 composition, and the
three forms bit-identical among themselves and to the separate operators they replace."""
import math

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
        add = staticmethod(lora_kernels.lora_add)
        add_quant = staticmethod(lora_kernels.lora_add_quant)
        add_restore = staticmethod(lora_kernels.lora_add_restore)
        quant = staticmethod(compress_function.compression_quantization)
        quant_zp = staticmethod(compress_function.compression_quantization_with_zero_point)
        dequant = staticmethod(compress_function.decompression_dequantization)
        dequant_zp = staticmethod(compress_function.decompression_dequantization_with_zero_point)
    return Ns


def inputs(seed, B, M, N, R, shift=0.0):
    g = torch.Generator().manual_seed(seed)
    main = (torch.randn(B, M, N, generator=g) + shift).to(BF16)
    a = torch.empty(R, 64)
    torch.nn.init.kaiming_uniform_(a, a=math.sqrt(5), generator=g)
    xa = (torch.randn(B, M, 64, generator=g) @ a.t()).to(BF16)
    b = (torch.randn(R, N, generator=g) * 0.3).to(BF16)            # large enough to move the sum
    return main, xa, b


def mostly_same_bits(a, b, what):
    """The rank-R dot product is accumulated in fp32 in a different order on the matrix cores than
    in the CPU matmul, so a bf16 rounding may land on the neighbour now and then: nearly every
    element identical, the rest within the bf16 tolerance."""
    same = np.mean(bits(a) == bits(b))
    assert same >= 0.998, f"{what}: only {same:.5f} of the elements bit-identical"
    assert_close_bf16(a, b, what=what)


DIMS = [(2, 64, 256, 16), (1, 37, 160, 16), (1, 16, 11008, 16), (2, 20, 256, 8), (1, 33, 384, 32),
        (1, 16, 128, 64), (1, 5, 96, 4), (3, 50, 4096, 16)]


@pytest.mark.parametrize("dims", DIMS)
def test_plain_add_out_of_place_and_in_place(K, dev, dims):
    B, M, N, R = dims
    main, xa, b = inputs(N + R, B, M, N, R)
    want = O.lora_add(main, xa, b)
    x = main.to(dev)
    y = K.add(x, xa.to(dev), b.to(dev))
    assert torch.equal(x.cpu(), main), "input must be left alone"
    mostly_same_bits(y, want, "lora_add vs oracle")
    assert_close_bf16(y, main.float() + xa.float() @ b.float(), what="lora_add vs fp32")
    y2 = K.add(x, xa.to(dev), b.to(dev), inplace=True)
    assert y2.data_ptr() == x.data_ptr()
    assert np.array_equal(bits(y2), bits(y)), "in place and out of place must agree bit for bit"


@pytest.mark.parametrize("q_bit", [2, 4, 8])
@pytest.mark.parametrize("zp", [False, True])
@pytest.mark.parametrize("dims", DIMS)
def test_add_with_quantiser_and_from_codes(K, dev, q_bit, zp, dims):
    B, M, N, R = dims
    main, xa, b = inputs(q_bit + N, B, M, N, R, shift=1.5 if zp else 0.0)
    if zp:
        s, z = O.scale_zero_point(main, q_bit)
    else:
        s, z = O.scale_only_quant(main, q_bit), None
    d = lambda t: None if t is None else t.to(dev)
    q, y = K.add_quant(d(main), d(xa), d(b), d(s), d(z), q_bit)
    q_ref = O.compress(main, s, q_bit, z)
    assert torch.equal(q.cpu(), q_ref), "packed codes must be bit-exact"
    sep = K.quant_zp(d(main), d(s), d(z), q_bit) if zp else K.quant(d(main), d(s), q_bit)
    assert torch.equal(q, sep), "same codes as the standalone quantiser"
    mostly_same_bits(y, O.lora_add(main, xa, b), "lora_add_quant y vs oracle")
    assert np.array_equal(bits(y), bits(K.add(d(main), d(xa), d(b)))), "same sum as the plain form"

    r = K.add_restore(q, d(s), d(xa), d(b), d(z), q_bit)
    x_hat_ref = O.decompress(q_ref, s, q_bit, z)
    mostly_same_bits(r, O.lora_add(x_hat_ref, xa, b), "lora_add_restore vs oracle")
    x_hat = K.dequant_zp(q, d(s), d(z), q_bit) if zp else K.dequant(q, d(s), q_bit)
    assert np.array_equal(bits(x_hat), bits(x_hat_ref))
    assert np.array_equal(bits(r), bits(K.add(x_hat, d(xa), d(b)))), "same as dequantise, then add"


@pytest.mark.parametrize("dims", [(2, 64, 256, 16), (1, 37, 160, 16), (3, 50, 4096, 16), (1, 5, 96, 4)])
def test_plain_add_with_residual(K, dev, dims):
    """y = residual + (x + xa.b), each sum rounded to bf16: bit-identical to the plain form followed
    by torch's add, out of place and in place."""
    B, M, N, R = dims
    main, xa, b = inputs(N + 3 * R, B, M, N, R)
    res = torch.randn(B, M, N, generator=torch.Generator().manual_seed(7)).to(BF16)
    d = lambda t: t.to(dev)
    two_steps = d(res) + K.add(d(main), d(xa), d(b))
    y = K.add(d(main), d(xa), d(b), residual=d(res))
    assert np.array_equal(bits(y), bits(two_steps))
    mostly_same_bits(y, res + O.lora_add(main, xa, b), "residual + lora_add vs oracle")
    x = d(main)
    y2 = K.add(x, d(xa), d(b), inplace=True, residual=d(res))
    assert y2.data_ptr() == x.data_ptr() and np.array_equal(bits(y2), bits(two_steps))
    with pytest.raises(ValueError):
        K.add(d(main), d(xa), d(b), residual=d(res)[:, :1])


@pytest.mark.parametrize("R", [4, 16, 32, 64])
def test_lora_b_in_linear_layout(K, dev, R):
    """A [R, N] view of an [N, R] contiguous weight - what `lora_B.weight.T` is - is read where it
    lies: same bits as with a contiguous [R, N] copy, in all three forms and in the fused kernels."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators.triton_fuse_lora_silu_hadamard_backward_kernels import triton_fuse_silu_backward
    from hyclora_amd.operators.triton_fuse_lora_silu_hadamard_forward_kernels import triton_fuse_silu_forward
    B, M, N = 2, 40, 384
    main, xa, b = inputs(R, B, M, N, R)
    s = O.scale_only_quant(main, 4)
    d = lambda t: t.to(dev)
    w = d(b).t().contiguous()                  # [N, R], the nn.Linear layout
    bt = w.t()                                 # [R, N] view
    assert not bt.is_contiguous()
    assert np.array_equal(bits(K.add(d(main), d(xa), bt)), bits(K.add(d(main), d(xa), d(b))))
    q1, y1 = K.add_quant(d(main), d(xa), bt, d(s), None, 4)
    q2, y2 = K.add_quant(d(main), d(xa), d(b), d(s), None, 4)
    assert torch.equal(q1, q2) and np.array_equal(bits(y1), bits(y2))
    assert np.array_equal(bits(K.add_restore(q1, d(s), d(xa), bt, None, 4)),
                          bits(K.add_restore(q1, d(s), d(xa), d(b), None, 4)))
    fa = triton_fuse_silu_forward(d(xa), bt, d(main), d(s), d(xa), bt, d(main), d(s), 4)
    fb = triton_fuse_silu_forward(d(xa), d(b), d(main), d(s), d(xa), d(b), d(main), d(s), 4)
    assert all(np.array_equal(u.cpu().view(torch.uint8).numpy(), v.cpu().view(torch.uint8).numpy()) for u, v in zip(fa, fb))
    g = torch.randn(B, M, N, generator=torch.Generator().manual_seed(3)).to(BF16).to(dev)
    ba = triton_fuse_silu_backward(d(xa), bt, fa[0], d(s), d(xa), bt, fa[1], d(s), g, 4)
    bb = triton_fuse_silu_backward(d(xa), d(b), fa[0], d(s), d(xa), d(b), fa[1], d(s), g, 4)
    assert all(np.array_equal(bits(u), bits(v)) for u, v in zip(ba, bb))


@pytest.mark.parametrize("q_bit", [2, 4, 8])
@pytest.mark.parametrize("zp", [False, True])
@pytest.mark.parametrize("table", [BF16, torch.float32])
@pytest.mark.parametrize("dims", [(2, 40, 256, 16), (1, 17, 128, 8), (3, 64, 1024, 16)])
def test_rotation_fused_into_the_add(K, dev, q_bit, zp, table, dims):
    """rope=(cos, sin): the sum leaves the kernel already rotated - bit-identical to the plain entry
    point followed by rope_forward on the [B, M, N/128, 128] view; the codes are those of the
    unrotated frozen part."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators.rope_kernels import rope_forward
    B, M, N, R = dims
    main, xa, b = inputs(q_bit + N + 1, B, M, N, R, shift=1.5 if zp else 0.0)
    s, z = O.scale_zero_point(main, q_bit) if zp else (O.scale_only_quant(main, q_bit), None)
    pos = torch.arange(M + 3, dtype=torch.float32)                 # a table longer than the sequence
    inv = 1.0 / (10000 ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))
    ang = torch.cat([pos[:, None] * inv[None, :]] * 2, dim=-1)
    cos, sin = ang.cos().to(table).to(dev)[None], ang.sin().to(table).to(dev)[None]
    d = lambda t: None if t is None else t.to(dev)
    q0, y0 = K.add_quant(d(main), d(xa), d(b), d(s), d(z), q_bit)
    want = rope_forward(y0.clone().view(B, M, N // 128, 128), cos, sin).view(B, M, N)
    q1, y1 = K.add_quant(d(main), d(xa), d(b), d(s), d(z), q_bit, rope=(cos, sin))
    assert torch.equal(q1, q0), "codes are taken before the rotation"
    assert np.array_equal(bits(y1), bits(want)), "fused rotation == rope_forward afterwards"
    r0 = K.add_restore(q0, d(s), d(xa), d(b), d(z), q_bit)
    r_want = rope_forward(r0.clone().view(B, M, N // 128, 128), cos, sin).view(B, M, N)
    r1 = K.add_restore(q0, d(s), d(xa), d(b), d(z), q_bit, rope=(cos, sin))
    assert np.array_equal(bits(r1), bits(r_want))
    assert_close_bf16(y1, O.rope(O.lora_add(main, xa, b).view(B, M, N // 128, 128), cos.cpu(), sin.cpu()).reshape(B, M, N),
                      what="rotated sum vs oracle")


def test_rotation_needs_whole_heads_of_128(K, dev):
    main, xa, b = inputs(2, 1, 8, 192, 16)
    s = O.scale_only_quant(main, 4)
    cos = torch.ones(1, 8, 128, device=dev, dtype=BF16)
    d = lambda t: t.to(dev)
    with pytest.raises(ValueError):
        K.add_quant(d(main), d(xa), d(b), d(s), None, 4, rope=(cos, cos))


def test_special_values_and_degenerate_steps(K, dev):
    """NaN / Inf inputs and steps outside the reciprocal path take the same codes as the standalone
    quantiser; an empty tensor is a no-op."""
    B, M, N, R = 1, 19, 128, 16
    main, xa, b = inputs(5, B, M, N, R)
    main[0, 3, 5] = float("nan")
    main[0, 4, 6] = float("inf")
    main[0, 5, 7] = -float("inf")
    s = O.scale_only_quant(main.nan_to_num(0.0, 0.0, 0.0), 4)
    s[0, 9] = 1e-30
    s[0, 10] = 1e25
    d = lambda t: t.to(dev)
    q, y = K.add_quant(d(main), d(xa), d(b), d(s), None, 4)
    assert torch.equal(q.cpu(), O.compress(main, s, 4))
    assert torch.equal(q, K.quant(d(main), d(s), 4))
    assert torch.isnan(y[0, 3, 5]) and torch.isinf(y[0, 4, 6]) and torch.isinf(y[0, 5, 7])
    r = K.add_restore(q, d(s), d(xa), d(b), None, 4)
    assert np.array_equal(bits(r), bits(K.add(K.dequant(q, d(s), 4), d(xa), d(b))))
    e = torch.empty(1, 0, N, device=dev, dtype=BF16)
    qe, ye = K.add_quant(e, torch.empty(1, 0, R, device=dev, dtype=BF16), d(b), d(s), None, 4)
    assert qe.shape == (1, 0, N // 2) and ye.shape == (1, 0, N)


def test_argument_checks(K, dev):
    main, xa, b = inputs(1, 1, 4, 64, 16)
    d = lambda t: t.to(dev)
    s = O.scale_only_quant(main, 4)
    with pytest.raises(ValueError):
        K.add(d(main), d(xa)[..., :8], d(b))                       # rank mismatch
    with pytest.raises(ValueError):
        K.add(d(main)[..., :48], d(xa), d(b)[:, :48])              # width not a multiple of 32
    with pytest.raises(ValueError):
        K.add_quant(d(main), d(xa), d(b), d(s), None, 3)
    with pytest.raises(ValueError):
        K.add_restore(torch.zeros(1, 4, 16, device=dev, dtype=torch.uint8), d(s), d(xa), d(b), None, 4)
    with pytest.raises(RuntimeError):
        K.add(main, xa, b)                                          # CPU tensors: no fallback


@pytest.mark.parametrize("q_bit", [2, 4, 8])
@pytest.mark.parametrize("with_zp", [False, True])
@pytest.mark.parametrize("dims", [(2, 96, (512, 128, 128), 16), (1, 37, (256, 256, 256, 384), 8), (3, 50, (1024,), 16),
                                  (1, 200, (4096, 1024, 1024), 16)])
def test_grouped_launch_equals_the_single_calls(K, dev, q_bit, with_zp, dims):
    """q, k and v (different widths, rotation on some members only) through ONE launch of the quantise form
    and ONE of the restore form: every member's codes and sums must be the bits its own call gives."""
    from hyclora_amd.operators import compress_function as cf
    from hyclora_amd.operators import lora_kernels
    B, M, widths, R = dims
    g = torch.Generator().manual_seed(M + q_bit)
    pos = torch.arange(M, dtype=torch.float32)
    inv = 1.0 / (10000.0 ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))
    ang = torch.cat([pos[:, None] * inv[None, :]] * 2, dim=-1)
    cos, sin = ang.cos().to(BF16).to(dev)[None], ang.sin().to(BF16).to(dev)[None]
    items, singles = [], []
    for i, n in enumerate(widths):
        main, xa, b = inputs(1000 * i + n + R, B, M, n, R, shift=0.5 if with_zp else 0.0)
        main, xa, b = main.to(dev), xa.to(dev), b.to(dev)
        if with_zp:
            s, z = cf.get_statistics_only_quant_zero_point(main, q_bit, 'per-channel')
        else:
            s, z = cf.get_statistics_only_quant(main, q_bit, 'per-channel'), None
        rope = (cos, sin) if (n % 128 == 0 and i != len(widths) - 1) else None       # the last member is not rotated
        items.append(dict(x_main=main, xa=xa, b=b, scale=s, zero_point=z, rope=rope))
        singles.append(lora_kernels.lora_add_quant(main, xa, b, s, z, q_bit, rope=rope))
    grouped = lora_kernels.lora_add_quant_group(items, q_bit)
    for (q1, y1), (q2, y2) in zip(singles, grouped):
        assert torch.equal(q1, q2) and torch.equal(y1, y2)
    back_items = [dict(q=q_, scale=it["scale"], xa=it["xa"], b=it["b"], zero_point=it["zero_point"], rope=it["rope"])
                  for it, (q_, _) in zip(items, grouped)]
    back = lora_kernels.lora_add_restore_group(back_items, q_bit)
    for it, y in zip(back_items, back):
        assert torch.equal(y, lora_kernels.lora_add_restore(it["q"], it["scale"], it["xa"], it["b"], it["zero_point"], q_bit,
                                                            rope=it["rope"]))


def test_grouped_launch_rejects_mixed_zero_points(K, dev):
    from hyclora_amd.operators import compress_function as cf
    from hyclora_amd.operators import lora_kernels
    main, xa, b = (t.to(dev) for t in inputs(5, 1, 32, 128, 16))
    s, z = cf.get_statistics_only_quant_zero_point(main, 4, 'per-channel')
    with pytest.raises(ValueError):
        lora_kernels.lora_add_quant_group([dict(x_main=main, xa=xa, b=b, scale=s, zero_point=z),
                                           dict(x_main=main, xa=xa, b=b, scale=s)], 4)
    with pytest.raises(ValueError):
        lora_kernels.lora_add_quant_group([dict(x_main=main, xa=xa, b=b, scale=s)] * 5, 4)


@pytest.mark.parametrize("count", [2, 3])
@pytest.mark.parametrize("T,N,R", [(64, 256, 16), (100, 1184, 8), (37, 96, 4), (272, 4096, 16), (4096, 1024, 12)])
@pytest.mark.parametrize("transposed", [False, True])
def test_sum_of_lora_adds_equals_the_chain(dev, count, T, N, R, transposed):
    """hyc_lora_add_sum is the chain lora_add(x_0), lora_add(x_1, residual=.), lora_add(x_2, residual=.) bit for bit:
    how the input gradients of projections that share an input are accumulated."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import lora_kernels as lk
    g = torch.Generator().manual_seed(T + N + R + count)
    rn = lambda *s, sc=1.0: (torch.randn(*s, generator=g) * sc).to(BF16).to(dev)
    terms = []
    for _ in range(count):
        b = rn(N, R, sc=0.2).t() if transposed else rn(R, N, sc=0.2)
        terms.append((rn(1, T, N), rn(1, T, R), b))
    assert lk.supported_sum(terms)
    originals = [(x.cpu().clone(), xa.cpu(), b.cpu()) for x, xa, b in terms]
    chain = None
    for x, xa, b in terms:
        chain = lk.lora_add(x.clone(), xa, b, inplace=True, residual=chain)
    first = terms[0][0]
    got = lk.lora_add_sum([(x.clone() if i else x, xa, b) for i, (x, xa, b) in enumerate(terms)])
    assert got.data_ptr() == first.data_ptr(), "the sum overwrites the first term"
    assert torch.equal(got, chain)
    # and the oracle's statement of one add (compute_utils.py:21-24), composed with bf16 additions
    want = None
    for x, xa, b in originals:
        t = O.lora_add(x, xa, b.contiguous())
        want = t if want is None else (want.float() + t.float()).to(BF16)
    assert_close_bf16(got, want, what="sum of LoRA adds vs the oracle's composition")


def test_sum_of_lora_adds_rejects_what_it_cannot_run(dev):
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import lora_kernels as lk
    g = torch.Generator().manual_seed(3)
    rn = lambda *s: torch.randn(*s, generator=g).to(BF16).to(dev)
    ok = [(rn(1, 32, 128), rn(1, 32, 16), rn(16, 128)) for _ in range(2)]
    assert lk.supported_sum(ok)
    assert not lk.supported_sum(ok[:1]) and not lk.supported_sum(ok * 2)
    wide = [(rn(1, 32, 128), rn(1, 32, 32), rn(32, 128)) for _ in range(2)]
    assert not lk.supported_sum(wide)
    with pytest.raises(ValueError):
        lk.lora_add_sum(wide)
    with pytest.raises(ValueError):
        lk.lora_add_sum([ok[0], (rn(1, 32, 256), rn(1, 32, 16), rn(16, 256))])


@pytest.mark.parametrize("dims", [(1, 300, 640, 16), (4, 1024, 4096, 16), (2, 1000, 1536, 8)])
def test_plain_add_does_not_depend_on_the_strip_height(K, dev, dims):
    """The plain add picks its strip height per shape (32, 48 or 64 rows a wave, whichever fills the resident
    waves' generations best; [4096, 4096] takes 48): every height gives the same bits, with and without a
    residual, and 0 restores the per-shape choice."""
    from hyclora_amd import _lib
    B, M, N, R = dims
    main, xa, b = inputs(7 + N, B, M, N, R)
    res = torch.randn(B, M, N, generator=torch.Generator().manual_seed(3)).to(BF16)
    d = lambda t: t.to(dev)
    want = K.add(d(main), d(xa), d(b))
    want_res = K.add(d(main), d(xa), d(b), residual=d(res))
    mostly_same_bits(want, O.lora_add(main, xa, b), "auto height")
    try:
        for rows in (16, 32, 48, 64, 112):
            _lib.set_tuning("add_rows_per_wave", rows)
            assert torch.equal(K.add(d(main), d(xa), d(b)), want), rows
            assert torch.equal(K.add(d(main), d(xa), d(b), residual=d(res)), want_res), rows
    finally:
        _lib.set_tuning("add_rows_per_wave", 0)
    assert torch.equal(K.add(d(main), d(xa), d(b)), want)
    with pytest.raises(Exception):
        _lib.set_tuning("add_quant_rows_per_wave", 0)          # only the plain add has a per-shape choice
