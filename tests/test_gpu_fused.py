"""GPU parity of the fused LoRA-SiLU-Hadamard forward / backward: packed codes bit-exact,
outputs and gradients within bf16 tolerance, against the oracle and against the unfused
composition built from independently pinned pieces."""
import math

import pytest
import torch
import torch.nn.functional as F

from helpers import BF16, assert_close_bf16
from oracle import hyc_oracle as O

pytestmark = pytest.mark.gpu
QBITS = [2, 4, 8]


@pytest.fixture(scope="module")
def fz():
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import triton_fuse_lora_silu_hadamard_backward_kernels as b
    from hyclora_amd.operators import triton_fuse_lora_silu_hadamard_forward_kernels as f

    class Fz:
        fwd = staticmethod(f.triton_fuse_silu_forward)
        bwd = staticmethod(b.triton_fuse_silu_backward)
    return Fz


def mlp_inputs(seed, B, M, H, I, R):
    """benchmark configuration 2 in the given size: x ~ N(0,1), frozen W ~ N(0,0.02), LoRA A
    kaiming-uniform(a=sqrt(5)) as PEFT initialises it, LoRA B ~ N(0,1e-3) (scaled up here so
    that the LoRA term is visible in the outputs)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, M, H, generator=g).to(BF16)
    out = {}
    for name in ("gate", "up"):
        w = (torch.randn(I, H, generator=g) * 0.02).to(BF16)
        a = torch.empty(R, H)
        torch.nn.init.kaiming_uniform_(a, a=math.sqrt(5), generator=g)
        b = (torch.randn(I, R, generator=g) * 0.05).to(BF16)
        main = (x.float() @ w.float().t()).to(BF16)
        xa = (x.float() @ a.to(BF16).float().t()).to(BF16)
        out[name] = (xa, b.t().contiguous(), main)
    return out


@pytest.mark.parametrize("q_bit", QBITS)
@pytest.mark.parametrize("dims", [(2, 64, 256, 1024, 16), (1, 37, 128, 160, 16), (1, 16, 64, 11008, 16),
                                  (2, 20, 64, 256, 8), (1, 33, 64, 384, 32), (1, 16, 64, 128, 64), (1, 5, 64, 96, 4),
                                  (2, 100, 64, 384, 48), (1, 130, 64, 256, 64),
                                  (2, 112, 64, 384, 32), (1, 200, 64, 256, 24)])      # ranks 17..32 over several strips
def test_fused_forward_and_backward(fz, dev, q_bit, dims):
    B, M, H, I, R = dims
    t = mlp_inputs(q_bit + I, B, M, H, I, R)
    xa1, b1, x1 = t["gate"]
    xa2, b2, x2 = t["up"]
    s1 = O.scale_only_quant(x1, q_bit)
    s2 = O.scale_only_quant(x2, q_bit)
    d = lambda *ts: [v.to(dev) for v in ts]
    q1, q2, o = fz.fwd(*d(xa1, b1, x1, s1, xa2, b2, x2, s2), q_bit)
    q1_ref, q2_ref, o_ref = O.fused_fwd(xa1, b1, x1, s1, xa2, b2, x2, s2, q_bit)
    assert torch.equal(q1.cpu(), q1_ref) and torch.equal(q2.cpu(), q2_ref), "packed codes must be bit-exact"
    assert_close_bf16(o, o_ref, what="fused forward o vs oracle")
    # unfused composition in fp32
    gate = x1.float() + xa1.float() @ b1.float()
    up = x2.float() + xa2.float() @ b2.float()
    # (the bar is the oracle comparison above; this one measures the reference's own bf16-per-operation
    # arithmetic against fp32, and the rounded LoRA term of a rank-64 adapter is a larger share of it)
    assert_close_bf16(o, F.silu(gate) * up, rel_tol=1e-2 if R <= 32 else 1.5e-2, what="fused forward o vs unfused fp32")

    g = torch.randn(B, M, I, generator=torch.Generator().manual_seed(1)).to(BF16)
    ob, gg, gu = fz.bwd(*d(xa1, b1), q1, s1.to(dev), *d(xa2, b2), q2, s2.to(dev), g.to(dev), q_bit)
    ob_ref, gg_ref, gu_ref = O.fused_bwd(xa1, b1, q1_ref, s1, xa2, b2, q2_ref, s2, g, q_bit)
    assert_close_bf16(ob, ob_ref, what="fused backward o vs oracle")
    assert_close_bf16(gg, gg_ref, what="grad_gate vs oracle")
    assert_close_bf16(gu, gu_ref, what="grad_up vs oracle")
    # autograd of silu(gate)*up at the dequantised inputs
    gate = (O.decompress(q1_ref, s1, q_bit).float() + xa1.float() @ b1.float()).requires_grad_()
    up = (O.decompress(q2_ref, s2, q_bit).float() + xa2.float() @ b2.float()).requires_grad_()
    (F.silu(gate) * up).backward(g.float())
    # the bf16-per-operation chain of the reference is several roundings away from fp32 autograd
    assert_close_bf16(gg, gate.grad, rel_tol=2e-2, what="grad_gate vs autograd")
    assert_close_bf16(gu, up.grad, what="grad_up vs autograd")


@pytest.mark.parametrize("q_bit", QBITS)
@pytest.mark.parametrize("R", [16, 8, 48, 64, 32, 24])      # 48 and 64: the deep-rank instantiations walk the same way;
                                                             # 32 and 24: forward on the rolling path, backward on the guarded one
def test_fused_results_do_not_depend_on_the_strip_height(fz, dev, q_bit, R):
    # Interior strips are walked with the next tile requested ahead: one tile per strip takes only
    # the closing step of that walk, two tiles the opening and the closing one, more the loop in
    # between.  All of them, and the guarded path of the ragged last strip, must agree bit for bit.
    from hyclora_amd import _lib
    B, M, H, I = 1, 200, 64, 384                     # 200 rows: whole strips and a ragged remainder
    t = mlp_inputs(7 + q_bit, B, M, H, I, R)
    xa1, b1, x1 = t["gate"]
    xa2, b2, x2 = t["up"]
    s1 = O.scale_only_quant(x1, q_bit)
    s2 = O.scale_only_quant(x2, q_bit)
    g = torch.randn(B, M, I, generator=torch.Generator().manual_seed(2)).to(BF16)
    d = lambda *ts: [v.to(dev) for v in ts]
    outs = []
    try:
        for rows in (16, 32, 48, 96, 208):
            _lib.set_tuning("fuse_rows_per_wave", rows)
            q1, q2, o = fz.fwd(*d(xa1, b1, x1, s1, xa2, b2, x2, s2), q_bit)
            ob, gg, gu = fz.bwd(*d(xa1, b1), q1, s1.to(dev), *d(xa2, b2), q2, s2.to(dev), g.to(dev), q_bit)
            outs.append((q1, q2, o, ob, gg, gu))
    finally:
        _lib.set_tuning("fuse_rows_per_wave", 0)           # the library's defaults
    for other in outs[1:]:
        for a, b in zip(outs[0], other):
            assert torch.equal(a, b)
    q1_ref, q2_ref, o_ref = O.fused_fwd(xa1, b1, x1, s1, xa2, b2, x2, s2, q_bit)
    assert torch.equal(outs[0][0].cpu(), q1_ref) and torch.equal(outs[0][1].cpu(), q2_ref)
    assert_close_bf16(outs[0][2], o_ref, what="fused forward o vs oracle")
    ob_ref, gg_ref, gu_ref = O.fused_bwd(xa1, b1, q1_ref, s1, xa2, b2, q2_ref, s2, g, q_bit)
    assert_close_bf16(outs[0][4], gg_ref, what="grad_gate vs oracle")
    assert_close_bf16(outs[0][5], gu_ref, what="grad_up vs oracle")


@pytest.mark.parametrize("R", [16, 32])
def test_two_bit_code_lines_written_whole(fz, dev, R):
    """At 2 bits the four waves of a workgroup hand the 32-byte pieces of a row's code line over through LDS
    and one wave writes the line, wherever the whole workgroup is on interior strips; workgroups at the
    ragged edges (a last group of column tiles that is not complete, a last strip that is cut off, a column
    whose step needs the division branch) store their pieces directly.  One launch with all of these side by
    side must give the oracle's codes, at every strip height."""
    from hyclora_amd import _lib
    B, M, H, I = 1, 272, 64, 1536 + 128              # three whole groups of 512 columns and a quarter of one
    t = mlp_inputs(11 + R, B, M, H, I, R)
    xa1, b1, x1 = t["gate"]
    xa2, b2, x2 = t["up"]
    x1[:, :, 700] = 0                                # a constant column: step 0, the division branch, in group 1
    s1 = O.scale_only_quant(x1, 2)
    s2 = O.scale_only_quant(x2, 2)
    assert s1.reshape(-1)[700].item() == 0
    d = lambda *ts: [v.to(dev) for v in ts]
    q1_ref, q2_ref, o_ref = O.fused_fwd(xa1, b1, x1, s1, xa2, b2, x2, s2, 2)
    try:
        for rows in (0, 16, 32, 96, 272 - 16):
            _lib.set_tuning("fuse_rows_per_wave", rows)
            q1, q2, o = fz.fwd(*d(xa1, b1, x1, s1, xa2, b2, x2, s2), 2)
            assert torch.equal(q1.cpu(), q1_ref) and torch.equal(q2.cpu(), q2_ref), f"codes at strip height {rows}"
            assert_close_bf16(o, o_ref, what=f"fused forward o vs oracle at strip height {rows}")
    finally:
        _lib.set_tuning("fuse_rows_per_wave", 0)


def test_fused_lora_term_is_applied_per_row_and_column(fz, dev):
    # x1 = x2 = 0 and a one-hot xa isolates the MFMA operand mapping: y = b[r, :] for row r
    R, N, M = 16, 256, 32
    xa = torch.zeros(1, M, R)
    for m in range(M):
        xa[0, m, m % R] = 1.0 + m // R
    b1 = torch.arange(R * N, dtype=torch.float32).reshape(R, N) % 251 / 64 - 2
    b2 = torch.ones(R, N)
    x0 = torch.zeros(1, M, N, dtype=BF16)
    s = torch.ones(1, N, dtype=BF16)
    d = lambda *ts: [v.to(BF16).to(dev) for v in ts]
    _, _, o = fz.fwd(*d(xa, b1, x0, s, xa, b2, x0, s), 8)
    y1 = (xa.to(BF16).float() @ b1.to(BF16).float()).to(BF16)
    y2 = (xa.to(BF16).float() @ b2.to(BF16).float()).to(BF16)
    ref = O.silu_mul(y1, y2)
    assert_close_bf16(o, ref, rel_tol=2e-3, what="one-hot LoRA mapping")


def test_fused_errors(fz, dev):
    z = lambda *s: torch.zeros(*s, dtype=BF16, device=dev)
    with pytest.raises(Exception):
        fz.fwd(z(1, 4, 6), z(6, 64), z(1, 4, 64), z(1, 64), z(1, 4, 6), z(6, 64), z(1, 4, 64), z(1, 64), 4)   # rank 6
    with pytest.raises(ValueError):
        fz.fwd(z(1, 4, 16), z(16, 48), z(1, 4, 48), z(1, 48), z(1, 4, 16), z(16, 48), z(1, 4, 48), z(1, 48), 4)
    with pytest.raises(ValueError):
        fz.fwd(z(1, 4, 16), z(16, 64), z(1, 4, 64), z(1, 64), z(1, 4, 16), z(16, 64), z(1, 4, 64), z(1, 64), 3)


@pytest.mark.parametrize("q_bit", [4])
def test_fused_full_size_config2(fz, dev, q_bit):
    # benchmark configuration 2: T = 4x1024, N = 11008, R = 16.  Codes against the standalone
    # quantiser (already pinned bit-exact), o against the unfused torch composition on the GPU.
    from hyclora_amd.operators import compress_function as cf
    g = torch.Generator(device=dev).manual_seed(0)
    B, M, N, R = 4, 1024, 11008, 16
    rn = lambda *s, sc=1.0: (torch.randn(*s, generator=g, device=dev, dtype=torch.float32) * sc).to(BF16)
    x1, x2 = rn(B, M, N), rn(B, M, N)
    xa1, xa2 = rn(B, M, R), rn(B, M, R)
    b1, b2 = rn(R, N, sc=0.05), rn(R, N, sc=0.05)
    s1 = cf.get_statistics_only_quant(x1, q_bit, 'per-channel')
    s2 = cf.get_statistics_only_quant(x2, q_bit, 'per-channel')
    q1, q2, o = fz.fwd(xa1, b1, x1, s1, xa2, b2, x2, s2, q_bit)
    assert torch.equal(q1, cf.compression_quantization(x1, s1, q_bit))
    assert torch.equal(q2, cf.compression_quantization(x2, s2, q_bit))
    ref = F.silu(x1.float() + xa1.float() @ b1.float()) * (x2.float() + xa2.float() @ b2.float())
    assert_close_bf16(o, ref, what="full-size fused forward")
    gr = rn(B, M, N)
    ob, gg, gu = fz.bwd(xa1, b1, q1, s1, xa2, b2, q2, s2, gr, q_bit)
    gate = (cf.decompression_dequantization(q1, s1, q_bit).float() + xa1.float() @ b1.float()).requires_grad_()
    up = (cf.decompression_dequantization(q2, s2, q_bit).float() + xa2.float() @ b2.float()).requires_grad_()
    out = F.silu(gate) * up
    out.backward(gr.float())
    assert_close_bf16(ob, out.detach(), what="full-size recomputed o")
    assert_close_bf16(gg, gate.grad, rel_tol=2e-2, what="full-size grad_gate")
    assert_close_bf16(gu, up.grad, what="full-size grad_up")
