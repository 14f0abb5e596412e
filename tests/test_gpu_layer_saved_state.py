"""Layer parity at the operator tolerance (max rel err <= 1e-2, cosine >= 0.9999) for every gradient at 2, 4
and 8 bits: the fused layer's backward against the oracle layer's backward run FROM THE SAME SAVED STATE.

Forward of the fused layer leaves codes, steps, outlier columns, channel lists, the sparse attention map, the
x @ A buffers and the norm statistics on its autograd node.  Those very tensors are handed to
oracle/layer_oracle.layer_backward (pinned on the CPU in tests/test_oracle_layer.py), so no code can differ
between the two sides and nothing a quantiser would amplify is left: what remains is the arithmetic of the
backward itself - which tensor is dequantised with which step, which channel list restores which outliers, what
is recomputed from what, the kernels' rounding.  The end-to-end comparisons in test_gpu_layers.py (forward and
backward both redone by the oracle, codes free to differ by a flip) stay as loose sanity checks."""
import pytest
import torch

from helpers import layer_saved_state, rel_err_and_cos
from test_gpu_layers import config, grads_of, make_layer_inputs, run_fused

pytestmark = pytest.mark.gpu

NAMES = ["x", "norm_w1", "norm_w2"] + [f"{n}.lora_{ab}" for n in ("q", "k", "v", "o", "gate", "up", "down") for ab in "AB"]


def oracle_backward_from_saved_state(t, out, layer_type, q_bit, attention, exact=False, library_attention=False, **kw):
    """Gradients in NAMES order.  exact=True: the same backward evaluated without intermediate bf16 rounding -
    float64 operands, the oracle's rounding dtype bound to float64; a dequantised activation is still rounded
    to bf16 once, which is part of the format.  library_attention=True (map-free layers): the attention backward
    inside the oracle's walk is the library kernel the layer itself calls (torch's flash-attention backward, on
    the oracle's own q, k, v, dequantised output and the saved log-sum-exps) instead of the dense fp32
    restatement - everything that is not this repository's code is then the same on both sides."""
    from oracle import hyc_oracle, layer_oracle
    S = layer_saved_state(out, t.heads)
    node = out.grad_fn
    raw = dict(zip(node.names, node.saved_tensors))
    restated = layer_oracle._flash_backward

    def library_flash_backward(g_o, q, k, v, o, lse, scale):
        cum_q, cum_k, max_q, max_k = node.flash
        assert abs(scale - q.shape[-1] ** -0.5) < 1e-12          # the library's default scale
        return torch.ops.aten._scaled_dot_product_flash_attention_backward(
            g_o, q, k, v, o, lse, cum_q, cum_k, max_q, max_k, 0.0, True, raw["sdpa_rng"], raw["sdpa_unused"])
    up = (lambda v: v.double() if torch.is_tensor(v) and v.is_floating_point() else v) if exact else (lambda v: v)
    S = {k: up(v) for k, v in S.items()}
    weights = {n: tuple(up(m.weight.detach()) for m in t.P[n]) for n in t.P}
    rounding = hyc_oracle.BF16
    try:
        if exact:
            hyc_oracle.BF16 = torch.float64
        if library_attention:
            assert not exact and attention == "flash"
            layer_oracle._flash_backward = library_flash_backward
        with torch.no_grad():
            G = layer_oracle.layer_backward(S, up(t.grad), up(t.nw1.detach()), up(t.nw2.detach()), up(t.cos), up(t.sin),
                                            weights, t.heads, t.kv_heads, mode=layer_type, q_bit=q_bit,
                                            attention=attention, **kw)
    finally:
        hyc_oracle.BF16 = rounding
        layer_oracle._flash_backward = restated
    expect = [G["x"], G["nw1"], G["nw2"]]
    for n in ("q", "k", "v", "o", "gate", "up", "down"):
        expect += [G[(n, "A")].sum(0).t(), G[(n, "B")].sum(0).t()]
    return expect


TALLY = {"compared": 0, "direct": 0, "with the library's attention backward": 0, "by the exact evaluation": 0}


def within(got, want, rel_tol, cos_tol):
    rel, cos = rel_err_and_cos(got, want)
    return rel <= rel_tol and cos >= cos_tol


def compare(grads, expect, what, exact=None, rel_tol=1e-2, cos_tol=0.9999, names=None, expect_library=None):
    """Every gradient against the oracle's backward from the same saved state (`expect`, bf16 arithmetic as the
    reference's) at the operator tolerance: max rel err <= 1e-2, cosine >= 0.9999.

    The layer and the bf16 evaluation round at different points (the layer adds residuals and accumulates GEMM
    pairs in fp32 before its single rounding; the reference rounds every intermediate tensor), so each carries
    its own bf16 noise, and in a chain of a dozen operators on a few hundred rows that noise alone reaches
    1e-2 .. 5e-2 of the largest element for sums with cancellation (norm-weight gradients, the input gradient):
    the bf16 evaluation itself is that far from the same backward evaluated WITHOUT intermediate rounding
    (`exact`).  A gradient beyond the tolerance of the bf16 evaluation therefore still passes if the layer is
    as close to the exact evaluation as the tolerance or twice the bf16 evaluation's own distance from it,
    whichever is larger - i.e. its error is rounding noise of the size the reference's own arithmetic has.
    Such cases are printed and counted.  `expect_library` (map-free layers): the bf16 evaluation again, with the
    attention backward inside the oracle's walk done by the library kernel the layer calls (torch's
    flash-attention backward, which rounds its probabilities to bf16 where the restatement keeps fp32 matrices):
    a gradient that misses the restatement but meets THAT evaluation at the tolerance differs only by what the
    library's kernel does, and counts as met."""
    report, bad, noise = [], [], []
    for i, (name, got, want) in enumerate(zip(names or NAMES, grads, expect)):
        if got is None:
            assert name.startswith("norm_w"), name
            continue
        assert got.shape == want.shape, name
        rel, cos = rel_err_and_cos(got, want)
        entry = f"{name} {rel:.1e}/{cos:.6f}"
        TALLY["compared"] += 1
        if rel <= rel_tol and cos >= cos_tol:
            TALLY["direct"] += 1
        elif expect_library is not None and within(got, expect_library[i], rel_tol, cos_tol):
            # within the tolerance of the bf16 evaluation whose attention backward is the library's own kernel
            rel_l, cos_l = rel_err_and_cos(got, expect_library[i])
            entry += f" [with the library's attention backward in the oracle: {rel_l:.1e}/{cos_l:.6f}]"
            TALLY["with the library's attention backward"] += 1
        elif exact is None:
            bad.append(entry)
        else:
            rel_x, cos_x = rel_err_and_cos(got, exact[i])
            rel_o, cos_o = rel_err_and_cos(want, exact[i])
            entry += f" [vs exact: layer {rel_x:.1e}/{cos_x:.6f}, bf16 oracle {rel_o:.1e}/{cos_o:.6f}]"
            if rel_x <= max(rel_tol, 2 * rel_o) and 1 - cos_x <= max(1 - cos_tol, 2 * (1 - cos_o)):
                noise.append(entry)
                TALLY["by the exact evaluation"] += 1
            else:
                bad.append(entry)
        report.append(entry)
    print(f"{what}: " + "; ".join(report))
    if noise:
        print(f"{what}: beyond {rel_tol:g} of the bf16 evaluation, at its noise level from the exact one: {noise}")
    print(f"tally so far: {TALLY}")
    assert not bad, f"{what}: gradients outside the bound from identical saved state: {bad}"


@pytest.mark.parametrize("layer_type", ["intra", "intra_inter", "intra_inter_full_fuse"])
@pytest.mark.parametrize("q_bit", [8, 4, 2])
@pytest.mark.parametrize("kv_heads", [4, 2])
def test_backward_from_the_layers_saved_state(dev, layer_type, q_bit, kv_heads):
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import llama
    t = make_layer_inputs(dev, seed=170 + q_bit, kv_heads=kv_heads)
    layer = llama.make_fused_llama_layer(config(layer_type, q_bit, sm_ratio=0.05, thr=1))
    for step in ("calibrating", "frozen statistics"):
        out = run_fused(layer, t)
        expect = oracle_backward_from_saved_state(t, out, layer_type, q_bit, "map")
        exact = oracle_backward_from_saved_state(t, out, layer_type, q_bit, "map", exact=True)
        compare(grads_of(t, out), expect, f"{layer_type} q{q_bit} kv{kv_heads} ({step})", exact)


@pytest.mark.parametrize("layer_type", ["intra", "intra_inter", "intra_inter_full_fuse"])
@pytest.mark.parametrize("q_bit", [8, 4, 2])
@pytest.mark.parametrize("kv_heads", [4, 2])
def test_map_free_backward_from_the_layers_saved_state(dev, layer_type, q_bit, kv_heads):
    """Map-free variant: zero-point codes for q and k, log-sum-exps of the flash kernel kept, its backward handed
    the dequantised output (llama_flash_attn/fused_llama_layer_intra_inter.py:450-468)."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import llama_flash_attn as lf
    cls = {"intra": lf.FusedLlamaLayerIntra, "intra_inter": lf.FusedLlamaLayerIntraInter,
           "intra_inter_full_fuse": lf.FusedLlamaLayerIntraInterFullFuse}[layer_type]
    t = make_layer_inputs(dev, seed=190 + q_bit, S=128, kv_heads=kv_heads)
    layer = cls()
    layer.set_hyclora_config(config(layer_type, q_bit, thr=1))
    for step in ("calibrating", "frozen statistics"):
        out = run_fused(layer, t, use_mask=False)
        expect = oracle_backward_from_saved_state(t, out, layer_type, q_bit, "flash")
        library = oracle_backward_from_saved_state(t, out, layer_type, q_bit, "flash", library_attention=True)
        exact = oracle_backward_from_saved_state(t, out, layer_type, q_bit, "flash", exact=True)
        compare(grads_of(t, out), expect, f"map-free {layer_type} q{q_bit} kv{kv_heads} ({step})", exact, expect_library=library)


@pytest.mark.parametrize("dims", [dict(hidden=5120, heads=40, kv_heads=40, inter=13824),       # Llama-2-13B widths
                                  dict(hidden=8192, heads=64, kv_heads=8, inter=28672),         # Llama-2-70B widths
                                  dict(hidden=3072, heads=24, kv_heads=8, inter=8192)])         # a hidden size of six 512-column slabs
@pytest.mark.parametrize("q_bit", [4, 2])
def test_other_model_widths_from_the_layers_saved_state(dev, dims, q_bit):
    """Hidden sizes other than 4096 take other instantiations of the norm kernels (rows of 6, 10 and 16 chunks per
    lane, 8-row tiles of the LoRA-A contraction beyond 4096 channels) and other group counts in the LoRA kernels:
    the same bar, one short sequence per width, both attention forms."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import llama
    from hyclora_amd.models import llama_flash_attn as lf
    t = make_layer_inputs(dev, seed=300 + q_bit, B=1, S=128, **dims)
    layer = llama.make_fused_llama_layer(config("intra_inter_full_fuse", q_bit, sm_ratio=0.05, thr=1))
    for step in ("calibrating", "frozen statistics"):
        out = run_fused(layer, t)
        expect = oracle_backward_from_saved_state(t, out, "intra_inter_full_fuse", q_bit, "map")
        exact = oracle_backward_from_saved_state(t, out, "intra_inter_full_fuse", q_bit, "map", exact=True)
        compare(grads_of(t, out), expect, f"hidden {dims['hidden']} full_fuse q{q_bit} ({step})", exact)
    layer = lf.FusedLlamaLayerIntraInter()
    layer.set_hyclora_config(config("intra_inter", q_bit, thr=1))
    for step in ("calibrating", "frozen statistics"):
        out = run_fused(layer, t, use_mask=False)
        expect = oracle_backward_from_saved_state(t, out, "intra_inter", q_bit, "flash")
        library = oracle_backward_from_saved_state(t, out, "intra_inter", q_bit, "flash", library_attention=True)
        exact = oracle_backward_from_saved_state(t, out, "intra_inter", q_bit, "flash", exact=True)
        compare(grads_of(t, out), expect, f"hidden {dims['hidden']} map-free intra_inter q{q_bit} ({step})", exact, expect_library=library)


@pytest.mark.parametrize("layer_type", ["intra_inter", "intra_inter_full_fuse"])
def test_reference_outlier_list_switch(dev, layer_type):
    """The reference's intra_inter / full_fuse backward puts the input-norm outliers back at the post-attention
    norm's channels (fused_llama_layer_intra_inter_full_fuse.py:484).  With `reference_outlier_list=True` the
    layer does the same and agrees with the oracle doing the same from the same saved state; the two settings
    differ from each other where the two channel lists differ."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import llama
    t = make_layer_inputs(dev, seed=91)
    cls = llama.LAYER_TYPES[layer_type]
    got = {}
    for as_reference in (False, True):
        layer = cls(reference_outlier_list=as_reference)
        layer.set_hyclora_config(config(layer_type, 4, sm_ratio=0.05, ln_ratio=0.02))
        out = run_fused(layer, t)
        S = layer_saved_state(out, t.heads)
        assert not torch.equal(torch.sort(S["x_channel_idx"]).values, torch.sort(S["x_medium_channel_idx"]).values)
        expect = oracle_backward_from_saved_state(t, out, layer_type, 4, "map", as_reference_restores_x=as_reference)
        exact = oracle_backward_from_saved_state(t, out, layer_type, 4, "map", exact=True, as_reference_restores_x=as_reference)
        got[as_reference] = grads_of(t, out)
        compare(got[as_reference], expect, f"{layer_type} reference_outlier_list={as_reference}", exact)
    assert not torch.equal(got[False][0], got[True][0]), "the switch changes nothing"
    for a, b in zip(got[False][3:], got[True][3:]):
        assert torch.equal(a, b)           # only the input gradient passes through that restore
