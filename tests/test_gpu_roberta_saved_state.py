"""Encoder (RoBERTa) layers at the operator tolerance: the fused layer's backward against the oracle layer's
backward run from the tensors the fused layer itself saved (codes, steps, outlier columns, channel lists, the
sparse attention map, x @ A buffers, LayerNorm statistics), at 8, 4 and 2 bits.  No code can differ between the two
sides, so every gradient must meet max rel err <= 1e-2 / cosine >= 0.9999; where the bf16 restatement itself is
further than that from the same backward evaluated without intermediate rounding, the layer is held to that
evaluation instead (see compare in test_gpu_layer_saved_state.py).  The oracle's backward is pinned on the CPU
against float64 autograd in tests/test_oracle_layer.py."""
import pytest
import torch

from test_gpu_layer_saved_state import compare
from test_gpu_layers import config
from test_gpu_roberta import NAMES, grads_of, make_inputs, run_fused

pytestmark = pytest.mark.gpu

GRAD_NAMES = ["x"] + [f"{n}.lora_{ab}" for n in NAMES for ab in "AB"]


def encoder_saved_state(out, heads):
    """The fused encoder layer's saved tensors under the reference's save-list names
    (models/roberta/fused_roberta_layer_intra_inter.py:202-232)."""
    node = out.grad_fn
    raw = dict(zip(node.names, node.saved_tensors))
    S = {}
    for name, t in raw.items():
        if name in ("a_idx", "a_val", "a_seg"):
            continue
        if name == "o_lora_a":
            name = "o_final_lora_a"
        for old, new in (("_s", "_scale"), ("_idx", "_channel_idx")):
            if name.endswith(old):
                name = name[:-len(old)] + new
                break
        S[name] = t
    nnz = int(raw["a_seg"][-1].item())
    S["a_o_indices"], S["a_o_values"] = raw["a_idx"][:nnz], raw["a_val"][:nnz]
    S["a_shape"] = (out.shape[0], heads, out.shape[1], out.shape[1])
    return S


def oracle_backward(t, out, layer_type, q_bit, exact):
    from oracle import hyc_oracle, layer_oracle
    up = (lambda v: v.double() if torch.is_tensor(v) and v.is_floating_point() else v) if exact else (lambda v: v)
    S = {k: up(v) for k, v in encoder_saved_state(out, t.heads).items()}
    weights = {n: (up(t.P[n][0].weight), up(t.P[n][0].bias), up(t.P[n][1].weight.detach()), up(t.P[n][2].weight.detach()))
               for n in NAMES}
    ln1, ln2 = tuple(up(v) for v in t.ln[0]), tuple(up(v) for v in t.ln[1])
    rounding = hyc_oracle.BF16
    try:
        if exact:
            hyc_oracle.BF16 = torch.float64
        with torch.no_grad():
            G = layer_oracle.roberta_layer_backward(S, up(t.grad), weights, ln1, ln2, t.heads, mode=layer_type, q_bit=q_bit)
    finally:
        hyc_oracle.BF16 = rounding
    expect = [G["x"]]
    for n in NAMES:
        expect += [G[(n, "A")].sum(0).t(), G[(n, "B")].sum(0).t()]
    return expect


@pytest.mark.parametrize("layer_type", ["intra", "intra_inter"])
@pytest.mark.parametrize("q_bit", [8, 4, 2])
@pytest.mark.parametrize("padding", [True, False])
def test_encoder_backward_from_the_layers_saved_state(dev, layer_type, q_bit, padding):
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import roberta
    t = make_inputs(dev, seed=60 + q_bit, padding=padding)
    layer = roberta.make_fused_roberta_layer(config(layer_type, q_bit, sm_ratio=0.05, thr=1))
    for step in ("calibrating", "frozen statistics"):
        out = run_fused(layer, t)
        expect = oracle_backward(t, out, layer_type, q_bit, exact=False)
        exact = oracle_backward(t, out, layer_type, q_bit, exact=True)
        compare(grads_of(t, out), expect, f"encoder {layer_type} q{q_bit} padding={padding} ({step})", exact, names=GRAD_NAMES)
