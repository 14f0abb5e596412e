"""The fused layers inside stock transformers models: every decoder layer of a small random LlamaForCausalLM /
MistralForCausalLM (eager attention, PEFT-style LoRA wrappers around its seven linears) runs through
`decoder_layer_forward` - the call the reference's model files make (models/llama/modeling_llama.py:745-786) -
and logits, loss and adapter gradients are compared with the stock model's own forward and autograd.  That is an
independent statement of the layer (transformers' RMSNorm, rotary embedding, grouped-query attention and MLP), not
this repository's."""
import types

import pytest
import torch

from helpers import BF16, rel_err_and_cos
from test_gpu_layers import RefRMSNorm, config

pytestmark = pytest.mark.gpu
transformers = pytest.importorskip("transformers")

WIRING_FLOOR = {8: 0.9, 4: 0.8}      # cosine of a compressed layer's adapter gradients against uncompressed autograd


class LoraLinear(torch.nn.Module):
    """A linear wrapped the way PEFT wraps it: `base_layer`, `lora_A` / `lora_B` as ModuleDicts keyed by adapter name."""

    def __init__(self, base, rank, gen):
        super().__init__()
        self.base_layer = base
        base.weight.requires_grad_(False)
        dev = base.weight.device
        a = torch.nn.Linear(base.in_features, rank, bias=False, device=dev, dtype=BF16)
        b = torch.nn.Linear(rank, base.out_features, bias=False, device=dev, dtype=BF16)
        with torch.no_grad():
            a.weight.copy_(torch.randn(a.weight.shape, generator=gen, device=dev) / base.in_features ** 0.5)
            b.weight.copy_(torch.randn(b.weight.shape, generator=gen, device=dev) * 0.05)
        self.lora_A = torch.nn.ModuleDict({"default": a})
        self.lora_B = torch.nn.ModuleDict({"default": b})

    def forward(self, x):
        return self.base_layer(x) + self.lora_B["default"](self.lora_A["default"](x))


def build(dev, family, head_dim):
    heads, kv = 4, (2 if family == "mistral" else 4)
    common = dict(vocab_size=128, hidden_size=heads * head_dim, intermediate_size=768, num_hidden_layers=2,
                  num_attention_heads=heads, num_key_value_heads=kv, max_position_embeddings=256, rms_norm_eps=1e-5,
                  attn_implementation="eager")
    torch.manual_seed(5)
    if family != "mistral":
        model = transformers.LlamaForCausalLM(transformers.LlamaConfig(**common))
    else:
        model = transformers.MistralForCausalLM(transformers.MistralConfig(sliding_window=None, **common))
    model = model.to(device=dev, dtype=BF16)
    gen = torch.Generator(device=dev).manual_seed(9)
    for p in model.parameters():
        p.requires_grad_(False)
    for layer in model.model.layers:
        for parent, names in ((layer.self_attn, ("q_proj", "k_proj", "v_proj", "o_proj")),
                              (layer.mlp, ("gate_proj", "up_proj", "down_proj"))):
            for n in names:
                setattr(parent, n, LoraLinear(getattr(parent, n), 16, gen))
    model.train()
    return model


def loss_and_grads(model, ids):
    for p in model.parameters():
        p.grad = None
    out = model(input_ids=ids, labels=ids, use_cache=False)
    out.loss.backward()
    grads = {n: p.grad.clone() for n, p in model.named_parameters() if p.requires_grad}
    return out.logits.detach().clone(), out.loss.item(), grads


@pytest.mark.parametrize("family, head_dim", [("llama", 64), ("llama", 128), ("mistral", 128), ("llama_flash_attn", 128)])
@pytest.mark.parametrize("layer_type, q_bit", [("baseline", 0), ("intra_inter_full_fuse", 8), ("intra_inter", 4)])
def test_stock_model_through_the_fused_layers(dev, family, head_dim, layer_type, q_bit):
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import llama, llama_flash_attn, mistral
    if family == "llama_flash_attn" and layer_type == "intra_inter_full_fuse":
        layer_type = "intra"                     # the three layer types of the reference's map-free model
    pkg = {"llama": llama, "mistral": mistral, "llama_flash_attn": llama_flash_attn}[family]
    model = build(dev, family, head_dim)
    ids = torch.randint(0, 128, (2, 256), generator=torch.Generator().manual_seed(1)).to(dev)
    # The stock layers and autograd - with one exception: the decoder layers' two norms take the reference's
    # RMSNorm backward (rmsnorm_kernels.py:92-100, whose mean term is not part of a true RMSNorm's derivative and
    # which the fused layers reproduce), so that the comparison is about everything else.
    for layer in model.model.layers:
        for norm in (layer.input_layernorm, layer.post_attention_layernorm):
            norm.forward = types.MethodType(lambda self, x: RefRMSNorm.apply(x, self.weight), norm)
    ref_logits, ref_loss, ref_grads = loss_and_grads(model, ids)

    switch = mistral.set_fused_mistral_layer if family == "mistral" else pkg.set_fused_llama_layer
    key_padding = torch.ones(ids.shape, dtype=torch.long, device=dev)     # what the map-free model hands its layers
    switch(model, config(layer_type, q_bit, sm_ratio=0.999, thr=5) if q_bit else
           types.SimpleNamespace(use_hyclora=True, layer_type="baseline"))

    def forward(self, hidden_states, attention_mask=None, position_embeddings=None, **_):
        cos, sin = position_embeddings
        if family == "llama_flash_attn":
            attention_mask = key_padding
        return pkg.decoder_layer_forward(self, hidden_states, attention_mask, cos, sin)
    for layer in model.model.layers:
        layer.forward = types.MethodType(forward, layer)
    logits, loss, grads = loss_and_grads(model, ids)

    rel, cos = rel_err_and_cos(logits, ref_logits)
    assert rel <= 2e-2 and cos >= 0.9999, f"logits: rel {rel:.2e} cos {cos:.6f}"       # two layers of bf16 rounding
    assert abs(loss - ref_loss) <= 1e-2 * abs(ref_loss)
    assert set(grads) == set(ref_grads) and len(grads) == 2 * 7 * 2
    worst = (0.0, 1.0, "")
    for name in sorted(grads):
        rel, cos = rel_err_and_cos(grads[name], ref_grads[name])
        if cos < worst[1]:
            worst = (rel, cos, name)
        if layer_type == "baseline":
            assert rel <= 3e-2 and cos >= 0.999, f"{family} d{head_dim} baseline {name}: rel {rel:.2e} cos {cos:.6f}"
        elif family == "llama_flash_attn" and (".q_proj." in name or ".k_proj." in name):
            # downstream of the flash backward, which the reference hands the *dequantised* attention output
            # (llama_flash_attn/fused_llama_layer_intra_inter.py:450-461): in a randomly initialised model that output
            # is close to a running mean of v, far outside its own range per channel, and the symmetric codes clip it -
            # the same at 8 and at 4 bits
            assert cos >= 0.5, f"{family} d{head_dim} {layer_type} q{q_bit} {name}: rel {rel:.2e} cos {cos:.5f}"
        else:
            # the scheme's own quantisation error on a 512-token batch whose steps come from batch element 0 of this
            # very step; a mis-wired projection would give a cosine near zero
            assert cos >= WIRING_FLOOR[q_bit], f"{family} d{head_dim} {layer_type} q{q_bit} {name}: rel {rel:.2e} cos {cos:.5f}"
    print(f"{family} d{head_dim} {layer_type} q{q_bit}: logits rel {rel_err_and_cos(logits, ref_logits)[0]:.2e}, "
          f"worst gradient {worst[2]}: rel {worst[0]:.2e} cos {worst[1]:.5f}")


@pytest.mark.parametrize("layer_type, q_bit", [("baseline", 0), ("intra_inter", 8), ("intra", 4)])
@pytest.mark.parametrize("padding", [False, True])
def test_stock_roberta_through_the_fused_layers(dev, layer_type, q_bit, padding):
    """The encoder layers the same way: a two-layer random RobertaForSequenceClassification (no dropout) whose
    layers call `encoder_layer_forward` (models/roberta/modeling_roberta.py:428-457) against the stock forward
    and autograd - transformers' attention, exact GELU and LayerNorm (the fused layer's GELU backward is the
    reference's tanh form, gelu_kernels.py:49-56)."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import roberta
    torch.manual_seed(6)
    cfg = transformers.RobertaConfig(vocab_size=128, hidden_size=256, intermediate_size=768, num_hidden_layers=2,
                                     num_attention_heads=4, max_position_embeddings=260, attn_implementation="eager",
                                     hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0, num_labels=3)
    model = transformers.RobertaForSequenceClassification(cfg).to(device=dev, dtype=BF16)
    gen = torch.Generator(device=dev).manual_seed(4)
    for p in model.parameters():
        p.requires_grad_(False)
    for layer in model.roberta.encoder.layer:
        for parent, names in ((layer.attention.self, ("query", "key", "value")), (layer.attention.output, ("dense",)),
                              (layer.intermediate, ("dense",)), (layer.output, ("dense",))):
            for n in names:
                setattr(parent, n, LoraLinear(getattr(parent, n), 16, gen))
    model.train()
    ids = torch.randint(3, 128, (4, 256), generator=torch.Generator().manual_seed(2)).to(dev)
    mask = torch.ones(4, 256, dtype=torch.long, device=dev)
    if padding:
        mask[1, 200:] = 0
        mask[3, 97:] = 0
    labels = torch.tensor([0, 2, 1, 1], device=dev)

    def run():
        for p in model.parameters():
            p.grad = None
        out = model(input_ids=ids, attention_mask=mask, labels=labels)
        out.loss.backward()
        return out.logits.detach().clone(), out.loss.item(), {n: p.grad.clone() for n, p in model.named_parameters() if p.requires_grad}
    ref_logits, ref_loss, ref_grads = run()
    roberta.set_fused_roberta_layer(model, config(layer_type, q_bit, sm_ratio=0.999, thr=5) if q_bit else
                                    types.SimpleNamespace(use_hyclora=True, layer_type="baseline"))

    def forward(self, hidden_states, attention_mask=None, *args, **kwargs):
        return roberta.encoder_layer_forward(self, hidden_states, attention_mask)
    for layer in model.roberta.encoder.layer:
        layer.forward = types.MethodType(forward, layer)
    logits, loss, grads = run()
    rel, cos = rel_err_and_cos(logits, ref_logits)
    assert rel <= 2e-2 and cos >= 0.9999, f"logits: rel {rel:.2e} cos {cos:.6f}"
    assert abs(loss - ref_loss) <= 1e-2 * abs(ref_loss)
    assert set(grads) == set(ref_grads) and len(grads) == 2 * 6 * 2
    worst = (0.0, 1.0, "")
    for name in sorted(grads):
        rel, cos = rel_err_and_cos(grads[name], ref_grads[name])
        if cos < worst[1]:
            worst = (rel, cos, name)
        if layer_type == "baseline":
            assert rel <= 3e-2 and cos >= 0.999, f"roberta baseline {name}: rel {rel:.2e} cos {cos:.6f}"
        elif ".attention.output.dense.lora_A" in name:
            # formed from the restored attention output.  Without a causal mask a randomly initialised model's
            # attention is nearly uniform, every token's output is close to the mean of v, and the reference's
            # symmetric codes (step = (max - min) / 255, no zero point) clip a channel whose mean is far outside
            # its own range: the scheme's error, the same at 8 and at 4 bits.
            assert cos >= 0.5, f"roberta {layer_type} q{q_bit} {name}: rel {rel:.2e} cos {cos:.5f}"
        else:
            assert cos >= WIRING_FLOOR[q_bit], f"roberta {layer_type} q{q_bit} {name}: rel {rel:.2e} cos {cos:.5f}"
    print(f"roberta {layer_type} q{q_bit} padding={padding}: logits rel {rel_err_and_cos(logits, ref_logits)[0]:.2e}, "
          f"worst gradient {worst[2]}: rel {worst[0]:.2e} cos {worst[1]:.5f}")


@pytest.mark.parametrize("padding", [False, True])
def test_install_under_the_sdpa_back_end(dev, padding):
    """With transformers' default attention back end the layers are handed no mask (causal, nothing padded) or a
    boolean one: `install` turns either into the additive mask of the fused layers.  Against the same model under
    the eager back end and autograd."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import hf
    ids = torch.randint(0, 128, (2, 128), generator=torch.Generator().manual_seed(1)).to(dev)
    mask = torch.ones(2, 128, dtype=torch.long, device=dev)
    if padding:
        mask[1, 100:] = 0
    labels = ids.masked_fill(mask == 0, -100)
    results = []
    for impl, fused in (("eager", False), ("sdpa", True)):
        model = build(dev, "llama", 128)
        model.config._attn_implementation = impl
        for layer in model.model.layers:
            for norm in (layer.input_layernorm, layer.post_attention_layernorm):
                norm.forward = types.MethodType(lambda self, x: RefRMSNorm.apply(x, self.weight), norm)
        seen = []
        if fused:
            hf.install(model, types.SimpleNamespace(use_hyclora=True, layer_type="baseline"))
            model.model.layers[0].register_forward_pre_hook(
                lambda mod, args, kwargs: seen.append(kwargs.get("attention_mask", args[1] if len(args) > 1 else None)),
                with_kwargs=True)
        for p in model.parameters():
            p.grad = None
        out = model(input_ids=ids, attention_mask=mask if padding else None, labels=labels, use_cache=False)
        out.loss.backward()
        if fused:
            assert all(layer.fused_llama_layer.iteration == 1 for layer in model.model.layers)
            # what this back end hands a layer: nothing, or a boolean mask
            assert len(seen) == 1 and (seen[0].dtype == torch.bool if padding else seen[0] is None), seen
        results.append((out.logits.detach()[mask.bool()].clone(), out.loss.item(),
                        {n: p.grad.clone() for n, p in model.named_parameters() if p.requires_grad}))
    (ref_logits, ref_loss, ref_grads), (logits, loss, grads) = results
    rel, cos = rel_err_and_cos(logits, ref_logits)                 # logits of the real tokens
    assert rel <= 2e-2 and cos >= 0.9999, f"logits: rel {rel:.2e} cos {cos:.6f}"
    assert abs(loss - ref_loss) <= 1e-2 * abs(ref_loss)
    for name in grads:
        rel, cos = rel_err_and_cos(grads[name], ref_grads[name])
        assert rel <= 3e-2 and cos >= 0.999, f"{name}: rel {rel:.2e} cos {cos:.6f}"


@pytest.mark.parametrize("family", ["llama", "mistral", "roberta"])
def test_install_routes_training_steps_through_the_fused_layers(dev, family):
    """`hyclora_amd.models.hf.install` on a stock model: training-mode steps run the fused layers (the calibration
    counter of every layer advances, gradients agree with the stock model's), evaluation runs the stock layers
    (bit-identical outputs), as the reference's model files do (modeling_llama.py:745, :788-790)."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import hf
    if family == "roberta":
        torch.manual_seed(6)
        cfg = transformers.RobertaConfig(vocab_size=128, hidden_size=256, intermediate_size=768, num_hidden_layers=2,
                                         num_attention_heads=4, max_position_embeddings=260, attn_implementation="eager",
                                         hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0, num_labels=3)
        model = transformers.RobertaForSequenceClassification(cfg).to(device=dev, dtype=BF16)
        gen = torch.Generator(device=dev).manual_seed(4)
        for p in model.parameters():
            p.requires_grad_(False)
        layers = model.roberta.encoder.layer
        for layer in layers:
            for parent, names in ((layer.attention.self, ("query", "key", "value")), (layer.attention.output, ("dense",)),
                                  (layer.intermediate, ("dense",)), (layer.output, ("dense",))):
                for n in names:
                    setattr(parent, n, LoraLinear(getattr(parent, n), 16, gen))
        ids = torch.randint(3, 128, (2, 128), generator=torch.Generator().manual_seed(2)).to(dev)
        call = lambda: model(input_ids=ids, labels=torch.tensor([0, 2], device=dev))
        attr = "fused_roberta_layer"
    else:
        model = build(dev, family, 128)
        layers = model.model.layers
        ids = torch.randint(0, 128, (2, 128), generator=torch.Generator().manual_seed(1)).to(dev)
        call = lambda: model(input_ids=ids, labels=ids, use_cache=False)
        attr = "fused_llama_layer" if family == "llama" else "fused_mistral_layer"
        for layer in layers:                     # the reference's norm backward in the stock run, as in the tests above
            for norm in (layer.input_layernorm, layer.post_attention_layernorm):
                norm.forward = types.MethodType(lambda self, x: RefRMSNorm.apply(x, self.weight), norm)

    def step():
        for p in model.parameters():
            p.grad = None
        out = call()
        out.loss.backward()
        return out.logits.detach().clone(), {n: p.grad.clone() for n, p in model.named_parameters() if p.requires_grad}
    model.train()
    ref_logits, ref_grads = step()
    model.eval()
    with torch.no_grad():
        eval_before = call().logits.clone()
    assert hf.install(model, types.SimpleNamespace(use_hyclora=True, layer_type="baseline")) is model
    model.train()
    logits, grads = step()
    assert all(getattr(layer, attr).iteration == 1 for layer in layers)          # the fused layers ran
    rel, cos = rel_err_and_cos(logits, ref_logits)
    assert rel <= 2e-2 and cos >= 0.9999
    for name in grads:
        rel, cos = rel_err_and_cos(grads[name], ref_grads[name])
        assert rel <= 3e-2 and cos >= 0.999, f"{family} {name}: rel {rel:.2e} cos {cos:.6f}"
    model.eval()
    with torch.no_grad():
        eval_after = call().logits
    assert torch.equal(eval_after, eval_before)                                  # evaluation takes the stock layers
    assert all(getattr(layer, attr).iteration == 1 for layer in layers)
    with pytest.raises(ValueError):
        hf.install(types.SimpleNamespace(config=types.SimpleNamespace(model_type="gpt2")), None)
