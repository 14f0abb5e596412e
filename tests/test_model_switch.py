"""The host layers under the reference's module and class names, its model-level switch
(`set_fused_*_layer`) as functions of a model, and the call forms of its model files (CPU: nothing is run)."""
import importlib
import inspect
from types import SimpleNamespace

import pytest
import torch

import hyclora_amd  # noqa: F401

CFG = SimpleNamespace(use_hyclora=True, layer_type="intra_inter", iteration_threshold=5, softmax_outlier_ratio=0.05,
                      layernorm_outlier_ratio=0.005, q_bit=2)

# module -> class, as the reference's model files import them (models/llama/modeling_llama.py:52-55,
# models/mistral/modeling_mistral.py, models/llama_flash_attn/modeling_llama.py, models/roberta/modeling_roberta.py)
REFERENCE_IMPORTS = {
    "llama.fused_llama_layer_baseline": "FusedLlamaLayerBaseline",
    "llama.fused_llama_layer_intra": "FusedLlamaLayerIntra",
    "llama.fused_llama_layer_intra_inter": "FusedLlamaLayerIntraInter",
    "llama.fused_llama_layer_intra_inter_full_fuse": "FusedLlamaLayerIntraInterFullFuse",
    "mistral.fused_mistral_layer_baseline": "FusedMistralLayerBaseline",
    "mistral.fused_mistral_layer_intra": "FusedMistralLayerIntra",
    "mistral.fused_mistral_layer_intra_inter": "FusedMistralLayerIntraInter",
    "mistral.fused_mistral_layer_intra_inter_full_fuse": "FusedMistralLayerIntraInterFullFuse",
    "llama_flash_attn.fused_llama_layer_baseline": "FusedLlamaLayerBaseline",
    "llama_flash_attn.fused_llama_layer_intra": "FusedLlamaLayerIntra",
    "llama_flash_attn.fused_llama_layer_intra_inter": "FusedLlamaLayerIntraInter",
    "roberta.fused_roberta_layer_baseline": "FusedRobertaLayer",
    "roberta.fused_roberta_layer_intra": "FusedRobertaLayerIntra",
    "roberta.fused_roberta_layer_intra_inter": "FusedRobertaLayerIntraInter",
}


@pytest.mark.parametrize("module, name", sorted(REFERENCE_IMPORTS.items()))
def test_reference_module_names_export_the_classes(module, name):
    mod = importlib.import_module("hyclora_amd.models." + module)
    cls = getattr(mod, name)
    family, kind = module.split(".")
    layer = cls()
    layer.set_hyclora_config(CFG)
    assert layer.use_hyclora and layer.q_bit == 2 and layer.iteration == 0
    want = "baseline" if kind.endswith("baseline") else kind.split("_layer_")[1]
    assert layer.layer_type == want
    if family == "llama_flash_attn":
        assert layer.spec.attention == "sdpa"
    elif family != "roberta":
        assert layer.spec.attention == "map"


def _dummy(n_layers, path):
    layers = [SimpleNamespace() for _ in range(n_layers)]
    root = SimpleNamespace()
    node = root
    for part in path[:-1]:
        setattr(node, part, SimpleNamespace())
        node = getattr(node, part)
    setattr(node, path[-1], layers)
    return root, layers


@pytest.mark.parametrize("family, attr, path", [("llama", "fused_llama_layer", ("model", "layers")),
                                                ("mistral", "fused_mistral_layer", ("model", "layers")),
                                                ("llama_flash_attn", "fused_llama_layer", ("model", "layers")),
                                                ("roberta", "fused_roberta_layer", ("roberta", "encoder", "layer"))])
def test_model_level_switch(family, attr, path):
    pkg = importlib.import_module("hyclora_amd.models." + family)
    switch = getattr(pkg, "set_" + attr)
    model, layers = _dummy(3, path)
    switch(model, CFG)
    assert model.hyclora_config is CFG
    fused = [getattr(layer, attr) for layer in layers]
    assert len({id(f) for f in fused}) == 3                       # one module, one calibration state per layer
    for f in fused:
        assert type(f) is pkg.LAYER_TYPES["intra_inter"] and f.use_hyclora and f.iteration_threshold == 5
    with pytest.raises(ValueError):
        switch(model, SimpleNamespace(use_hyclora=True, layer_type="no_such_type"))


def test_switch_on_stock_transformers_models():
    """The attribute paths the switch walks are those of the stock model classes."""
    transformers = pytest.importorskip("transformers")
    from hyclora_amd.models import llama, roberta
    cfg = transformers.LlamaConfig(vocab_size=64, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                                   num_attention_heads=2, num_key_value_heads=2, max_position_embeddings=64)
    model = transformers.LlamaForCausalLM(cfg)
    llama.set_fused_llama_layer(model, CFG)
    assert all(isinstance(layer.fused_llama_layer, llama.FusedLlamaLayerIntraInter) for layer in model.model.layers)
    # registered as submodules: the calibration state travels with the model's state_dict
    assert any(k.endswith("fused_llama_layer._extra_state") for k in model.state_dict())
    rcfg = transformers.RobertaConfig(vocab_size=64, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                                      num_attention_heads=2, max_position_embeddings=66)
    rmodel = transformers.RobertaForSequenceClassification(rcfg)
    roberta.set_fused_roberta_layer(rmodel, CFG)
    assert all(isinstance(layer.fused_roberta_layer, roberta.FusedRobertaLayerIntraInter)
               for layer in rmodel.roberta.encoder.layer)


def test_forward_signatures_take_the_references_calls():
    """Positional argument counts of the calls in the reference's model files: 32 for the Llama / Mistral map
    layers (…, attention_mask, num_heads, head_dim, num_key_value_heads; modeling_llama.py:753-786), 31 for the
    map-free ones (no num_key_value_heads; llama_flash_attn/modeling_llama.py:620-653), 26 for the encoder
    layers (modeling_roberta.py:429-456)."""
    from hyclora_amd.models import llama, llama_flash_attn, roberta
    dec = inspect.signature(llama.FusedLlamaLayerIntraInter.forward).parameters
    names = list(dec)[1:]
    assert len(names) == 32 and names[-4:] == ["attention_mask", "num_heads", "head_dim", "num_key_value_heads"]
    assert dec["num_key_value_heads"].default is None            # may be left out, as the map-free call does
    assert llama_flash_attn.FusedLlamaLayerIntraInter.forward is llama.FusedLlamaLayerIntraInter.forward
    enc = list(inspect.signature(roberta.FusedRobertaLayerIntraInter.forward).parameters)[1:]
    assert len(enc) == 26 and enc[-3:] == ["attention_mask", "num_heads", "head_dim"]


def test_key_padding_mask_helper_on_cpu():
    """[B, S] key-padding mask -> additive causal mask among the real tokens + the rows to keep; a mask that
    pads nothing -> (None, None)."""
    from hyclora_amd.models.fused_decoder_layer import key_padding_attention_mask
    full = torch.ones(2, 5, dtype=torch.int64)
    assert key_padding_attention_mask(full, torch.float32) == (None, None)
    mask = torch.tensor([[1, 1, 1, 1], [0, 1, 1, 0]])
    add, keep = key_padding_attention_mask(mask, torch.float32)
    assert add.shape == (2, 1, 4, 4) and keep.shape == (2, 1, 4, 1)
    ninf = float("-inf")
    assert add[0, 0].tolist() == [[0, ninf, ninf, ninf], [0, 0, ninf, ninf], [0, 0, 0, ninf], [0, 0, 0, 0]]
    # batch 1: positions 0 and 3 are padding; a padded query sees itself only where nothing else is allowed
    assert add[1, 0].tolist() == [[0, ninf, ninf, ninf], [ninf, 0, ninf, ninf], [ninf, 0, 0, ninf], [ninf, 0, 0, 0]]
    assert keep[:, 0, :, 0].tolist() == [[1, 1, 1, 1], [0, 1, 1, 0]]
    with pytest.raises(ValueError):
        key_padding_attention_mask(torch.ones(2, 1, 4, 4), torch.float32)


def test_padding_helpers_round_trip():
    """unpad_input / pad_input of the reference's compute_utils (models/utils/compute_utils.py:53-97)."""
    from hyclora_amd.models.compute_utils import pad_input, repeat_kv, repeat_kv_backward, unpad_input
    g = torch.Generator().manual_seed(0)
    x = torch.randn(3, 5, 2, 4, generator=g)
    mask = torch.tensor([[1, 1, 1, 0, 0], [1, 1, 1, 1, 1], [0, 0, 1, 1, 0]])
    rows, indices, cu, longest = unpad_input(x, mask)
    assert rows.shape == (10, 2, 4) and longest == 5 and cu.dtype == torch.int32 and cu.tolist() == [0, 3, 8, 10]
    assert indices.tolist() == [0, 1, 2, 5, 6, 7, 8, 9, 12, 13]
    back = pad_input(rows, indices, 3, 5)
    assert torch.equal(back, x * mask[:, :, None, None])
    # keyword names of the reference's signatures
    h = torch.randn(2, 2, 3, 4, generator=g)
    r = repeat_kv(hidden_states=h, n_rep=3)
    assert r.shape == (2, 6, 3, 4) and torch.equal(r[:, 3:6], h[:, 1:2].expand(2, 3, 3, 4))
    assert torch.allclose(repeat_kv_backward(grad_output=r, n_rep=3), 3 * h)


def test_lora_scaling_other_than_one_is_refused():
    """The fused layers apply no LoRA scaling, like the reference (run_gsm8k.py:373-374 refuses lora_alpha != rank)."""
    from hyclora_amd.models.fused_decoder_layer import lora_linear_parts
    lin = SimpleNamespace(base_layer=1, lora_A=2, lora_B=3)
    assert lora_linear_parts(lin) == (1, 2, 3)
    lin.scaling = {"default": 1.0}
    assert lora_linear_parts(lin) == (1, 2, 3)
    lin.scaling = {"default": 2.0}
    with pytest.raises(ValueError):
        lora_linear_parts(lin)


def test_install_on_a_stock_model_routes_by_training_mode():
    """hyclora_amd.models.hf.install on the CPU: evaluation keeps the stock layers (same bits as before); a
    training-mode step reaches the fused layers, which refuse CPU tensors (there is no fallback path)."""
    transformers = pytest.importorskip("transformers")
    from hyclora_amd.models import hf, llama
    cfg = transformers.LlamaConfig(vocab_size=64, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                                   num_attention_heads=2, num_key_value_heads=2, max_position_embeddings=64,
                                   attn_implementation="eager")
    torch.manual_seed(0)
    model = transformers.LlamaForCausalLM(cfg).eval()
    ids = torch.randint(0, 64, (2, 8))
    with torch.no_grad():
        before = model(input_ids=ids).logits
        hf.install(model, CFG)
        assert all(isinstance(layer.fused_llama_layer, llama.FusedLlamaLayerIntraInter) for layer in model.model.layers)
        assert torch.equal(model(input_ids=ids).logits, before)
    model.train()
    with pytest.raises((RuntimeError, AttributeError)):          # no LoRA wrappers / no GPU: the fused path is taken and fails loudly
        model(input_ids=ids, use_cache=False)
    with pytest.raises(ValueError):
        hf.install(SimpleNamespace(config=SimpleNamespace(model_type="gpt2")), CFG)
    with pytest.raises(ValueError):
        hf.install(SimpleNamespace(config=SimpleNamespace(model_type="mistral")), CFG, map_free=True)
