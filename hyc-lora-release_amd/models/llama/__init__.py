"""Llama decoder layers with compressed saved activations; class names as in the reference
(models/llama/fused_llama_layer_{baseline,intra,intra_inter,intra_inter_full_fuse}.py)."""
from ..fused_decoder_layer import FusedDecoderLayer, call_from_decoder_layer


class FusedLlamaLayerBaseline(FusedDecoderLayer):
    layer_type = "baseline"


class FusedLlamaLayerIntra(FusedDecoderLayer):
    layer_type = "intra"


class FusedLlamaLayerIntraInter(FusedDecoderLayer):
    layer_type = "intra_inter"


class FusedLlamaLayerIntraInterFullFuse(FusedDecoderLayer):
    layer_type = "intra_inter_full_fuse"


LAYER_TYPES = {
    "baseline": FusedLlamaLayerBaseline,
    "intra": FusedLlamaLayerIntra,
    "intra_inter": FusedLlamaLayerIntraInter,
    "intra_inter_full_fuse": FusedLlamaLayerIntraInterFullFuse,
}


def make_fused_llama_layer(hyclora_config):
    """What LlamaForCausalLM.set_fused_llama_layer does per decoder layer
    (models/llama/modeling_llama.py:1151-1180): pick the class by `layer_type` and configure it."""
    try:
        layer = LAYER_TYPES[hyclora_config.layer_type]()
    except KeyError:
        raise ValueError(f"Unknown layer type: {hyclora_config.layer_type}") from None
    layer.set_hyclora_config(hyclora_config)
    return layer


def set_fused_llama_layer(model, hyclora_config):
    """LlamaForCausalLM.set_fused_llama_layer of the reference as a function of the model
    (models/llama/modeling_llama.py:1151-1180): every decoder layer in `model.model.layers` gets a configured
    fused layer of the configured type as its `fused_llama_layer`, which the decoder layer's forward calls
    while training (:745-786).  The configuration is kept on the model as `hyclora_config`."""
    if hyclora_config.layer_type not in LAYER_TYPES:
        raise ValueError(f"Unknown layer type: {hyclora_config.layer_type} (available: {sorted(LAYER_TYPES)})")
    model.hyclora_config = hyclora_config
    for layer in model.model.layers:
        layer.fused_llama_layer = make_fused_llama_layer(hyclora_config)


def decoder_layer_forward(decoder_layer, hidden_states, attention_mask, cos, sin):
    """What the reference's decoder layer does in training mode (models/llama/modeling_llama.py:745-786): one call of the layer's
    `fused_llama_layer` with the layer's own weights.  `decoder_layer` is a decoder layer with the stock attribute names
    whose linears are PEFT-style LoRA wrappers (`base_layer`, `lora_A`, `lora_B`)."""
    return call_from_decoder_layer(decoder_layer.fused_llama_layer, decoder_layer, hidden_states, attention_mask, cos, sin)
