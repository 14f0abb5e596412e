"""Mistral decoder layers (grouped-query attention: 32 query / 8 key-value heads); class names as in
the reference (models/mistral/fused_mistral_layer_*.py).  The computation is the generic layer: the
reference's Mistral files differ from the Llama ones only in always calling repeat_kv and in a dtype
cast of lora_B (fused_mistral_layer_intra_inter_full_fuse.py:226-227), both covered there."""
from ..fused_decoder_layer import FusedDecoderLayer, call_from_decoder_layer


class FusedMistralLayerBaseline(FusedDecoderLayer):
    layer_type = "baseline"


class FusedMistralLayerIntra(FusedDecoderLayer):
    layer_type = "intra"


class FusedMistralLayerIntraInter(FusedDecoderLayer):
    layer_type = "intra_inter"


class FusedMistralLayerIntraInterFullFuse(FusedDecoderLayer):
    layer_type = "intra_inter_full_fuse"


LAYER_TYPES = {
    "baseline": FusedMistralLayerBaseline,
    "intra": FusedMistralLayerIntra,
    "intra_inter": FusedMistralLayerIntraInter,
    "intra_inter_full_fuse": FusedMistralLayerIntraInterFullFuse,
}


def make_fused_mistral_layer(hyclora_config):
    try:
        layer = LAYER_TYPES[hyclora_config.layer_type]()
    except KeyError:
        raise ValueError(f"Unknown layer type: {hyclora_config.layer_type}") from None
    layer.set_hyclora_config(hyclora_config)
    return layer


def set_fused_mistral_layer(model, hyclora_config):
    """MistralForCausalLM.set_fused_mistral_layer of the reference as a function of the model
    (models/mistral/modeling_mistral.py:998-1027): a configured fused layer per decoder layer, as
    `fused_mistral_layer`."""
    if hyclora_config.layer_type not in LAYER_TYPES:
        raise ValueError(f"Unknown layer type: {hyclora_config.layer_type} (available: {sorted(LAYER_TYPES)})")
    model.hyclora_config = hyclora_config
    for layer in model.model.layers:
        layer.fused_mistral_layer = make_fused_mistral_layer(hyclora_config)


def decoder_layer_forward(decoder_layer, hidden_states, attention_mask, cos, sin):
    """What the reference's decoder layer does in training mode (models/mistral/modeling_mistral.py:611-646): one call of the layer's
    `fused_mistral_layer` with the layer's own weights.  `decoder_layer` is a decoder layer with the stock attribute names
    whose linears are PEFT-style LoRA wrappers (`base_layer`, `lora_A`, `lora_B`)."""
    return call_from_decoder_layer(decoder_layer.fused_mistral_layer, decoder_layer, hidden_states, attention_mask, cos, sin)
