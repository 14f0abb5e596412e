"""Long-sequence Llama layers: no attention map is materialised or saved, q/k main are quantised
with a zero point, norm weights receive gradients
(models/llama_flash_attn/fused_llama_layer_{baseline,intra,intra_inter}.py).  The flash-attn varlen kernels
of the reference are replaced by the flash kernels behind torch's scaled_dot_product_attention, called
through their aten entry points: forward returns the log-sum-exps, backward takes them and the
dequantised attention output, as the reference's call does (…intra_inter.py:450-468)."""
from ..fused_decoder_layer import FusedDecoderLayer, call_from_decoder_layer


class FusedLlamaLayerBaseline(FusedDecoderLayer):
    layer_type = "baseline"
    attention = "sdpa"


class FusedLlamaLayerIntra(FusedDecoderLayer):
    layer_type = "intra"
    attention = "sdpa"


class FusedLlamaLayerIntraInter(FusedDecoderLayer):
    layer_type = "intra_inter"
    attention = "sdpa"


class FusedLlamaLayerIntraInterFullFuse(FusedDecoderLayer):
    """Not present in the reference's flash variant; the fused MLP kernels apply unchanged."""
    layer_type = "intra_inter_full_fuse"
    attention = "sdpa"


LAYER_TYPES = {
    "baseline": FusedLlamaLayerBaseline,
    "intra": FusedLlamaLayerIntra,
    "intra_inter": FusedLlamaLayerIntraInter,
    "intra_inter_full_fuse": FusedLlamaLayerIntraInterFullFuse,
}


def make_fused_llama_layer(hyclora_config):
    try:
        layer = LAYER_TYPES[hyclora_config.layer_type]()
    except KeyError:
        raise ValueError(f"Unknown layer type: {hyclora_config.layer_type}") from None
    layer.set_hyclora_config(hyclora_config)
    return layer


def set_fused_llama_layer(model, hyclora_config):
    """LlamaForCausalLM.set_fused_llama_layer of the reference's long-sequence model as a function of the
    model (models/llama_flash_attn/modeling_llama.py:1026-1053): a configured map-free fused layer per
    decoder layer, as `fused_llama_layer`."""
    if hyclora_config.layer_type not in LAYER_TYPES:
        raise ValueError(f"Unknown layer type: {hyclora_config.layer_type} (available: {sorted(LAYER_TYPES)})")
    model.hyclora_config = hyclora_config
    for layer in model.model.layers:
        layer.fused_llama_layer = make_fused_llama_layer(hyclora_config)


def decoder_layer_forward(decoder_layer, hidden_states, attention_mask, cos, sin):
    """What the reference's decoder layer does in training mode (models/llama_flash_attn/modeling_llama.py:610-654): one call of the layer's
    `fused_llama_layer` with the layer's own weights.  `decoder_layer` is a decoder layer with the stock attribute names
    whose linears are PEFT-style LoRA wrappers (`base_layer`, `lora_A`, `lora_B`)."""
    return call_from_decoder_layer(decoder_layer.fused_llama_layer, decoder_layer, hidden_states, attention_mask, cos, sin)
