"""Llama decoder layers with compressed saved activations; class names as in the reference
(models/llama/fused_llama_layer_{baseline,intra,intra_inter,intra_inter_full_fuse}.py)."""
from .fused_decoder_layer import FusedDecoderLayer


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
