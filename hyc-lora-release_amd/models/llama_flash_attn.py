"""Long-sequence Llama layers: no attention map is materialised or saved, q/k main are quantised
with a zero point, norm weights receive gradients
(models/llama_flash_attn/fused_llama_layer_{baseline,intra,intra_inter}.py).  The flash-attn varlen kernels
of the reference are replaced by the flash kernels behind torch's scaled_dot_product_attention, called
through their aten entry points: forward returns the log-sum-exps, backward takes them and the
dequantised attention output, as the reference's call does (…intra_inter.py:450-468)."""
from .fused_decoder_layer import FusedDecoderLayer


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
