"""Host-side fused decoder layers that save compressed activations (reference: models/*/fused_*_layer_*.py).

One generic implementation (`fused_decoder_layer.py`) serves the Llama, Mistral and long-sequence
(no attention map) variants and the layer types (baseline, intra, intra_inter, intra_inter_full_fuse); the reference's class names are exported from the
packages `llama`, `mistral` and `llama_flash_attn`, each of which also has the reference's module names
(`llama/fused_llama_layer_intra.py`, ...) and its model-level switch as a function
(`set_fused_llama_layer(model, cfg)`, ...).  `roberta` holds the encoder layers (LayerNorm, GELU; reference:
models/roberta/fused_roberta_layer_*.py)."""
from .llama import (FusedLlamaLayerBaseline, FusedLlamaLayerIntra, FusedLlamaLayerIntraInter,  # noqa: F401
                    FusedLlamaLayerIntraInterFullFuse)
from .mistral import (FusedMistralLayerBaseline, FusedMistralLayerIntra, FusedMistralLayerIntraInter,  # noqa: F401
                      FusedMistralLayerIntraInterFullFuse)
from .roberta import FusedRobertaLayer, FusedRobertaLayerBaseline, FusedRobertaLayerIntra, FusedRobertaLayerIntraInter  # noqa: F401
