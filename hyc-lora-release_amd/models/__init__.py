"""Host-side fused decoder layers that save compressed activations (reference: models/*/fused_*_layer_*.py).

One generic implementation (`fused_decoder_layer.py`) serves the Llama, Mistral and long-sequence
(no attention map) variants and the layer types (baseline, intra, intra_inter, intra_inter_full_fuse); the reference's class names are exported from
`llama.py`, `mistral.py` and `llama_flash_attn.py`.  `roberta.py` holds the encoder layers (LayerNorm,
GELU; reference: models/roberta/fused_roberta_layer_*.py)."""
from .llama import (FusedLlamaLayerBaseline, FusedLlamaLayerIntra, FusedLlamaLayerIntraInter,  # noqa: F401
                    FusedLlamaLayerIntraInterFullFuse)
from .mistral import (FusedMistralLayerBaseline, FusedMistralLayerIntra, FusedMistralLayerIntraInter,  # noqa: F401
                      FusedMistralLayerIntraInterFullFuse)
from .roberta import FusedRobertaLayer, FusedRobertaLayerBaseline, FusedRobertaLayerIntra, FusedRobertaLayerIntraInter  # noqa: F401
