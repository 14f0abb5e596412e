"""Host-side fused decoder layers that save compressed activations (reference: models/*/fused_*_layer_*.py).

One generic implementation (`fused_decoder_layer.py`) serves the Llama, Mistral and long-sequence
(no attention map) variants and the three layer types; the reference's class names are exported from
`llama.py`, `mistral.py` and `llama_flash_attn.py`.  `roberta.py` holds the encoder layers (LayerNorm,
GELU; reference: models/roberta/fused_roberta_layer_*.py)."""
from .llama import (FusedLlamaLayerIntra, FusedLlamaLayerIntraInter,  # noqa: F401
                    FusedLlamaLayerIntraInterFullFuse)
from .mistral import (FusedMistralLayerIntra, FusedMistralLayerIntraInter,  # noqa: F401
                      FusedMistralLayerIntraInterFullFuse)
from .roberta import FusedRobertaLayerIntra, FusedRobertaLayerIntraInter  # noqa: F401
