"""The reference's module name for this class (models/llama/fused_llama_layer_intra_inter.py), so that its model file's import line
`from .fused_llama_layer_intra_inter import FusedLlamaLayerIntraInter` only needs the package prefix changed."""
from . import FusedLlamaLayerIntraInter  # noqa: F401
