"""The reference's module name for this class (models/llama/fused_llama_layer_intra_inter_full_fuse.py), so that its model file's import line
`from .fused_llama_layer_intra_inter_full_fuse import FusedLlamaLayerIntraInterFullFuse` only needs the package prefix changed."""
from . import FusedLlamaLayerIntraInterFullFuse  # noqa: F401
