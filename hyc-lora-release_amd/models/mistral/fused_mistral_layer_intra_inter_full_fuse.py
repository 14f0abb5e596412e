"""The reference's module name for this class (models/mistral/fused_mistral_layer_intra_inter_full_fuse.py), so that its model file's import line
`from .fused_mistral_layer_intra_inter_full_fuse import FusedMistralLayerIntraInterFullFuse` only needs the package prefix changed."""
from . import FusedMistralLayerIntraInterFullFuse  # noqa: F401
