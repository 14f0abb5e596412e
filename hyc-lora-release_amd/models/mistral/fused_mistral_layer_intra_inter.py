"""The reference's module name for this class (models/mistral/fused_mistral_layer_intra_inter.py), so that its model file's import line
`from .fused_mistral_layer_intra_inter import FusedMistralLayerIntraInter` only needs the package prefix changed."""
from . import FusedMistralLayerIntraInter  # noqa: F401
