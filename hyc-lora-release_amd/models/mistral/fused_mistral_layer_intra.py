"""The reference's module name for this class (models/mistral/fused_mistral_layer_intra.py), so that its model file's import line
`from .fused_mistral_layer_intra import FusedMistralLayerIntra` only needs the package prefix changed."""
from . import FusedMistralLayerIntra  # noqa: F401
