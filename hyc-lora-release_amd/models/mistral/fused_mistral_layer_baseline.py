"""The reference's module name for this class (models/mistral/fused_mistral_layer_baseline.py), so that its model file's import line
`from .fused_mistral_layer_baseline import FusedMistralLayerBaseline` only needs the package prefix changed."""
from . import FusedMistralLayerBaseline  # noqa: F401
