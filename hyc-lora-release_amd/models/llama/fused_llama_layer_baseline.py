"""The reference's module name for this class (models/llama/fused_llama_layer_baseline.py), so that its model file's import line
`from .fused_llama_layer_baseline import FusedLlamaLayerBaseline` only needs the package prefix changed."""
from . import FusedLlamaLayerBaseline  # noqa: F401
