"""The reference's module name for this class (models/llama_flash_attn/fused_llama_layer_intra.py), so that its model file's import line
`from .fused_llama_layer_intra import FusedLlamaLayerIntra` only needs the package prefix changed."""
from . import FusedLlamaLayerIntra  # noqa: F401
