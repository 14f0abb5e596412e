"""The reference's module name for this class (models/roberta/fused_roberta_layer_intra.py), so that its model file's import line
`from .fused_roberta_layer_intra import FusedRobertaLayerIntra` only needs the package prefix changed."""
from . import FusedRobertaLayerIntra  # noqa: F401
