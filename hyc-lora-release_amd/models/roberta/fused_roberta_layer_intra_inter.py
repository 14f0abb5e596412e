"""The reference's module name for this class (models/roberta/fused_roberta_layer_intra_inter.py), so that its model file's import line
`from .fused_roberta_layer_intra_inter import FusedRobertaLayerIntraInter` only needs the package prefix changed."""
from . import FusedRobertaLayerIntraInter  # noqa: F401
