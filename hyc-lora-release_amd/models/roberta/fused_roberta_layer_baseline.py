"""The reference's module name for this class (models/roberta/fused_roberta_layer_baseline.py), so that its model file's import line
`from .fused_roberta_layer_baseline import FusedRobertaLayer` only needs the package prefix changed."""
from . import FusedRobertaLayer  # noqa: F401
