"""hyclora_amd — HyC-LoRA's activation-compression hot path on MI355X (gfx950).

The directory is named after the upstream project and is not a valid Python identifier;
import it through the top-level `hyclora_amd` module, which registers this package under
that name.
"""
from . import _lib  # noqa: F401

__all__ = ["_lib", "operators"]
