"""Import shim: makes the package in `hyc-lora-release_amd/` importable as `hyclora_amd`.

    import hyclora_amd
    from hyclora_amd.operators.compress_function import compression_quantization
"""
import importlib.util
import sys
from pathlib import Path

_pkg_dir = Path(__file__).resolve().parent / "hyc-lora-release_amd"
_spec = importlib.util.spec_from_file_location(
    "hyclora_amd", _pkg_dir / "__init__.py", submodule_search_locations=[str(_pkg_dir)])
_module = importlib.util.module_from_spec(_spec)
sys.modules["hyclora_amd"] = _module
_spec.loader.exec_module(_module)
