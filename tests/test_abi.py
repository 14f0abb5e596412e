"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol the
public header declares, and rejects bad arguments with the documented codes before
anything is launched."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def L():
    import hyclora_amd  # noqa: F401
    from hyclora_amd import _lib
    if not _lib.LIB_PATH.exists():
        from importlib import import_module
        import_module("__graft_entry__").build()
    return _lib


def header_functions():
    text = (ROOT / "include" / "hyclora.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hyc_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(L):
    names = header_functions()
    assert names, "no declarations found in include/hyclora.h"
    handle = L.lib()
    for n in names:
        assert hasattr(handle, n), f"{n} declared in hyclora.h but not exported by libhyclora.so"
    assert sorted(L.declared_symbols()) == names, "ctypes signature table and header disagree"


def test_error_strings(L):
    assert L.error_string(0) == "ok"
    for code in range(-8, 0):
        assert L.error_string(code) not in ("ok", "unknown error code")
    assert L.error_string(-99) == "unknown error code"
    assert L.lib().hyc_abi_version() == L.ABI_VERSION


def test_argument_validation_without_launch(L):
    h = L.lib()
    fake = ctypes.c_void_p(0x1000)     # never dereferenced: validation fails first
    common = (2, 4, 64, 256, 64, 64, 0)
    assert h.hyc_quant_pack(fake, fake, None, fake, None, 0, None, 0, *common, 3, None) == -2
    assert h.hyc_quant_pack(fake, fake, None, fake, None, 0, None, 0, 2, 4, 48, 192, 48, 48, 0, 4, None) == -3
    assert h.hyc_quant_pack(None, fake, None, fake, None, 0, None, 0, *common, 4, None) == -1
    assert h.hyc_quant_pack(fake, fake, None, fake, None, 3, None, 0, *common, 4, None) == -1
    assert h.hyc_quant_pack(ctypes.c_void_p(0x1004), fake, None, fake, None, 0, None, 0, *common, 4, None) == -4
    assert h.hyc_quant_pack(fake, fake, None, fake, None, 0, None, 0, 2, 4, 64, 250, 64, 64, 0, 4, None) == -4
    assert h.hyc_unpack_dequant(fake, fake, None, fake, None, 0, None, *common, 16, None) == -2
    assert h.hyc_unpack_dequant(fake, None, None, fake, None, 0, None, *common, 8, None) == -1
    # empty tensors are accepted and do nothing
    assert h.hyc_quant_pack(None, None, None, None, None, 0, None, 0, 0, 4, 64, 256, 64, 64, 0, 4, None) == 0
    assert h.hyc_set_tuning(b"no_such_key", 1) == -8
    assert h.hyc_set_tuning(b"quant_rows_per_wave", 0) == -8
    # the knobs are process-wide: put the default back so later tests run with it
    try:
        assert h.hyc_set_tuning(b"quant_rows_per_wave", 16) == 0
    finally:
        assert h.hyc_set_tuning(b"quant_rows_per_wave", 8) == 0


def test_argument_validation_of_the_newer_entry_points(L):
    """Error codes that come back before any launch (fake pointers are never dereferenced)."""
    h = L.lib()
    fake = ctypes.c_void_p(0x1000)
    one_ptr = (ctypes.c_void_p * 1)(0x1000)
    five_ptr = (ctypes.c_void_p * 5)(*[0x1000] * 5)
    rank = lambda *r: (ctypes.c_int64 * len(r))(*r)

    def norm_lora(rows, n, n_adapters, weights, ranks, outs):
        return h.hyc_rmsnorm_fwd_compress_lora(fake, fake, fake, fake, rows, n, 1e-5, 4, None, None, None, None, None, 0,
                                               None, n_adapters, weights, ranks, outs, None)
    assert norm_lora(8, 1024, 0, one_ptr, rank(16), one_ptr) == -8               # no adapter
    assert norm_lora(8, 1024, 5, five_ptr, rank(16, 16, 16, 16, 16), five_ptr) == -8
    assert norm_lora(8, 1024, 1, one_ptr, rank(0), one_ptr) == -5                # rank out of range
    assert norm_lora(8, 1024, 1, one_ptr, rank(65), one_ptr) == -5
    two_ptr = (ctypes.c_void_p * 2)(0x1000, 0x1000)
    assert norm_lora(8, 1024, 2, two_ptr, rank(48, 32), two_ptr) == -5           # five 16-row blocks
    assert norm_lora(8, 1056, 1, one_ptr, rank(16), one_ptr) == -3               # not whole 512-column slabs
    assert norm_lora(7, 1024, 1, one_ptr, rank(16), one_ptr) == -3               # odd row count
    assert norm_lora(8, 1024, 1, None, rank(16), one_ptr) == -1
    assert norm_lora(8, 1024, 1, (ctypes.c_void_p * 1)(0x1008), rank(16), one_ptr) == -4   # adapter rows not 16-byte aligned
    # bounded compaction: a negative capacity is a shape error, no room at all is a no-op
    assert h.hyc_sparse_write_bounded(fake, 4096, fake, 0, fake, -1, fake, fake, None) == -3
    assert h.hyc_sparse_write_bounded(fake, 4096, fake, 0, fake, 0, fake, fake, None) == 0
    assert h.hyc_sparse_write_bounded(None, 4096, fake, 0, fake, 10, fake, fake, None) == -1
    # the entry point with its own scratch memory: sizes first
    assert h.hyc_rmsnorm_bwd_static(fake, fake, fake, 0, fake, fake, fake, 16, 8200, None) == -7
    assert h.hyc_rmsnorm_bwd_static(fake, fake, fake, 0, fake, fake, None, 16, 64, None) == -1
    assert h.hyc_rmsnorm_bwd_static_max_bytes() == 512 * 8192 * 4


def test_missing_library_is_an_error(L, monkeypatch, tmp_path):
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", tmp_path / "libhyclora.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        L.lib()
