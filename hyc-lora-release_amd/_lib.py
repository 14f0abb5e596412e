"""ctypes binding of libhyclora.so (the C ABI declared in include/hyclora.h).

The library is the only implementation: if it is missing, or a call returns an error
code, an exception is raised — there is no CPU or torch fallback.
"""
from __future__ import annotations

import ctypes
import weakref
from ctypes import c_char_p, c_int, c_int64, c_void_p
from pathlib import Path

import torch

_HERE = Path(__file__).resolve().parent
LIB_PATH = _HERE / "libhyclora.so"

_lib = None


class HycError(RuntimeError):
    """A C-ABI entry point returned a negative code."""

    def __init__(self, fn: str, code: int, text: str):
        super().__init__(f"{fn} failed: {text} (code {code})")
        self.code = code


# name -> (restype, argtypes)
ABI_VERSION = 11          # hyc_abi_version() of the library these signatures describe
_P, _I, _L = c_void_p, c_int, c_int64


class LoraAddMember(ctypes.Structure):
    """hyc_lora_add_member of include/hyclora.h: one operand set of a grouped LoRA-add launch."""
    _fields_ = [("xa", _P), ("b", _P), ("x", _P), ("scale", _P), ("zero_point", _P), ("q", _P), ("y", _P),
                ("cos_t", _P), ("sin_t", _P), ("seq_len", _L), ("stride_cos", _L), ("stride_sin", _L), ("N", _L),
                ("b_transposed", _I), ("table_is_fp32", _I)]


class LoraSumMember(ctypes.Structure):
    """hyc_lora_sum_member of include/hyclora.h: one term of hyc_lora_add_sum."""
    _fields_ = [("xa", _P), ("b", _P), ("b_transposed", _I), ("x", _P)]


_SIGNATURES = {
    "hyc_error_string": (c_char_p, [_I]),
    "hyc_abi_version": (_I, []),
    "hyc_set_tuning": (_I, [c_char_p, _I]),
    "hyc_quant_pack": (_I, [_P, _P, _P, _P, _P, _L, _P, _I, _L, _L, _L, _L, _L, _L, _L, _I, _P]),
    "hyc_unpack_dequant": (_I, [_P, _P, _P, _P, _P, _L, _P, _L, _L, _L, _L, _L, _L, _L, _I, _P]),
    "hyc_channel_stats_strips": (_L, [_L, _L]),
    "hyc_channel_stats": (_I, [_P, _L, _L, _L, _L, _L, _P, _L, _P]),
    "hyc_channel_select": (_I, [_P, _L, _L, _L, _I, _I, _P, _P, _P, _P]),
    "hyc_stream_probe": (_I, [_P, _I, _P, _I, _L, _L, _I, _I, _P]),
    "hyc_hist16": (_I, [_P, _L, _P, _P]),
    "hyc_hist_select": (_I, [_P, _L, _P, _P]),
    "hyc_sparse_num_segments": (_L, [_L]),
    "hyc_sparse_count": (_I, [_P, _L, _P, _I, _P, _P, _P]),
    "hyc_sparse_write": (_I, [_P, _L, _P, _I, _P, _P, _P, _P]),
    "hyc_sparse_write_bounded": (_I, [_P, _L, _P, _I, _P, _L, _P, _P, _P]),
    "hyc_sparse_segment_offsets": (_I, [_P, _L, _L, _P, _P]),
    "hyc_sparse_restore": (_I, [_P, _P, _P, _L, _P, _P]),
    "hyc_softmax_bwd": (_I, [_P, _P, _P, _L, _L, _P]),
    "hyc_nf4_dequant": (_I, [_P, _P, _I, _P, _P, _P, _L, _P, _P, _L, _L, _P]),
    "hyc_layernorm_fwd": (_I, [_P, _P, _P, _I, _P, _P, _P, _L, _L, ctypes.c_float, _P]),
    "hyc_layernorm_bwd": (_I, [_P, _P, _P, _I, _P, _P, _P, _L, _L, _P]),
    "hyc_outlier_table": (_I, [_P, _L, _L, _P, _P]),
    "hyc_rmsnorm_fwd_compress": (_I, [_P, _P, _I, _P, _P, _L, _L, ctypes.c_float, _I, _P, _P, _P, _P, _P, _L, _P, _P]),
    "hyc_rmsnorm_fwd_compress_lora": (_I, [_P, _P, _P, _P, _L, _L, ctypes.c_float, _I, _P, _P, _P, _P, _P, _L, _P,
                                           _I, _P, _P, _P, _P]),
    "hyc_rope": (_I, [_P, _P, _P, _I, _L, _L, _L, _L, _L, _L, _L, _L, _L, _I, _P]),
    "hyc_softmax_fwd": (_I, [_P, _P, _P, _L, _L, ctypes.c_float, _L, _L, _L, _L, _P, _P, _P, _P]),
    "hyc_softmax_bwd_restore": (_I, [_P, _P, _P, _P, _P, _P, _L, _L, ctypes.c_float, _P]),
    "hyc_rmsnorm_fwd": (_I, [_P, _P, _I, _P, _P, _L, _L, ctypes.c_float, _P]),
    "hyc_rmsnorm_bwd_workspace": (_L, [_L, _L]),
    "hyc_rmsnorm_bwd": (_I, [_P, _P, _P, _I, _P, _P, _P, _P, _L, _L, _L, _P]),
    "hyc_rmsnorm_bwd_static_max_bytes": (_L, []),
    "hyc_rmsnorm_bwd_static": (_I, [_P, _P, _P, _I, _P, _P, _P, _L, _L, _P]),
    "hyc_rmsnorm_bwd_add": (_I, [_P, _P, _P, _I, _P, _P, _P, _P, _P, _L, _L, _L, _P]),
    "hyc_rmsnorm_bwd_codes": (_I, [_P, _P, _P, _P, _L, _P, _I, _P, _I, _P, _P, _P, _L, _L, _P]),
    "hyc_silu_bwd": (_I, [_P, _P, _P, _L, _P]),
    "hyc_silu_mul": (_I, [_P, _P, _P, _L, _P]),
    "hyc_silu_once_mul": (_I, [_P, _P, _P, _L, _P]),
    "hyc_silu_mul_bwd": (_I, [_P, _P, _P, _P, _P, _L, _P]),
    "hyc_gelu_bwd": (_I, [_P, _P, _P, _L, _P]),
    "hyc_lora_silu_mul_fwd": (_I, [_P] * 11 + [_L, _L, _L, _I, _I, _P]),
    "hyc_lora_silu_mul_bwd": (_I, [_P] * 12 + [_L, _L, _L, _I, _I, _P]),
    "hyc_lora_contract_workspace": (_L, [_L, _L, _L, _I, _I]),
    "hyc_lora_contract": (_I, [_P, _P, _P, _P, _I, _P, _P, _I, _P, _I, _P, _P, _L, _L, _L, _L, _P]),
    "hyc_lora_add": (_I, [_P, _P, _I, _P, _P, _P, _L, _L, _L, _P]),
    "hyc_lora_add_quant": (_I, [_P, _P, _I] + [_P] * 5 + [_L, _L, _L, _I, _P]),
    "hyc_lora_add_restore": (_I, [_P, _P, _I] + [_P] * 4 + [_L, _L, _L, _I, _P]),
    "hyc_lora_add_quant_rope": (_I, [_P, _P, _I] + [_P] * 7 + [_I, _L, _L, _L, _L, _L, _L, _I, _P]),
    "hyc_lora_add_restore_rope": (_I, [_P, _P, _I] + [_P] * 6 + [_I, _L, _L, _L, _L, _L, _L, _I, _P]),
    "hyc_lora_add_sum": (_I, [_P, _I, _P, _L, _L, _L, _P]),
    "hyc_lora_add_quant_group": (_I, [_P, _I, _L, _L, _I, _P]),
    "hyc_lora_add_restore_group": (_I, [_P, _I, _L, _L, _I, _P]),
}


def declared_symbols():
    return sorted(_SIGNATURES)


def lib() -> ctypes.CDLL:
    """Load the kernel library once; fail loudly when it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} not found: build it with `python {(_HERE / 'build.py')}` "
                "(hipcc, gfx950). There is no fallback implementation.")
        handle = ctypes.CDLL(str(LIB_PATH))
        handle.hyc_abi_version.restype = ctypes.c_int
        have = handle.hyc_abi_version()
        if have != ABI_VERSION:
            # calling through signatures of another revision would hand kernels misplaced arguments
            raise RuntimeError(f"{LIB_PATH} has ABI revision {have}, these bindings are written for {ABI_VERSION}: "
                               f"rebuild it with `python {(_HERE / 'build.py')}`")
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def error_string(code: int) -> str:
    return lib().hyc_error_string(code).decode()


def call(name: str, *args) -> None:
    rc = getattr(lib(), name)(*args)
    if rc != 0:
        raise HycError(name, rc, error_string(rc))


def ptr(t):
    """Device address of a tensor (None -> NULL)."""
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_of(t: torch.Tensor):
    """The HIP stream torch is currently enqueuing on for t's device.  Asked of torch's C layer
    directly where it offers that: building a torch.cuda.Stream object per launch costs about as
    much host time as the launch itself."""
    if _raw_stream is not None:
        index = t.device.index
        return _raw_stream(torch.cuda.current_device() if index is None else index)
    return torch.cuda.current_stream(t.device).cuda_stream


def require_gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("hyclora kernels run on the GPU only; got a tensor on " + str(t.device))


def set_tuning(key: str, value: int) -> None:
    call("hyc_set_tuning", key.encode(), int(value))


_BF16_VECTORS = {}       # id(tensor) -> (weak reference to it, its version, its bfloat16 copy)


def bf16_vector(t: torch.Tensor) -> torch.Tensor:
    """`t.to(bfloat16).reshape(-1)` for a per-channel vector that is not bfloat16 (a frozen zero point is kept as the
    running mean of int8 values, a float tensor), converted once per tensor object: the frozen statistics are the
    same objects step after step, and a conversion kernel per use costs a launch each.  The copy is kept with the
    tensor (weakly) and made again when the tensor has been modified in place."""
    if t.dtype == torch.bfloat16:
        return t.reshape(-1)
    key = id(t)
    hit = _BF16_VECTORS.get(key)
    if hit is not None and hit[0]() is t and hit[1] == t._version:
        return hit[2]
    conv = t.to(torch.bfloat16).reshape(-1).contiguous()
    _BF16_VECTORS[key] = (weakref.ref(t, lambda _r, k=key: _BF16_VECTORS.pop(k, None)), t._version, conv)
    return conv
