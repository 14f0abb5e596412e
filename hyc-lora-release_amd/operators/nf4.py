"""NF4 weight dequantisation on gfx950 for bitsandbytes-format frozen weights (the reference calls
bitsandbytes.functional.dequantize_nf4, models/utils/compute_utils.py:19, :29; bitsandbytes 0.43.2).

`dequantize_nf4(w, quant_state)` takes the packed uint8 weight and any object with the attributes of
bitsandbytes' QuantState (`absmax, shape, dtype, blocksize, quant_type, code`, and for double
quantisation `nested, offset, state2.absmax, state2.code, state2.blocksize`), so a 4-bit checkpoint
loads and runs without bitsandbytes being importable."""
from types import SimpleNamespace

import torch

from .. import _lib

# The 16 NF4 levels (QLoRA, Dettmers et al. 2023, appendix E; bitsandbytes functional.py get_4bit_type('nf4')).
NF4_TABLE = (-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635,
             -0.18477343022823334, -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725,
             0.24611230194568634, 0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
             0.7229568362236023, 1.0)


_DEFAULT_TABLE = {}      # device -> the NF4 levels as a float32 tensor there


def _default_table(dev):
    """The NF4 levels on `dev`, uploaded once: a host tensor copied at every call would make each
    dequantisation wait for the stream to drain (a pageable host-to-device copy is synchronous)."""
    t = _DEFAULT_TABLE.get(dev)
    if t is None:
        t = _DEFAULT_TABLE[dev] = torch.tensor(NF4_TABLE, dtype=torch.float32).to(dev)
    return t


def make_quant_state(absmax, shape, blocksize=64, dtype=torch.bfloat16, code=None, offset=None, state2=None):
    """A plain stand-in for bitsandbytes.functional.QuantState with the fields dequantize_nf4 reads."""
    return SimpleNamespace(absmax=absmax, shape=torch.Size(shape), dtype=dtype, blocksize=blocksize, quant_type="nf4",
                           code=code, nested=state2 is not None, offset=offset, state2=state2)


def dequantize_nf4(w, quant_state):
    """Dense bf16 tensor of quant_state.shape from the packed NF4 weight `w` (uint8, two codes per byte)."""
    _lib.require_gpu(w)
    qs = quant_state
    if getattr(qs, "quant_type", "nf4") != "nf4":
        raise NotImplementedError(f"only the nf4 code book is supported, got {qs.quant_type!r}")
    if getattr(qs, "dtype", torch.bfloat16) != torch.bfloat16:
        raise NotImplementedError("dequantize_nf4 produces bfloat16 weights")
    dev = w.device
    n = 1
    for d in qs.shape:
        n *= int(d)
    packed = w.reshape(-1).contiguous()
    if packed.dtype != torch.uint8 or packed.numel() * 2 != n:
        raise ValueError(f"{packed.numel()} packed bytes do not hold {n} 4-bit codes")
    table = getattr(qs, "code", None)
    table = _default_table(dev) if table is None else table.to(device=dev, dtype=torch.float32).contiguous()
    if table.numel() != 16:
        raise ValueError("the 4-bit code book must have 16 entries")
    out = torch.empty(n, device=dev, dtype=torch.bfloat16)
    nested = bool(getattr(qs, "nested", False))
    if nested:
        absmax = qs.absmax.reshape(-1).contiguous()
        s2 = qs.state2
        code2 = s2.code.to(device=dev, dtype=torch.float32).contiguous()
        absmax2 = s2.absmax.to(device=dev, dtype=torch.float32).reshape(-1).contiguous()
        if absmax.dtype != torch.uint8 or code2.numel() != 256:
            raise ValueError("nested statistics must be uint8 codes with a 256-entry code book")
        offset = None
        if qs.offset is not None:                            # a device scalar: no host read-back
            offset = torch.as_tensor(qs.offset).to(device=dev, dtype=torch.float32).reshape(-1).contiguous()
        bs2 = int(s2.blocksize)
    else:
        absmax = qs.absmax.to(torch.float32).reshape(-1).contiguous()
        code2 = absmax2 = None
        offset, bs2 = None, 1
    nblocks = -(-n // int(qs.blocksize))
    if absmax.numel() < nblocks or (nested and absmax2.numel() < -(-nblocks // bs2)):
        raise ValueError("not enough block statistics for the weight")
    _lib.call("hyc_nf4_dequant", packed.data_ptr(), absmax.data_ptr(), int(nested), _lib.ptr(code2), _lib.ptr(absmax2),
              _lib.ptr(offset), bs2, table.data_ptr(), out.data_ptr(), n, int(qs.blocksize), _lib.stream_of(w))
    return out.reshape(tuple(qs.shape))
