"""Shared test utilities: seeded inputs shaped like the benchmark configurations, the
scalar C oracle binding and the tolerance metric."""
import ctypes
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parent.parent
BF16 = torch.bfloat16


def bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> uint16 bit patterns (numpy)."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(BF16)


def same_bits(a: torch.Tensor, b: torch.Tensor) -> bool:
    return a.shape == b.shape and np.array_equal(bits(a), bits(b))


def activation_with_outlier_channels(seed, shape=(2, 512, 4096), frac=0.005, gain=50.0):
    """benchmark configuration 1: N(0,1) values, a fixed random 0.5 % of channels scaled x50.
    Returns (x bf16, planted channel indices sorted)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=g)
    n = shape[-1]
    k = int(n * frac)
    planted = torch.randperm(n, generator=g)[:k]
    x[..., planted] *= gain
    return x.to(BF16), torch.sort(planted).values


def rel_err_and_cos(a: torch.Tensor, b: torch.Tensor):
    """(max |a-b| / max |b|, cosine similarity) in float64 — the bf16 tolerance metric:
    max rel err <= 1e-2 and cosine >= 0.9999."""
    a = a.detach().cpu().double().flatten()
    b = b.detach().cpu().double().flatten()
    denom = b.abs().max().clamp_min(1e-30)
    rel = ((a - b).abs().max() / denom).item()
    cos = (torch.dot(a, b) / (a.norm() * b.norm()).clamp_min(1e-30)).item()
    return rel, cos


def assert_close_bf16(a, b, rel_tol=1e-2, cos_tol=0.9999, what=""):
    rel, cos = rel_err_and_cos(a, b)
    assert rel <= rel_tol and cos >= cos_tol, f"{what}: max rel err {rel:.3e}, cosine {cos:.6f}"


_scalar = None


def scalar_ref():
    """ctypes handle of oracle/_build/libscalar_ref.so (built on demand)."""
    global _scalar
    if _scalar is None:
        so = ROOT / "oracle" / "_build" / "libscalar_ref.so"
        if not so.exists():
            import importlib.util
            spec = importlib.util.spec_from_file_location("oracle_build", ROOT / "oracle" / "build.py")
            m = importlib.util.module_from_spec(spec)
            spec.loader.exec_module(m)
            m.build(verbose=False)
        _scalar = ctypes.CDLL(str(so))
    return _scalar


def scalar_quant_pack(x, s, z, q_bit):
    B, M, N = x.shape
    xb, sb = bits(x), bits(s.reshape(-1))
    zb = None if z is None else bits(z.to(BF16).reshape(-1))
    out = np.zeros((B, M, N * q_bit // 8), dtype=np.uint8)
    scalar_ref().ref_quant_pack(
        xb.ctypes.data_as(ctypes.c_void_p), sb.ctypes.data_as(ctypes.c_void_p),
        None if zb is None else zb.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p),
        ctypes.c_long(B), ctypes.c_long(M), ctypes.c_long(N), ctypes.c_int(q_bit))
    return torch.from_numpy(out)


def scalar_unpack_dequant(q, s, z, q_bit):
    B, M, nb = q.shape
    N = nb * 8 // q_bit
    qb = q.cpu().contiguous().numpy()
    sb = bits(s.reshape(-1))
    zb = None if z is None else bits(z.to(BF16).reshape(-1))
    out = np.zeros((B, M, N), dtype=np.uint16)
    scalar_ref().ref_unpack_dequant(
        qb.ctypes.data_as(ctypes.c_void_p), sb.ctypes.data_as(ctypes.c_void_p),
        None if zb is None else zb.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p),
        ctypes.c_long(B), ctypes.c_long(M), ctypes.c_long(N), ctypes.c_int(q_bit))
    return from_bits(out)


def layer_saved_state(out: torch.Tensor, heads: int) -> dict:
    """What a fused decoder layer kept for backward, read off the autograd node of its output and renamed to
    the reference's save-list names (the keys oracle/layer_oracle.py's backward reads).  Call it before
    backward runs: the node drops its tensors afterwards.  The attention map's lists are cut to the entries
    that were written (the layer may have sized them with headroom)."""
    node = out.grad_fn
    raw = dict(zip(node.names, node.saved_tensors))
    prefix = {"q_rope": "q", "k_rope": "k", "v_rep": "v", "o_lora_a": "o_final_lora_a"}
    suffix = {"_s": "_scale", "_z": "_zero_point", "_idx": "_channel_idx"}
    S = {}
    for name, t in raw.items():
        if name in ("a_idx", "a_val", "a_seg", "sdpa_rng", "sdpa_unused") or name.endswith("_raw"):
            continue
        for old, new in prefix.items():
            if name == old or name.startswith(old + "_"):
                name = new + name[len(old):]
                break
        for old, new in suffix.items():
            if name.endswith(old):
                name = name[:-len(old)] + new
                break
        S[name] = t
    if "sdpa_lse" in S:
        S["softmax_lse"] = S.pop("sdpa_lse")
    if "a_idx" in raw:
        nnz = int(raw["a_seg"][-1].item())
        S["a_o_indices"], S["a_o_values"] = raw["a_idx"][:nnz], raw["a_val"][:nnz]
        b, s = out.shape[0], out.shape[1]
        S["a_shape"] = (b, heads, s, s)
    return S
