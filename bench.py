#!/usr/bin/env python3
"""Benchmark of the HyC-LoRA activation-compression hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload: benchmark configuration 2 — the activations of a Llama-2-7B-shaped MLP layer,
T = 4 x 1024 tokens, intermediate size 11008, LoRA rank 16, q_bit = 4, synthetic N(0,1) data.

A step = one compress (quantise + pack) followed by one decompress (unpack + dequantise) of
one [4, 1024, 11008] bf16 activation through the C ABI, inputs resident in HBM.  Successive
steps rotate over distinct buffers whose total size exceeds the 256 MiB last-level cache, so
every step streams from HBM.  `value` = algorithmic bytes of the round trip / time.

The same JSON line also carries
  roofline      the dominant kernel (quantise+pack, q=4) against the 8 TB/s HBM peak, its
                launch time measured with HIP events on the launching stream;
  cpu_baseline  the CPU oracle (a port: the reference has no CPU implementation of its Triton
                kernels) timed on the host cores on the same tensor;
  fused         fused LoRA-SiLU-Hadamard forward+backward ms against unfused bf16 torch;
  kernels       achieved GB/s of the other kernels of the path.
"""
import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0
SETTLE_MS = 60.0          # every timed arm first runs its own kernels this long: the GPU reaches its
                          # steady clocks only after tens of milliseconds of work, whatever --warmup says
# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# `bench.py --only quant` and `--only copy`; `bench.py --pmc-summary DIR` writes this file from their
# CSVs together with a hash of the kernel sources it was measured on.
TRAFFIC_JSON = ROOT / "profiles" / "quant_pack_q4_config2_hbm_traffic.json"
TRAFFIC_SOURCES = ["quant_pack.hip", "hyc_pack.hpp", "hyc_quant_math.h", "hyc_common.hpp"]


def kernel_source_hash():
    import hashlib
    h = hashlib.sha256()
    for name in TRAFFIC_SOURCES:
        h.update((ROOT / "hyc-lora-release_amd" / "csrc" / name).read_bytes())
    return h.hexdigest()[:16]


def measured_traffic():
    """(bytes per launch or None, note): the counter measurement is only quoted while the kernel
    sources are the ones it was taken on."""
    if not TRAFFIC_JSON.exists():
        return None, "no counter measurement committed"
    rec = json.loads(TRAFFIC_JSON.read_text())
    if rec.get("source_sha256_16") != kernel_source_hash():
        return None, f"counter measurement is of other kernel sources ({rec.get('source_sha256_16')}); re-run the pmc passes"
    return int(rec["traffic_bytes"]), f"rocprofv3 FETCH_SIZE/WRITE_SIZE at commit {rec.get('commit', '?')}, scale factors {rec['fetch_scale']:.5f}/{rec['write_scale']:.5f}"


def pmc_summary(directory):
    """Reads DIR/pmc_{quant,copy}_{FETCH_SIZE,WRITE_SIZE}/**/*counter_collection.csv (one rocprofv3
    --pmc run each of `bench.py --only quant` / `--only copy`) and writes TRAFFIC_JSON: KiB per
    dispatch of the quantiser, each counter scaled by what it reads for a plain copy of known size."""
    import csv
    import glob
    import statistics
    import subprocess

    def median(mode, counter, match):
        files = glob.glob(f"{directory}/pmc_{mode}_{counter}/**/*counter_collection.csv", recursive=True)
        if not files:
            raise SystemExit(f"no counter CSV under {directory}/pmc_{mode}_{counter}")
        vals = [float(r["Counter_Value"]) for r in csv.DictReader(open(files[0])) if match in r["Kernel_Name"]]
        if not vals:
            raise SystemExit(f"no dispatch of {match} in {files[0]}")
        return statistics.median(vals), len(vals)
    B, M, N = 4, 1024, 11008
    copy_kib = B * M * N * 2 / 1024                       # the copy arm reads and writes one activation
    cf, ncf = median("copy", "FETCH_SIZE", "copyBuffer")
    cw, _ = median("copy", "WRITE_SIZE", "copyBuffer")
    qf, nq = median("quant", "FETCH_SIZE", "quant_pack_kernel<4")
    qw, _ = median("quant", "WRITE_SIZE", "quant_pack_kernel<4")
    fs, ws = copy_kib / cf, copy_kib / cw
    commit = subprocess.run(["git", "-C", str(ROOT), "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    rec = {"kernel": "hyc::quant_pack_kernel<4,false,false>", "workload": "bf16 [4,1024,11008], q_bit 4",
           "fetch_kib_raw": qf, "write_kib_raw": qw, "copy_fetch_kib_raw": cf, "copy_write_kib_raw": cw,
           "copy_kib_per_direction": copy_kib, "fetch_scale": fs, "write_scale": ws, "dispatches": nq,
           "read_bytes": qf * fs * 1024, "written_bytes": qw * ws * 1024,
           "traffic_bytes": int((qf * fs + qw * ws) * 1024),
           "algorithmic_bytes": int(B * M * N * 2.5 + 2 * N),
           "source_sha256_16": kernel_source_hash(), "commit": commit or "unknown"}
    rec["ratio_to_algorithmic"] = rec["traffic_bytes"] / rec["algorithmic_bytes"]
    TRAFFIC_JSON.write_text(json.dumps(rec, indent=1) + "\n")
    print(json.dumps(rec))


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=1000,
                    help="untimed steps; ~50 ms of work lets the GPU reach its steady clocks (20 steps do not)")
    ap.add_argument("--skip-cpu", action="store_true", help="omit the CPU-oracle timing (for profiler runs)")
    ap.add_argument("--only", choices=["all", "roundtrip", "quant", "fused", "fused4", "mlp", "lora", "kernels", "copy", "layers", "stack"], default="all",
                    help="restrict the run to one part (for profiler runs)")
    ap.add_argument("--pmc-summary", default="", metavar="DIR",
                    help="no GPU work: turn the rocprofv3 counter CSVs under DIR into profiles/quant_pack_q4_config2_hbm_traffic.json")
    ap.add_argument("--fused4-bits", default="2,4,8", help="with --only fused4: the code widths to run")
    ap.add_argument("--layer-case", default="", help="with --only layers: run only the cases whose name contains this")
    ap.add_argument("--layer-seq", type=int, default=0, help="with --only layers: sequence length instead of the configuration's")
    ap.add_argument("--layer-dims", default="", help="with --only layers: override dimensions of the configuration, "
                    "e.g. hidden=5120,heads=40,kv=40,inter=13824")
    ap.add_argument("--layer-arm", choices=["both", "plain", "compressed"], default="both",
                    help="with --only layers: run only one arm (for profiler runs)")
    return ap.parse_args()


def bench_layers(torch, dev, only_case="", arm="both", seq=0, dims_override=None):
    """Forward+backward of one decoder layer with random-init bf16 weights N(0, 0.02) and LoRA r=16 on
    all seven linears: the compressed layer of this package against an uncompressed bf16
    torch-autograd layer of the same architecture, with the activation bytes each keeps for backward."""
    import math
    from types import SimpleNamespace

    import torch.nn.functional as F

    from hyclora_amd.models import llama, llama_flash_attn, mistral
    from hyclora_amd.models.compute_utils import head_to_hidden_shape, hidden_to_head_shape, repeat_kv

    def rope_forward(x, cos, sin):            # differentiable torch rotation for the uncompressed autograd arm
        half, cos, sin = x.shape[-1] // 2, cos.squeeze(), sin.squeeze()
        c, s = cos[None, :x.shape[1], None, :half], sin[None, :x.shape[1], None, :half]
        x1, x2 = x[..., :half], x[..., half:]
        return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)
    BF16 = torch.bfloat16
    gen = torch.Generator(device=dev).manual_seed(1)

    class Lin:
        def __init__(self, w):
            self.weight, self.bias = w, None

    def make(B, S, hidden, heads, kv, inter, theta, rank=16):
        rn = lambda *s, sc: (torch.randn(*s, generator=gen, device=dev) * sc).to(BF16)
        hd = hidden // heads
        dims = dict(q=(hidden, hidden), k=(kv * hd, hidden), v=(kv * hd, hidden), o=(hidden, hidden),
                    gate=(inter, hidden), up=(inter, hidden), down=(hidden, inter))
        P = {}
        for n, (o_f, i_f) in dims.items():
            a = torch.empty(rank, i_f, device=dev)
            torch.nn.init.kaiming_uniform_(a, a=math.sqrt(5), generator=gen)
            P[n] = (Lin(rn(o_f, i_f, sc=0.02)), Lin(a.to(BF16).requires_grad_()), Lin(rn(o_f, rank, sc=1e-3).requires_grad_()))
        x = rn(B, S, hidden, sc=1.0).requires_grad_()
        nw1 = torch.ones(hidden, device=dev, dtype=BF16)
        nw2 = torch.ones(hidden, device=dev, dtype=BF16)
        pos = torch.arange(S, device=dev, dtype=torch.float32)
        inv = 1.0 / (theta ** (torch.arange(0, hd, 2, device=dev, dtype=torch.float32) / hd))
        ang = torch.cat([pos[:, None] * inv[None, :]] * 2, dim=-1)
        return SimpleNamespace(P=P, x=x, nw1=nw1, nw2=nw2, cos=ang.cos().to(BF16)[None], sin=ang.sin().to(BF16)[None],
                               grad=rn(B, S, hidden, sc=1.0), heads=heads, kv=kv, hd=hd, S=S)

    def run_fused(layer, t, mask):
        args = [t.x, t.nw1, None, t.cos, t.sin]
        for n in ("q", "k", "v", "o"):
            args += list(t.P[n])
        args += [t.nw2, None]
        for n in ("gate", "up", "down"):
            args += list(t.P[n])
        return layer(*args, mask, t.heads, t.hd, t.kv)

    def run_plain(t, mask, sdpa):
        def proj(n, inp):
            base, la, lb = t.P[n]
            return inp @ base.weight.t() + (inp @ la.weight.t()) @ lb.weight.t()
        rms = lambda v, w: (v.float() * torch.rsqrt(v.float().pow(2).mean(-1, keepdim=True) + 1e-5)).to(BF16) * w
        xn = rms(t.x, t.nw1)
        q, k, v = (hidden_to_head_shape(proj(n, xn), h) for n, h in (("q", t.heads), ("k", t.kv), ("v", t.kv)))
        q = rope_forward(q.transpose(1, 2), t.cos, t.sin).transpose(1, 2)
        k = rope_forward(k.transpose(1, 2), t.cos, t.sin).transpose(1, 2)
        k, v = repeat_kv(k, t.heads // t.kv), repeat_kv(v, t.heads // t.kv)
        if sdpa:
            o = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        else:
            a = torch.softmax(q @ k.transpose(-2, -1) / math.sqrt(t.hd) + mask, dim=-1, dtype=BF16)
            o = a @ v
        xm = t.x + proj("o", head_to_hidden_shape(o))
        xn2 = rms(xm, t.nw2)
        return xm + proj("down", F.silu(proj("gate", xn2)) * proj("up", xn2))

    def measure(fn, t, steps=5, warmup=2):
        weights = {m.weight.data_ptr() for n in t.P for m in t.P[n]} | {t.nw1.data_ptr(), t.nw2.data_ptr(), t.cos.data_ptr(), t.sin.data_ptr()}
        seen = {}

        def pack(v):
            if v.data_ptr() not in weights:
                seen[(v.data_ptr(), v.numel())] = v.numel() * v.element_size()
            return v
        with torch.autograd.graph.saved_tensors_hooks(pack, lambda v: v):
            y = fn()                                  # what the forward keeps alive for backward
        saved = sum(seen.values())
        adapters = [m.weight for n in t.P for m in t.P[n][1:]]

        def clear():          # as optimizer.zero_grad(set_to_none=True): no gradient-accumulation kernels in the timed steps
            t.x.grad = None
            for p in adapters:
                p.grad = None
        clear()
        y.backward(t.grad)
        result = (y.detach(), t.x.grad.clone(), [p.grad.clone() for p in adapters])
        for _ in range(warmup):
            clear()
            fn().backward(t.grad)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        h0 = time.perf_counter()
        for _ in range(steps):
            clear()
            fn().backward(t.grad)
        e1.record()
        measure.host_ms = (time.perf_counter() - h0) * 1e3 / steps      # the host's share: enqueueing one step
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps, saved, result

    def agreement(got, want, q=8):
        """A wrong but fast layer must not post a number: forward output (never compressed) and the
        input gradient (carries the codes' quantisation error) against the uncompressed autograd arm."""
        (y, gx, ga), (y0, gx0, ga0) = got, want
        rel = ((y.float() - y0.float()).abs().max() / y0.float().abs().max()).item()
        cos = F.cosine_similarity(gx.float().flatten(), gx0.float().flatten(), dim=0).item()
        assert rel <= 2e-2, f"layer output differs from the uncompressed layer: max rel err {rel:.2e}"
        floor = 0.4 if q == 2 else 0.8           # 2-bit codes: a quarter of a channel's range per step
        assert cos >= floor, f"input gradient differs from the uncompressed layer: cosine {cos:.4f} (q_bit {q})"
        # every one of the fourteen adapter gradients as well: a broken one (zero, wrong sign, another projection's)
        # would sit far below these floors however coarse the codes are
        cos_a = [F.cosine_similarity(a.float().flatten(), b.float().flatten(), dim=0).item() for a, b in zip(ga, ga0)]
        assert min(cos_a) >= floor, f"an adapter gradient differs from the uncompressed layer's: cosines {cos_a} (q_bit {q})"
        return {"out_max_rel_err": rel, "grad_x_cos": cos, "min_adapter_grad_cos": min(cos_a)}

    cfg = lambda lt, q: SimpleNamespace(use_hyclora=True, layer_type=lt, iteration_threshold=2,
                                        softmax_outlier_ratio=0.05, layernorm_outlier_ratio=0.005, q_bit=q)
    out = {}
    cases = [("config2_llama7b_b4_s1024_full_fuse", dict(B=4, S=1024, hidden=4096, heads=32, kv=32, inter=11008, theta=1e4),
              llama.make_fused_llama_layer, "intra_inter_full_fuse", [4], False),
             ("config4_mistral7b_b2_s2048_full_fuse", dict(B=2, S=2048, hidden=4096, heads=32, kv=8, inter=14336, theta=1e6),
              mistral.make_fused_mistral_layer, "intra_inter_full_fuse", [2, 4, 8], False),
             ("config5_llama7b_b1_s8192_mapfree_intra_inter", dict(B=1, S=8192, hidden=4096, heads=32, kv=32, inter=11008, theta=1e4),
              None, "intra_inter", [4], True)]
    for name, dims, maker, lt, qbits, sdpa in cases:
        if only_case not in name:
            continue
        if seq:                                       # another sequence length than the configuration's
            dims = dict(dims, S=seq)
            name = f"{name}_at_s{seq}"
        if dims_override:                             # other widths (e.g. hidden=5120,heads=40,kv=40,inter=13824)
            dims = dict(dims, **dims_override)
            name = name + "_with_" + "_".join(f"{k}{v}" for k, v in sorted(dims_override.items()))
        t = make(**dims)
        mask = None if sdpa else torch.full((t.S, t.S), float("-inf"), device=dev).triu(1).to(BF16)[None, None]
        entry, saved_p, plain, res_b = {}, 0, None, None
        if arm != "compressed":
            ms_p, saved_p, plain = measure(lambda: run_plain(t, mask, sdpa), t)
            entry["bf16_uncompressed"] = {"fwd_bwd_ms": ms_p, "host_enqueue_ms": measure.host_ms, "saved_activation_MB": saved_p / 1e6}
            # the reference's own comparison arm: its default layer type, hand-written backward, nothing compressed
            base = llama_flash_attn.FusedLlamaLayerBaseline() if maker is None else maker(cfg("baseline", 0))
            base.set_hyclora_config(cfg("baseline", 0))
            ms_b, saved_b, res_b = measure(lambda: run_fused(base, t, mask), t)
            entry["baseline_layer"] = {"fwd_bwd_ms": ms_b, "host_enqueue_ms": measure.host_ms, "saved_activation_MB": saved_b / 1e6,
                                       "check_against_uncompressed": agreement(res_b, plain)}
            del base
        for q in (qbits if arm != "plain" else []):
            if maker is None:
                layer = llama_flash_attn.FusedLlamaLayerIntraInter()
                layer.set_hyclora_config(cfg(lt, q))
            else:
                layer = maker(cfg(lt, q))
            for _ in range(3):                       # run past calibration so the steady state is timed
                run_fused(layer, t, mask).backward(t.grad)
            ms_f, saved_f, res_f = measure(lambda: run_fused(layer, t, mask), t)
            entry[f"compressed_q{q}"] = {"fwd_bwd_ms": ms_f, "host_enqueue_ms": measure.host_ms, "saved_activation_MB": saved_f / 1e6,
                                         "saved_vs_bf16": saved_p / max(saved_f, 1) if saved_p else None,
                                         "check_against_uncompressed": agreement(res_f, plain, q) if plain else None,
                                         "check_against_baseline_layer": agreement(res_f, res_b, q) if res_b else None}
            del layer, res_f
        out[name] = entry
        del t, mask, plain, res_b
        torch.cuda.empty_cache()
    return out


def bench_stack(torch, dev, n_layers=4, steps=5):
    """The reference's memory / throughput harness (run_memory_throughput.py:178-191: allocated memory
    before the first forward and after the forward of steps 0 and 1; run_memory_throughput.sh: Llama-2-7B,
    batch 4, seq 512, intra_inter, q_bit 2, NF4 frozen weights, LoRA r=16) on a stack of decoder layers
    with random NF4 weights: the compressed layers of this package against an uncompressed bf16
    torch-autograd stack that dequantises the same NF4 weights at every use."""
    import math
    from types import SimpleNamespace

    import torch.nn.functional as F

    from hyclora_amd.models import llama
    from hyclora_amd.models.compute_utils import dense_weight, head_to_hidden_shape, hidden_to_head_shape
    from hyclora_amd.operators import nf4
    BF16 = torch.bfloat16
    gen = torch.Generator(device=dev).manual_seed(2)
    B, S, hidden, heads, inter, rank = 4, 512, 4096, 32, 11008, 16
    hd = hidden // heads
    code2 = torch.cat([-torch.logspace(-7, 0, 127).flip(0), torch.zeros(2), torch.logspace(-7, 0, 127)]).sort().values.to(dev)

    class Lin:
        def __init__(self, w, qs=None):
            self.weight, self.bias = w, None
            if qs is not None:
                self.weight.quant_state = qs

    def nf4_weight(out_f, in_f):
        n = out_f * in_f
        packed = torch.randint(0, 256, (n // 2, 1), generator=gen, device=dev, dtype=torch.uint8)
        nb = n // 64
        state2 = SimpleNamespace(absmax=torch.full((-(-nb // 256),), 0.01, device=dev), code=code2, blocksize=256)
        qs = nf4.make_quant_state(torch.randint(0, 256, (nb,), generator=gen, device=dev, dtype=torch.uint8), (out_f, in_f),
                                  offset=torch.tensor(0.03, device=dev), state2=state2)
        return Lin(packed, qs)

    dims = dict(q=(hidden, hidden), k=(hidden, hidden), v=(hidden, hidden), o=(hidden, hidden),
                gate=(inter, hidden), up=(inter, hidden), down=(hidden, inter))
    layers = []
    for _ in range(n_layers):
        P = {}
        for n, (o_f, i_f) in dims.items():
            a = torch.empty(rank, i_f, device=dev)
            torch.nn.init.kaiming_uniform_(a, a=math.sqrt(5), generator=gen)
            P[n] = (nf4_weight(o_f, i_f), Lin(a.to(BF16).requires_grad_()),
                    Lin((torch.randn(o_f, rank, generator=gen, device=dev) * 1e-3).to(BF16).requires_grad_()))
        layers.append(SimpleNamespace(P=P, nw1=torch.ones(hidden, device=dev, dtype=BF16), nw2=torch.ones(hidden, device=dev, dtype=BF16)))
    pos = torch.arange(S, device=dev, dtype=torch.float32)
    inv = 1.0 / (1e4 ** (torch.arange(0, hd, 2, device=dev, dtype=torch.float32) / hd))
    ang = torch.cat([pos[:, None] * inv[None, :]] * 2, dim=-1)
    cos, sin = ang.cos().to(BF16)[None], ang.sin().to(BF16)[None]
    mask = torch.full((S, S), float("-inf"), device=dev).triu(1).to(BF16)[None, None]
    x0 = (torch.randn(B, S, hidden, generator=gen, device=dev)).to(BF16).requires_grad_()

    def rope(x):
        half = hd // 2
        c, s_ = cos[0][None, :, None, :half], sin[0][None, :, None, :half]
        x1, x2 = x[..., :half], x[..., half:]
        return torch.cat([x1 * c - x2 * s_, x2 * c + x1 * s_], dim=-1)

    class FrozenNF4Matmul(torch.autograd.Function):
        """x @ dequant(W)^T that keeps only the packed weight for backward and dequantises again
        there, like bitsandbytes' 4-bit matmul in an uncompressed QLoRA run."""
        @staticmethod
        def forward(ctx, inp, base):
            ctx.base = base
            return inp @ dense_weight(base.weight, base.weight.quant_state).t()

        @staticmethod
        def backward(ctx, gy):
            return gy @ dense_weight(ctx.base.weight, ctx.base.weight.quant_state), None

    def plain_layer(L, x):
        def proj(n, inp):
            base, la, lb = L.P[n]
            return FrozenNF4Matmul.apply(inp, base) + (inp @ la.weight.t()) @ lb.weight.t()
        rms = lambda v, w: (v.float() * torch.rsqrt(v.float().pow(2).mean(-1, keepdim=True) + 1e-5)).to(BF16) * w
        xn = rms(x, L.nw1)
        q, k, v = (hidden_to_head_shape(proj(n, xn), heads) for n in ("q", "k", "v"))
        q = rope(q.transpose(1, 2)).transpose(1, 2)
        k = rope(k.transpose(1, 2)).transpose(1, 2)
        a = torch.softmax(q @ k.transpose(-2, -1) / math.sqrt(hd) + mask, dim=-1, dtype=BF16)
        xm = x + proj("o", head_to_hidden_shape(a @ v))
        xn2 = rms(xm, L.nw2)
        return xm + proj("down", F.silu(proj("gate", xn2)) * proj("up", xn2))

    cfg = SimpleNamespace(use_hyclora=True, layer_type="intra_inter", iteration_threshold=2, softmax_outlier_ratio=0.05,
                          layernorm_outlier_ratio=0.005, q_bit=2)
    fused = [llama.make_fused_llama_layer(cfg) for _ in layers]

    def fused_layer(i, x):
        L = layers[i]
        args = [x, L.nw1, None, cos, sin]
        for n in ("q", "k", "v", "o"):
            args += list(L.P[n])
        args += [L.nw2, None]
        for n in ("gate", "up", "down"):
            args += list(L.P[n])
        return fused[i](*args, mask, heads, hd, heads)

    def forward(arm):
        x = x0
        for i, L in enumerate(layers):
            x = fused_layer(i, x) if arm == "compressed" else plain_layer(L, x)
        return x.float().pow(2).mean()

    out = {"layers": n_layers, "batch": B, "seq_len": S, "q_bit": 2, "layer_type": "intra_inter", "weights": "NF4, double-quantised statistics"}
    mib = lambda: torch.cuda.memory_allocated() / 2 ** 20
    import gc
    for arm in ("plain", "compressed"):
        gc.collect()
        x0.grad = None
        for L in layers:
            for n in L.P:
                L.P[n][1].weight.grad = L.P[n][2].weight.grad = None
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
        static = mib()
        after = []
        for it in range(3):                                   # steps 0 and 1 as in the reference, 2 = first frozen step
            loss = forward(arm)
            after.append(mib() - static)
            loss.backward()
            del loss
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        h0 = time.perf_counter()
        for _ in range(steps):
            forward(arm).backward()
        e1.record()
        host_ms = (time.perf_counter() - h0) * 1e3 / steps       # the host's share: enqueueing one step
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        out[arm] = {"static_MiB": static, "allocated_after_forward_minus_static_MiB": after,
                    "fwd_bwd_ms": ms, "host_enqueue_ms": host_ms, "sequences_per_s": B / (ms * 1e-3)}
    out["activation_memory_ratio"] = out["plain"]["allocated_after_forward_minus_static_MiB"][1] / \
        out["compressed"]["allocated_after_forward_minus_static_MiB"][1]
    return out


def main():
    args = parse()
    if args.pmc_summary:
        pmc_summary(args.pmc_summary)
        return
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this path has no cross-GPU work (got --gpus {args.gpus}); "
              "run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    import torch.nn.functional as F

    import hyclora_amd  # noqa: F401
    from hyclora_amd import _lib
    from hyclora_amd.operators import compress_function as cf
    from hyclora_amd.operators import rmsnorm_kernels, silu_kernels, softmax_kernels
    from hyclora_amd.operators._fuse import fuse_backward, fuse_forward

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L = _lib.lib()
    BF16 = torch.bfloat16
    B, M, H, N, R, QB = 4, 1024, 4096, 11008, 16, 4
    T = B * M
    E = T * N
    K, W = args.steps, args.warmup
    stream = torch.cuda.current_stream(dev).cuda_stream
    gen = torch.Generator(device=dev).manual_seed(0)

    def randn(*shape, scale=1.0):
        return (torch.randn(*shape, generator=gen, device=dev, dtype=torch.float32) * scale).to(BF16)

    def settle(run, min_ms=SETTLE_MS):
        """Runs `run()` (a batch of the arm's own launches) until min_ms of wall time have passed."""
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while min_ms > 0:
            run()
            torch.cuda.synchronize()
            if (time.perf_counter() - t0) * 1e3 >= min_ms:
                break

    def timed(fn, steps, warmup, settle_ms=SETTLE_MS):
        """ms per call: `steps` calls between two events on the launching stream, bracketed
        by synchronisation; the host clock around the same region is returned as well.  Before the
        timed region: `warmup` calls, then the arm's own calls for settle_ms more."""
        for i in range(warmup):
            fn(i)
        settle(lambda: [fn(i) for i in range(max(steps, 1))], settle_ms)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for i in range(steps):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / steps
        return e0.elapsed_time(e1) / steps, wall

    # ---- compress + decompress round trip -------------------------------------------------
    NB = 8                                    # 8 x (90 + 22.5 + 90) MB >> 256 MiB cache
    xs = [randn(B, M, N) for _ in range(NB)]
    scale = cf.get_statistics_only_quant(xs[0], QB, 'per-channel').reshape(-1).contiguous()
    qs = [torch.empty(B, M, N * QB // 8, device=dev, dtype=torch.uint8) for _ in range(NB)]
    xh = [torch.empty(B, M, N, device=dev, dtype=BF16) for _ in range(NB)]
    sp = scale.data_ptr()

    def quant(i, st=None):
        j = i % NB
        rc = L.hyc_quant_pack(xs[j].data_ptr(), sp, None, qs[j].data_ptr(), None, 0, None, 0,
                              B, M, N, M * N, N, N, 0, QB, st or stream)
        assert rc == 0, _lib.error_string(rc)

    def dequant(i, st=None):
        j = i % NB
        rc = L.hyc_unpack_dequant(qs[j].data_ptr(), sp, None, xh[j].data_ptr(), None, 0, None,
                                  B, M, N, M * N, N, N, 0, QB, st or stream)
        assert rc == 0, _lib.error_string(rc)

    def roundtrip(i, st=None):
        quant(i, st)
        dequant(i, st)

    def timed_graph(fn, steps, warmup, lanes=1):
        """The same `steps` calls recorded once into a HIP graph and replayed as one launch: takes
        the per-launch host latency out of a loop whose kernels run ~20 us each.  The library
        allocates nothing and records only kernel nodes, so it can be captured as it is.
        lanes > 1 records step i on stream i % lanes (default-priority streams forked from and
        joined to the capture stream), so the graph holds `lanes` independent chains: steps work on
        different activations, and the start-up and tail of one step's kernels overlap the next's."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            extra = [torch.cuda.Stream() for _ in range(lanes - 1)]
            for st in extra:
                st.wait_stream(side)
            handles = [side.cuda_stream] + [st.cuda_stream for st in extra]
            for i in range(steps):
                fn(i, handles[i % lanes])
            for st in extra:
                side.wait_stream(st)
        for _ in range(max(1, -(-warmup // steps))):
            graph.replay()
        settle(graph.replay)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / steps
        return e0.elapsed_time(e1) / steps, wall

    if args.only == "copy":
        # calibration arm for the profiler's HBM counters: a plain device copy of known size
        ms_c, _ = timed(lambda i: xh[i % NB].copy_(xs[i % NB]), K, W)
        print(json.dumps({"copy_bytes_read": E * 2, "copy_bytes_written": E * 2, "ms": ms_c,
                          "GBps": E * 4 / ms_c / 1e6}))
        return

    bytes_quant = E * (2 + QB / 8) + 2 * N            # read bf16, write codes, read steps
    bytes_round = 2 * bytes_quant
    out = {}
    kernels = {}
    if args.only in ("all", "roundtrip"):
        ms_eager, wall_eager = timed(roundtrip, K, W)
        ms_one, _ = timed_graph(roundtrip, K, W)
        ms_step, wall_step = timed_graph(roundtrip, K, W, lanes=2)
        for j in range(NB):                              # the replayed graph did the work: same bytes as eager
            assert torch.equal(xh[j], cf.decompression_dequantization(
                cf.compression_quantization(xs[j], scale, QB), scale, QB)), "graph replay output differs"
        out["ms_per_step"] = ms_step
        out["value"] = bytes_round / (ms_step * 1e-3) / 1e9
        out["wall_ms_per_step"] = wall_step
        out["launch_mode"] = {"timed": f"{K} steps recorded in one HIP graph as two independent chains (step i on "
                                       "stream i % 2; each step's dequantise still follows its own quantise), replayed once",
                              "graph_one_chain_ms_per_step": ms_one,
                              "graph_one_chain_GBps": bytes_round / (ms_one * 1e-3) / 1e9,
                              "eager_ms_per_step": ms_eager, "eager_wall_ms_per_step": wall_eager,
                              "eager_GBps": bytes_round / (ms_eager * 1e-3) / 1e9}
    if args.only in ("all", "quant", "roundtrip"):
        # the single-kernel loops time at least 400 launches: with fewer, the start-up of the first launch
        # into an empty queue (~10 us) is a visible share of the average
        Kq = max(K, 400)
        ms_q, _ = timed(quant, Kq, W)
        ms_d, _ = timed(dequant, Kq, W)
        traffic, traffic_note = measured_traffic()
        kernels["quant_pack_q4"] = {"ms": ms_q, "GBps": bytes_quant / ms_q / 1e6}
        kernels["unpack_dequant_q4"] = {"ms": ms_d, "GBps": bytes_quant / ms_d / 1e6}
        roofline = {"bound": "hbm", "kernel": "hyc::quant_pack_kernel<4,false,false>",
                    "achieved": bytes_quant / ms_q / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": bytes_quant / ms_q / 1e6 / HBM_PEAK_GBS,
                    "algorithmic_bytes_per_launch": bytes_quant, "launch_ms": ms_q, "launches_timed": Kq,
                    "traffic": traffic, "traffic_source": traffic_note}
    else:
        roofline = None

    # ---- the other kernels of the path, same shape ---------------------------------------------
    def fused_at(Bf, Mf, Nf, qb, with_torch):
        """Fused LoRA-SiLU-Hadamard forward and backward on [Bf, Mf, Nf] at qb bits through the C ABI, checked
        against the wrappers and the unfused composite before timing; HIP-graph replays."""
        NF = 3
        Tf, Ef = Bf * Mf, Bf * Mf * Nf
        sets = []
        for _ in range(NF):
            d = dict(x1=randn(Bf, Mf, Nf), x2=randn(Bf, Mf, Nf), xa1=randn(Bf, Mf, R), xa2=randn(Bf, Mf, R),
                     b1=randn(R, Nf, scale=0.05), b2=randn(R, Nf, scale=0.05), g=randn(Bf, Mf, Nf))
            sets.append(d)
        s1 = cf.get_statistics_only_quant(sets[0]["x1"], qb, 'per-channel')
        s2 = cf.get_statistics_only_quant(sets[0]["x2"], qb, 'per-channel')
        # outputs are allocated once and the C ABI is called directly, so that both kernels can be
        # timed as HIP-graph replays like every other kernel that runs shorter than an eager launch costs
        bt = 0
        for d in sets:
            d["q1"] = torch.empty(Bf, Mf, Nf * qb // 8, device=dev, dtype=torch.uint8)
            d["q2"] = torch.empty_like(d["q1"])
            d["o"] = torch.empty(Bf, Mf, Nf, device=dev, dtype=BF16)
            d["ob"], d["gg"], d["gu"] = torch.empty_like(d["o"]), torch.empty_like(d["o"]), torch.empty_like(d["o"])
        s1v, s2v = s1.reshape(-1).contiguous(), s2.reshape(-1).contiguous()

        def f_fwd(i, st=None):
            d = sets[i % NF]
            rc = L.hyc_lora_silu_mul_fwd(d["xa1"].data_ptr(), d["b1"].data_ptr(), d["x1"].data_ptr(), s1v.data_ptr(),
                                         d["xa2"].data_ptr(), d["b2"].data_ptr(), d["x2"].data_ptr(), s2v.data_ptr(),
                                         d["q1"].data_ptr(), d["q2"].data_ptr(), d["o"].data_ptr(), Tf, Nf, R, qb, bt, st or stream)
            assert rc == 0, _lib.error_string(rc)

        def f_bwd(i, st=None):
            d = sets[i % NF]
            rc = L.hyc_lora_silu_mul_bwd(d["xa1"].data_ptr(), d["b1"].data_ptr(), d["q1"].data_ptr(), s1v.data_ptr(),
                                         d["xa2"].data_ptr(), d["b2"].data_ptr(), d["q2"].data_ptr(), s2v.data_ptr(),
                                         d["g"].data_ptr(), d["ob"].data_ptr(), d["gg"].data_ptr(), d["gu"].data_ptr(),
                                         Tf, Nf, R, qb, bt, st or stream)
            assert rc == 0, _lib.error_string(rc)

        Kf, Wf = 30, 3
        f_fwd(0)
        f_bwd(0)
        # a wrong but fast kernel must not post a number: the timed entry points against the wrappers'
        # results and against the unfused fp32 composite
        d0 = sets[0]
        q1w, q2w, ow = fuse_forward(d0["xa1"], d0["b1"], d0["x1"], s1, d0["xa2"], d0["b2"], d0["x2"], s2, qb)
        assert torch.equal(q1w, d0["q1"]) and torch.equal(q2w, d0["q2"]) and torch.equal(ow, d0["o"])
        assert torch.equal(q1w, cf.compression_quantization(d0["x1"], s1, qb)), "fused codes differ from the quantiser's"
        obw, ggw, guw = fuse_backward(d0["xa1"], d0["b1"], q1w, s1, d0["xa2"], d0["b2"], q2w, s2, d0["g"], qb)
        assert torch.equal(obw, d0["ob"]) and torch.equal(ggw, d0["gg"]) and torch.equal(guw, d0["gu"])
        ref = F.silu(d0["x1"].float() + d0["xa1"].float() @ d0["b1"].float()) * (d0["x2"].float() + d0["xa2"].float() @ d0["b2"].float())
        err = ((ow.float() - ref).abs().max() / ref.abs().max()).item()
        assert err <= 1e-2, f"fused forward differs from the unfused composite: {err:.2e}"
        del ref, q1w, q2w, ow, obw, ggw, guw
        ms_ff, _ = timed_graph(f_fwd, Kf, Wf)
        ms_fb, _ = timed_graph(f_bwd, Kf, Wf)
        bytes_ff = Ef * (6 + qb / 4) + 2 * Tf * R * 2 + 2 * R * Nf * 2 + 4 * Nf
        bytes_fb = Ef * (8 + qb / 4) + 2 * Tf * R * 2 + 2 * R * Nf * 2 + 4 * Nf
        res = {"fwd_ms": ms_ff, "bwd_ms": ms_fb, "fwd_bwd_ms": ms_ff + ms_fb,
               "timing": f"{Kf} launches over {NF} rotating operand sets recorded in one HIP graph, replayed once, "
                         f"after {SETTLE_MS:.0f} ms of the same replays",
               "fwd_GBps": bytes_ff / ms_ff / 1e6, "bwd_GBps": bytes_fb / ms_fb / 1e6,
               "fwd_frac_of_hbm_peak": bytes_ff / ms_ff / 1e6 / HBM_PEAK_GBS,
               "bwd_frac_of_hbm_peak": bytes_fb / ms_fb / 1e6 / HBM_PEAK_GBS}
        # what the memory system gives a kernel that only loads and stores the same bf16 tensors with the same
        # access shape (a wave = 128 columns x 4 rows per instruction, 16-row tiles) and no arithmetic: forward-like
        # = read two tensors, write one (the codes, q/8 bytes an element each, are on top of that in the real
        # kernel); backward-like = read one, write three
        import ctypes
        ptrs = lambda ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])

        def probe(n_reads, n_writes, rows):
            def f(i, st=None):
                d = sets[i % NF]
                rd = ptrs([d["x1"], d["x2"]][:n_reads]) if n_reads == 2 else ptrs([d["g"]])
                wr = ptrs([d["ob"], d["gg"], d["gu"]][:n_writes])
                rc = L.hyc_stream_probe(rd, n_reads, wr, n_writes, Tf, Nf, 0, rows, st or stream)
                assert rc == 0, _lib.error_string(rc)
            f(0)
            ms = timed_graph(f, Kf, Wf)[0]
            nb = (n_reads + n_writes) * Ef * 2
            return {"ms": ms, "GBps": nb / ms / 1e6, "frac_of_hbm_peak": nb / ms / 1e6 / HBM_PEAK_GBS, "rows_per_wave": rows}
        res["memory_only_probe"] = {"read2_write1": probe(2, 1, 32), "read1_write3": probe(1, 3, 16),
                                    "note": "hyc_stream_probe: loads and stores only, the fused kernels' access shape"}
        # the probe overwrote the backward's outputs of set 0..2; nothing reads them afterwards
        if not with_torch:
            return res
        res["eager_fwd_ms"], _ = timed(f_fwd, Kf, Wf)
        res["eager_bwd_ms"], _ = timed(f_bwd, Kf, Wf)

        # unfused bf16 torch on the same GPU: LoRA add, SiLU, product and their autograd backward
        def t_fwdbwd(i):
            d = sets[i % NF]
            x1 = d["x1"].detach().requires_grad_()
            x2 = d["x2"].detach().requires_grad_()
            y1 = x1 + d["xa1"] @ d["b1"]
            y2 = x2 + d["xa2"] @ d["b2"]
            o = F.silu(y1) * y2
            o.backward(d["g"])

        def t_fwd(i):
            d = sets[i % NF]
            with torch.no_grad():
                y1 = d["x1"] + d["xa1"] @ d["b1"]
                y2 = d["x2"] + d["xa2"] @ d["b2"]
                F.silu(y1) * y2

        ms_tf, _ = timed(t_fwd, Kf, Wf)
        ms_tfb, _ = timed(t_fwdbwd, Kf, Wf)
        res.update({"torch_unfused_fwd_ms": ms_tf, "torch_unfused_fwd_bwd_ms": ms_tfb,
                    "speedup_vs_torch_unfused": ms_tfb / (ms_ff + ms_fb),
                    "note": "the fused kernels also produce/consume the 4-bit saved activations; the torch arm keeps bf16"})
        return res

    fused = fused_at(B, M, N, QB, True) if args.only in ("all", "fused") else None
    # configuration 4's MLP width and its sweep of code widths: [2, 2048, 14336] at 2, 4 and 8 bits
    fused_config4 = None
    if args.only in ("all", "fused4"):
        widths = [int(w) for w in args.fused4_bits.split(",")]
        fused_config4 = {"shape": [2, 2048, 14336], "rank": R}
        for qb in widths:
            fused_config4[f"q{qb}"] = fused_at(2, 2048, 14336, qb, False)

    # ---- the whole MLP block of the layer: x_norm_2 -> gate/up -> LoRA-SiLU-product -> down, forward
    # and backward with the frozen GEMMs, new kernels against unfused bf16 torch autograd --------------
    mlp = None
    if args.only in ("all", "mlp"):
        import math

        from hyclora_amd.models.compute_utils import lora_backward, lora_forward
        from hyclora_amd.operators import lora_kernels
        from hyclora_amd.operators.triton_fuse_lora_silu_hadamard_backward_kernels import triton_fuse_silu_backward
        from hyclora_amd.operators.triton_fuse_lora_silu_hadamard_forward_kernels import triton_fuse_silu_forward

        def adapter(out_f, in_f):
            a = torch.empty(R, in_f, device=dev)
            torch.nn.init.kaiming_uniform_(a, a=math.sqrt(5), generator=gen)      # as PEFT initialises lora_A
            return a.to(BF16).requires_grad_(), randn(out_f, R, scale=1e-3).requires_grad_()
        Wm = {"gate": randn(N, H, scale=0.02), "up": randn(N, H, scale=0.02), "down": randn(H, N, scale=0.02)}
        Ad = {"gate": adapter(N, H), "up": adapter(N, H), "down": adapter(H, N)}
        NX = 4
        x_in = [rmsnorm_kernels.rmsnorm_forward(randn(B, M, H), torch.ones(H, device=dev, dtype=BF16), 1e-5)[0] for _ in range(NX)]
        g_out = [randn(B, M, H) for _ in range(NX)]
        with torch.no_grad():
            s_x = cf.get_statistics_only_quant(x_in[0], QB, 'per-channel')
            s_gate = cf.get_statistics_only_quant(x_in[0] @ Wm["gate"].t(), QB, 'per-channel')
            s_up = cf.get_statistics_only_quant(x_in[0] @ Wm["up"].t(), QB, 'per-channel')
        lora_t = {n: (Ad[n][0].detach().t(), Ad[n][1].detach().t()) for n in Ad}       # [in, R], [R, out] views

        def new_fwd(x):
            """What the full_fuse layer does between its second norm and its output
            (models/llama/fused_llama_layer_intra_inter_full_fuse.py:218-251), statistics frozen."""
            gate_main, up_main = x @ Wm["gate"].t(), x @ Wm["up"].t()
            gate_xa, up_xa = x @ lora_t["gate"][0], x @ lora_t["up"][0]
            q1, q2, had = triton_fuse_silu_forward(gate_xa, lora_t["gate"][1], gate_main, s_gate,
                                                   up_xa, lora_t["up"][1], up_main, s_up, QB)
            xq = cf.compression_quantization(x, s_x, QB)                  # the block's input is kept as codes
            out, _, down_xa = lora_forward(Wm["down"], None, *lora_t["down"], None, had)
            return out, (q1, q2, gate_xa, up_xa, xq, down_xa)

        def new_bwd(saved, g):
            """(…full_fuse.py:359-383): gradients of the block's input and of the six adapter matrices."""
            q1, q2, gate_xa, up_xa, xq, down_xa = saved
            a_d, b_d = lora_t["down"]
            gb_down, g_mid = lora_kernels.lora_products(g, u=down_xa, v=b_d)
            g_down = lora_kernels.lora_add(g @ Wm["down"], g_mid, a_d.mT, inplace=True)
            had, g_gate, g_up = triton_fuse_silu_backward(gate_xa, lora_t["gate"][1], q1, s_gate,
                                                          up_xa, lora_t["up"][1], q2, s_up, g_down, QB)
            ga_down = lora_kernels.lora_products(had, u=g_mid)[0].t()
            codes = (xq, s_x, None, QB)
            ga_g, gb_g, gx = lora_backward(Wm["gate"], None, *lora_t["gate"], None, gate_xa, g_gate, x_codes=codes)
            ga_u, gb_u, gx = lora_backward(Wm["up"], None, *lora_t["up"], None, up_xa, g_up, x_codes=codes, accumulate=gx)
            return gx, (ga_g, gb_g, ga_u, gb_u, ga_down, gb_down)

        def new_step(i):
            with torch.no_grad():
                out, saved = new_fwd(x_in[i % NX])
                return out, new_bwd(saved, g_out[i % NX])

        def torch_step(i, want=False):
            x = x_in[i % NX].detach().requires_grad_()

            def proj(n, inp):
                return inp @ Wm[n].t() + (inp @ Ad[n][0].t()) @ Ad[n][1].t()
            out = proj("down", F.silu(proj("gate", x)) * proj("up", x))
            out.backward(g_out[i % NX])
            res = (out.detach(), x.grad, [Ad[n][j].grad.clone() for n in ("gate", "up", "down") for j in (0, 1)]) if want else None
            for n in Ad:
                Ad[n][0].grad = Ad[n][1].grad = None
            return res

        # the two arms must agree before either is timed (the new arm keeps 4-bit activations: its
        # gradients carry their quantisation error, its forward output does not)
        out_n, (gx_n, gl_n) = new_step(0)
        out_t, gx_t, gl_t = torch_step(0, want=True)
        cosine = lambda a, b: F.cosine_similarity(a.float().flatten(), b.float().flatten(), dim=0).item()
        chk = {"out_max_rel_err": ((out_n.float() - out_t.float()).abs().max() / out_t.float().abs().max()).item(),
               "out_cos": cosine(out_n, out_t), "grad_x_cos": cosine(gx_n, gx_t),
               "adapter_grad_cos_min": min(cosine(a, b)
                                           for a, b in zip((g.t() for g in gl_n), gl_t))}
        assert chk["out_max_rel_err"] <= 2e-2 and chk["out_cos"] >= 0.9999, f"MLP forward differs from torch: {chk}"
        assert chk["grad_x_cos"] >= 0.95 and chk["adapter_grad_cos_min"] >= 0.9, f"MLP gradients differ from torch: {chk}"
        del out_n, gx_n, gl_n, out_t, gx_t, gl_t
        Km = 10
        ms_new, _ = timed(new_step, Km, 2)
        ms_new_f, _ = timed(lambda i: new_fwd(x_in[i % NX]), Km, 2)
        ms_t, _ = timed(torch_step, Km, 2)
        gemm_flop = 2 * T * H * N * 3 * 2                       # three frozen GEMMs forward, three for grad_x
        mlp = {"mlp_fwd_bwd_ms": ms_new, "mlp_fwd_ms": ms_new_f, "torch_mlp_fwd_bwd_ms": ms_t,
               "speedup_vs_torch_unfused": ms_t / ms_new,
               "frozen_gemm_TFLOP": gemm_flop / 1e12, "frozen_gemm_floor_ms_at_2.5_PFLOPs": gemm_flop / 2.5e15 * 1e3,
               "check_against_torch": chk,
               "note": "both arms run the same six hipBLASLt GEMMs on the frozen weights; the new arm keeps gate/up/x as "
                       "4-bit codes (saved activations 4x smaller), the torch arm keeps bf16 tensors for autograd"}
        del Wm, Ad, x_in, g_out

    lora = None
    if args.only in ("all", "lora"):
        # The LoRA kernels around a projection's frozen part, at the two widths of the layer (hidden
        # 4096, intermediate 11008), beside the torch / library calls they replace.  All arms are
        # timed as HIP-graph replays (the kernels run 5-40 us, less than an eager launch costs).
        lora = {}
        Kl = 40
        for wname, Nw in (("n4096", H), ("n11008", N)):
            NBl = -(-600_000_000 // (T * Nw * 2))        # the rotating inputs alone exceed the 256 MiB last-level cache
            x_l = [randn(B, M, Nw) for _ in range(NBl)]
            y_l = [torch.empty(B, M, Nw, device=dev, dtype=BF16) for _ in range(NBl)]
            q_l = [torch.empty(B, M, Nw * QB // 8, device=dev, dtype=torch.uint8) for _ in range(NBl)]
            xa = randn(B, M, R)
            w_b = randn(Nw, R, scale=0.05)                     # lora_B.weight as nn.Linear keeps it: [N, R]
            b_view = w_b.t()                                   # the [R, N] view the layers pass around
            s_l = cf.get_statistics_only_quant(x_l[0], QB, 'per-channel').reshape(-1).contiguous()
            ws_bytes = L.hyc_lora_contract_workspace(T, Nw, R, 1, 1)
            # one set of outputs and workspace per chain of the two-chain timing below
            p1s = [torch.empty(R, Nw, device=dev, dtype=BF16) for _ in range(2)]
            p2s = [torch.empty(B * M, R, device=dev, dtype=BF16) for _ in range(2)]
            wss = [torch.empty(ws_bytes, device=dev, dtype=torch.uint8) for _ in range(2)]
            El = T * Nw

            def c_add(i, st):
                j = i % NBl
                assert L.hyc_lora_add(xa.data_ptr(), w_b.data_ptr(), 1, x_l[j].data_ptr(), None, y_l[j].data_ptr(), T, Nw, R, st) == 0

            def c_add_quant(i, st):
                j = i % NBl
                assert L.hyc_lora_add_quant(xa.data_ptr(), w_b.data_ptr(), 1, x_l[j].data_ptr(), s_l.data_ptr(), None,
                                            q_l[j].data_ptr(), y_l[j].data_ptr(), T, Nw, R, QB, st) == 0

            def c_add_restore(i, st):
                j = i % NBl
                assert L.hyc_lora_add_restore(xa.data_ptr(), w_b.data_ptr(), 1, q_l[j].data_ptr(), s_l.data_ptr(), None,
                                              y_l[j].data_ptr(), T, Nw, R, QB, st) == 0

            def c_both(i, st):
                j = i % NBl
                assert L.hyc_lora_contract(x_l[j].data_ptr(), None, None, None, 0, xa.data_ptr(), w_b.data_ptr(), 1,
                                           p1s[i % 2].data_ptr(), 0, p2s[i % 2].data_ptr(), wss[i % 2].data_ptr(), ws_bytes,
                                           T, Nw, R, st) == 0

            def c_codes(i, st):
                j = i % NBl
                assert L.hyc_lora_contract(None, q_l[j].data_ptr(), s_l.data_ptr(), None, QB, xa.data_ptr(), None, 0,
                                           p1s[i % 2].data_ptr(), 0, None, wss[i % 2].data_ptr(), ws_bytes, T, Nw, R, st) == 0

            # the input gradients of projections that share their input, added up: three LoRA adds chained through
            # a running sum against the one-pass sum of the same three terms
            xa3 = [randn(B, M, R) for _ in range(3)]
            wb3 = [randn(Nw, R, scale=0.05) for _ in range(3)]

            def c_sum_chain(i, st):
                j = i % NBl
                assert L.hyc_lora_add(xa3[0].data_ptr(), wb3[0].data_ptr(), 1, x_l[j].data_ptr(), None, y_l[j].data_ptr(), T, Nw, R, st) == 0
                for c in (1, 2):
                    assert L.hyc_lora_add(xa3[c].data_ptr(), wb3[c].data_ptr(), 1, x_l[(j + c) % NBl].data_ptr(), y_l[j].data_ptr(),
                                          y_l[j].data_ptr(), T, Nw, R, st) == 0

            def c_sum(i, st):
                j = i % NBl
                arr = (_lib.LoraSumMember * 3)(*[_lib.LoraSumMember(xa3[c].data_ptr(), wb3[c].data_ptr(), 1, x_l[(j + c) % NBl].data_ptr())
                                                 for c in range(3)])
                assert L.hyc_lora_add_sum(arr, 3, y_l[j].data_ptr(), T, Nw, R, st) == 0

            def on(st, fn):
                with torch.cuda.stream(torch.cuda.ExternalStream(st)):
                    fn()

            def t_add(i, st):
                on(st, lambda: torch.add(x_l[i % NBl], xa @ b_view, out=y_l[i % NBl]))

            def t_quant(i, st):
                on(st, lambda: cf.compression_quantization(x_l[i % NBl], s_l, QB))

            def t_dequant(i, st):
                on(st, lambda: cf.decompression_dequantization(q_l[i % NBl], s_l, QB))

            def t_both(i, st):
                on(st, lambda: (x_l[i % NBl] @ b_view.mT, (xa.mT @ x_l[i % NBl]).sum(0)))

            def t_xt(i, st):
                on(st, lambda: (x_l[i % NBl].mT @ xa).sum(0))

            e = {}
            for key, fn, nbytes in (("lora_add", c_add, 4 * El), ("lora_add_quant", c_add_quant, (4 + QB / 8) * El),
                                    ("lora_add_restore", c_add_restore, (2 + QB / 8) * El),
                                    ("contract_both_products", c_both, 2 * El), ("contract_from_codes", c_codes, QB / 8 * El)):
                fn(0, stream)                                   # once eagerly: nothing may initialise during capture
                torch.cuda.synchronize()
                ms, _ = timed_graph(fn, Kl, 200)
                # the same calls as two independent chains (call i on stream i % 2), as the headline figure is
                # taken: the drain of one kernel and the ramp of the next overlap, which leaves the kernels' own
                # rate; "ms" is what a chain of dependent calls pays per call
                ms2, _ = timed_graph(fn, Kl, 200, lanes=2)
                e[key] = {"ms": ms, "GBps": nbytes / ms / 1e6, "ms_two_chains": ms2, "GBps_two_chains": nbytes / ms2 / 1e6}
            for key, fn in (("torch_add_after_lora_gemm", t_add), ("quantiser_alone", t_quant), ("dequantiser_alone", t_dequant),
                            ("torch_both_products", t_both), ("torch_xT_grad_medium", t_xt)):
                fn(0, stream)
                torch.cuda.synchronize()
                e[key] = {"ms": timed_graph(fn, Kl, 200)[0]}
            c_sum_chain(0, stream)
            want3 = y_l[0].clone()
            c_sum(0, stream)
            assert torch.equal(y_l[0], want3), "one-pass sum of three LoRA adds differs from the chain"
            ms_c, ms_1 = timed_graph(c_sum_chain, Kl, 200)[0], timed_graph(c_sum, Kl, 200)[0]
            e["sum_of_three_lora_adds"] = {"ms": ms_1, "GBps": 8 * El / ms_1 / 1e6, "chain_of_three_calls_ms": ms_c}
            lora[wname] = e
            del x_l, y_l, q_l, wss

    if args.only in ("all", "kernels"):
        Kx, Wx = max(K // 4, 10), max(W // 4, 3)
        Kg = 40

        def tg(fn):
            """ms per call of a wrapper that allocates and launches but never synchronises: Kg calls recorded
            into one HIP graph (outputs come from the graph's private pool), replayed once.  These kernels
            run 5-25 us, less than an eager call through the Python wrapper costs on the host."""
            fn(0)
            torch.cuda.synchronize()
            return timed_graph(lambda i, st: fn(i), Kg, 3)[0]

        def tg_pair(fn, nbytes):
            """The entry of a [T, 4096] kernel: per call in one chain of dependent calls ("ms"), and as two
            independent chains (call i on stream i % 2), where one call's drain overlaps the next one's ramp
            and the kernel's own rate remains."""
            ms = tg(fn)

            def on_lane(i, st):
                with torch.cuda.stream(torch.cuda.ExternalStream(st)):
                    fn(i)
            ms2 = timed_graph(on_lane, Kg, 3, lanes=2)[0]
            return {"ms": ms, "GBps": nbytes / ms / 1e6, "ms_two_chains": ms2, "GBps_two_chains": nbytes / ms2 / 1e6}
        NH = 16                                   # 16 x 33.5 MB: past the 256 MiB last-level cache
        x_h = [randn(B, M, H) for _ in range(NH)]
        w_h = torch.ones(H, device=dev, dtype=BF16)
        ms = tg(lambda i: rmsnorm_kernels.rmsnorm_forward(x_h[i % NH], w_h, 1e-5))
        kernels["rmsnorm_fwd_4096"] = {"ms": ms, "GBps": T * H * 4 / ms / 1e6}
        y, mean, rstd, bs, nw = rmsnorm_kernels.rmsnorm_forward(x_h[0], w_h, 1e-5)
        ms = tg(lambda i: rmsnorm_kernels.rmsnorm_backward(x_h[(i + 1) % NH], x_h[i % NH], w_h, mean, rstd, True, 1e-5, nw, bs))
        kernels["rmsnorm_bwd_4096"] = {"ms": ms, "GBps": T * H * 6 / ms / 1e6}
        ms = tg(lambda i: silu_kernels.silu_backward(xs[i % NB], xs[(i + 1) % NB]))
        kernels["silu_bwd"] = {"ms": ms, "GBps": E * 6 / ms / 1e6}
        idx = torch.randperm(H, device=dev)[:20].contiguous()
        _, sc = cf.get_statistics_channel_base(x_h[0], 0.005, QB, 'per-channel')
        kernels["quant_pack_q4_outlier_4096"] = tg_pair(
            lambda i: cf.outlier_subtraction_fuse_compression_quantization(x_h[i % NH], sc, idx, QB), T * H * 2.5)
        kernels["quant_pack_q4_outlier_4096"]["note"] = "the wrapper's zero fill of x_outlier is part of a call"
        sy = cf.get_statistics_only_quant(y, QB, 'per-channel')
        tbl = rmsnorm_kernels.outlier_table(idx, H)
        e_nc = tg_pair(lambda i: rmsnorm_kernels.rmsnorm_forward_compress(x_h[i % NH], w_h, 1e-5, QB, scale_y=sy, scale_x=sc,
                                                                          outlier_idx=idx, table=tbl), T * H * (4 + 2 * QB / 8))
        ms3 = tg(lambda i: (rmsnorm_kernels.rmsnorm_forward(x_h[i % NH], w_h, 1e-5),
                            cf.outlier_subtraction_fuse_compression_quantization(x_h[i % NH], sc, idx, QB),
                            cf.compression_quantization(x_h[(i + 1) % NH], sy, QB)))
        kernels["rmsnorm_fwd_compress_4096"] = dict(e_nc, three_separate_kernels_ms=ms3)
        # the same pass that also forms x_norm @ lora_A^T for the three adapters fed by the norm (q, k, v),
        # against the fused norm followed by one library GEMM per adapter
        a_w = [randn(R, H, scale=H ** -0.5) for _ in range(3)]
        a_v = [a.t() for a in a_w]
        ms = tg(lambda i: rmsnorm_kernels.rmsnorm_forward_compress(x_h[i % NH], w_h, 1e-5, QB, scale_y=sy, scale_x=sc,
                                                                   outlier_idx=idx, table=tbl, lora_a=a_v))
        ms_lib = tg(lambda i: [x_h[i % NH] @ v for v in a_v])
        kernels["rmsnorm_fwd_compress_lora3_4096"] = {"ms": ms, "GBps": T * H * (4 + 2 * QB / 8) / ms / 1e6,
                                                      "three_library_gemms_ms": ms_lib,
                                                      "norm_then_three_library_gemms_ms": kernels["rmsnorm_fwd_compress_4096"]["ms"] + ms_lib}
        ms = tg(lambda i: cf.get_statistics_channel_base(x_h[i % NH], 0.005, QB, 'per-channel'))
        kernels["calibration_stats_4096"] = {"ms": ms, "what": "get_statistics_channel_base of [4, 1024, 4096] (batch element 0, "
                                                                "20 outlier channels): statistics pass, strip fold and channel choice"}

        # the calibration kernels one by one, through the C ABI on preallocated buffers, at the batch-0 slices of
        # configuration 1 ([512, 4096], 20 outlier channels) and configuration 4 ([2048, 14336], 71)
        def calibration_kernels(Mc, Nc, kc):
            nbuf = max(2, min(160, -(-600_000_000 // (Mc * Nc * 2))))         # rotate past the 256 MiB cache
            xc = [randn(1, Mc, Nc) for _ in range(nbuf)]
            strips = int(L.hyc_channel_stats_strips(Mc, Nc))
            stats_c = torch.empty(strips * 3 + 1, Nc, device=dev, dtype=torch.float32)
            idx_c = torch.empty(kc, device=dev, dtype=torch.int64)
            sc_c = torch.empty(Nc, device=dev, dtype=BF16)

            def k_stats(i, st):
                rc = L.hyc_channel_stats(xc[i % nbuf].data_ptr(), Mc, Nc, Nc, Nc, 0, stats_c.data_ptr(), stats_c.numel() * 4, st)
                assert rc == 0, _lib.error_string(rc)

            def k_select(i, st):
                rc = L.hyc_channel_select(stats_c.data_ptr(), strips, Nc, kc, QB, 1, idx_c.data_ptr(), sc_c.data_ptr(), None, st)
                assert rc == 0, _lib.error_string(rc)

            def k_steps_only(i, st):
                rc = L.hyc_channel_select(stats_c.data_ptr(), strips, Nc, 0, QB, 0, None, sc_c.data_ptr(), None, st)
                assert rc == 0, _lib.error_string(rc)

            k_stats(0, stream)
            k_select(0, stream)
            want_idx, want_s = cf.get_statistics_channel_base(xc[0], kc / Nc + 1e-9, QB, 'per-channel')
            assert torch.equal(idx_c, want_idx) and torch.equal(sc_c, want_s.reshape(-1)), "timed calibration kernels differ from the wrapper"
            assert torch.equal(stats_c[1], xc[0][0].max(dim=0).values.float()), "channel maxima differ from torch.max"
            ms_s = timed_graph(k_stats, Kg, 3)[0]
            k_stats(0, stream)
            ms_k = timed_graph(k_select, Kg, 3)[0]
            k_stats(0, stream)
            ms_0 = timed_graph(k_steps_only, Kg, 3)[0]
            nb = Mc * Nc * 2
            return {"channel_stats": {"ms": ms_s, "bytes": nb, "GBps": nb / ms_s / 1e6, "frac_of_hbm_peak": nb / ms_s / 1e6 / HBM_PEAK_GBS,
                                      "row_strips": strips},
                    "channel_select": {"ms": ms_k, "channels": Nc, "chosen": kc,
                                       "note": "fold of the strips + steps (one thread per channel), then the choice of "
                                               "the outlier channels by a single workgroup: latency, not bandwidth"},
                    "channel_select_no_outliers": {"ms": ms_0, "channels": Nc}}
        kernels["calibration_config1_512x4096"] = calibration_kernels(512, 4096, 20)
        kernels["calibration_config4_2048x14336"] = calibration_kernels(2048, 14336, 71)
        # norm backward straight from the channel-base compressed input, residual gradient added, against
        # restore + backward with the same add
        xo_h, qx_h = cf.outlier_subtraction_fuse_compression_quantization(x_h[0].clone(), sc, idx, QB)
        e_bc = tg_pair(lambda i: rmsnorm_kernels.rmsnorm_backward_from_codes(x_h[i % NH], qx_h, sc, xo_h, idx, QB, w_h, rstd,
                                                                             residual=x_h[(i + 1) % NH], table=tbl),
                       T * H * (6 + QB / 8))
        ms2 = tg(lambda i: rmsnorm_kernels._backward(
            x_h[i % NH], cf.outlier_addition_fuse_decompression_dequantization(qx_h, sc, xo_h, idx, QB), w_h, rstd,
            want_dw=False, residual=x_h[(i + 1) % NH]))
        kernels["rmsnorm_bwd_from_codes_4096"] = dict(e_bc, restore_then_backward_ms=ms2)
        ms = tg(lambda i: silu_kernels.silu_hadamard_backward(xs[i % NB], xs[(i + 1) % NB], xs[(i + 2) % NB]))
        kernels["silu_mul_bwd"] = {"ms": ms, "GBps": E * 10 / ms / 1e6}
        # attention map (configuration 3 shape): compaction, restore, softmax backward
        a = torch.softmax(torch.randn(4, 32, 1024, 1024, generator=gen, device=dev) * 0.707
                          + torch.full((1024, 1024), float("-inf"), device=dev).triu(1), dim=-1).to(BF16)
        g_a = randn(4, 32, 1024, 1024)
        Ea = a.numel()
        thr = cf.get_statistics_softmax(a, 0.05)
        ms, _ = timed(lambda i: cf.get_statistics_softmax(a, 0.05), 5, 2)
        kernels["softmax_threshold_kth"] = {"ms": ms, "GBps": Ea * 2 / ms / 1e6}
        # its two kernels one by one (the histogram is cleared by a fill kernel inside hyc_hist16)
        hist_c = torch.empty(65536, device=dev, dtype=torch.int32)
        thr_c = torch.empty((), device=dev, dtype=torch.float32)
        kth_c = int(Ea * (1 - 0.05))

        def k_hist(i, st):
            rc = L.hyc_hist16(a.data_ptr(), Ea, hist_c.data_ptr(), st)
            assert rc == 0, _lib.error_string(rc)

        def k_hsel(i, st):
            rc = L.hyc_hist_select(hist_c.data_ptr(), kth_c, thr_c.data_ptr(), st)
            assert rc == 0, _lib.error_string(rc)

        k_hist(0, stream)
        k_hsel(0, stream)
        assert thr_c.item() == thr.item() == torch.kthvalue(a.float().flatten(), kth_c).values.item()
        ms_h = timed_graph(k_hist, 10, 2)[0]
        ms_hs = timed_graph(k_hsel, Kg, 3)[0]
        kernels["hist16"] = {"ms": ms_h, "bytes": Ea * 2, "GBps": Ea * 2 / ms_h / 1e6, "frac_of_hbm_peak": Ea * 2 / ms_h / 1e6 / HBM_PEAK_GBS,
                             "shape": [4, 32, 1024, 1024]}
        kernels["hist_select"] = {"ms": ms_hs, "bins": 65536, "note": "single workgroup: latency, not bandwidth"}
        idx_a, val_a, seg_a = cf.compress_attention_map(a, thr)
        nnz = idx_a.numel()
        ms, _ = timed(lambda i: cf.compress_attention_map(a, thr), 5, 2)
        kernels["softmax_compress"] = {"ms": ms, "GBps": (2 * Ea + 10 * nnz) / ms / 1e6, "nnz": nnz,
                                       "note": "includes the host read-back of nnz"}
        cap_a = nnz + nnz // 16 + 64
        ms, _ = timed(lambda i: cf.compress_attention_map(a, thr, seg_a, capacity=cap_a), 10, 2)
        kernels["sparse_write"] = {"ms": ms, "GBps": (2 * Ea + 10 * nnz) / ms / 1e6, "nnz": nnz,
                                   "note": "the write pass alone: segment offsets given, lists sized from a capacity, no read-back"}
        ms, _ = timed(lambda i: cf.restore_attention_map(idx_a, val_a, seg_a, a.shape), 10, 2)
        kernels["softmax_restore"] = {"ms": ms, "GBps": (2 * Ea + 10 * nnz) / ms / 1e6}
        ms, _ = timed(lambda i: softmax_kernels.softmax_backward(a, g_a), 10, 2)
        kernels["softmax_bwd"] = {"ms": ms, "GBps": 6 * Ea / ms / 1e6}
        causal = torch.full((1024, 1024), float("-inf"), device=dev).triu(1).to(BF16)[None, None]
        ms, _ = timed(lambda i: softmax_kernels.softmax_forward(g_a, 0.0884, causal), 10, 2)
        kernels["softmax_fwd_scale_mask"] = {"ms": ms, "GBps": 4 * Ea / ms / 1e6}
        ms, _ = timed(lambda i: softmax_kernels.softmax_forward(g_a, 0.0884, causal, threshold=thr), 10, 2)
        kernels["softmax_fwd_scale_mask_count"] = {"ms": ms, "GBps": 4 * Ea / ms / 1e6}
        ms, _ = timed(lambda i: torch.softmax(g_a / 11.3137 + causal, dim=-1, dtype=BF16), 10, 2)
        kernels["softmax_fwd_scale_mask"]["torch_three_passes_ms"] = ms
        ms, _ = timed(lambda i: softmax_kernels.softmax_backward_from_compressed(idx_a, val_a, seg_a, g_a), 10, 2)
        kernels["softmax_restore_bwd_one_pass"] = {"ms": ms, "GBps": (6 * Ea + 10 * nnz) / ms / 1e6}
        del a, g_a, idx_a, val_a, seg_a

        # the same kernels on configuration 4's map: [2, 32, 2048, 2048], rows of 2048
        S4 = 2048
        g4 = randn(2, 32, S4, S4)
        E4 = g4.numel()
        causal4 = torch.full((S4, S4), float("-inf"), device=dev).triu(1).to(BF16)[None, None]
        a4 = softmax_kernels.softmax_forward(g4, 0.0884, causal4)
        ref4 = torch.softmax(((g4.float() * torch.tensor(0.0884, device=dev)).to(BF16) + causal4).float(), dim=-1)
        assert ((a4.float() - ref4).abs().max() / ref4.max()).item() <= 1e-2, "softmax_forward differs from the torch composite at rows of 2048"
        del ref4
        thr4 = cf.get_statistics_softmax(a4, 0.05)
        a4c, seg4 = softmax_kernels.softmax_forward(g4, 0.0884, causal4, threshold=thr4)
        idx4, val4, seg4b = cf.compress_attention_map(a4, thr4, seg4)
        nnz4 = idx4.numel()
        assert torch.equal(a4c, a4) and torch.equal(seg4b, seg4)
        a_two, o_two = cf.restore_attention_map(idx4, val4, seg4, a4.shape), None
        o_two = softmax_kernels.softmax_backward(a_two, g4)
        a_one, o_one = softmax_kernels.softmax_backward_from_compressed(idx4, val4, seg4, g4)
        assert torch.equal(a_one, a_two) and torch.equal(o_one, o_two), "one-pass restore + backward differs from the two kernels"
        del a_two, o_two, a_one, o_one, a4c
        m4 = {}
        ms, _ = timed(lambda i: softmax_kernels.softmax_forward(g4, 0.0884, causal4), 10, 2)
        m4["softmax_fwd_scale_mask"] = {"ms": ms, "GBps": 4 * E4 / ms / 1e6, "frac_of_hbm_peak": 4 * E4 / ms / 1e6 / HBM_PEAK_GBS}
        ms, _ = timed(lambda i: softmax_kernels.softmax_forward(g4, 0.0884, causal4, threshold=thr4), 10, 2)
        m4["softmax_fwd_scale_mask_count"] = {"ms": ms, "GBps": 4 * E4 / ms / 1e6, "frac_of_hbm_peak": 4 * E4 / ms / 1e6 / HBM_PEAK_GBS}
        cap4 = nnz4 + nnz4 // 16 + 64
        ms, _ = timed(lambda i: cf.compress_attention_map(a4, thr4, seg4, capacity=cap4), 10, 2)
        nb = 2 * E4 + 10 * nnz4
        m4["sparse_write"] = {"ms": ms, "GBps": nb / ms / 1e6, "frac_of_hbm_peak": nb / ms / 1e6 / HBM_PEAK_GBS, "nnz": nnz4,
                              "note": "lists sized from a capacity, no read-back; counts come from the forward kernel"}
        ms, _ = timed(lambda i: softmax_kernels.softmax_backward_from_compressed(idx4, val4, seg4, g4), 10, 2)
        nb = 6 * E4 + 10 * nnz4
        m4["softmax_restore_bwd_one_pass"] = {"ms": ms, "GBps": nb / ms / 1e6, "frac_of_hbm_peak": nb / ms / 1e6 / HBM_PEAK_GBS}
        kernels["attention_map_config4_2x32x2048x2048"] = m4
        del a4, g4, idx4, val4, seg4

    # ---- whole decoder layers (benchmark configurations 2, 4, 5): fwd+bwd ms and saved bytes ----
    layers = None
    want_cpu = args.only == "all" and not args.skip_cpu
    if want_cpu:
        x_cpu, s_cpu = xs[0].cpu(), scale.cpu().reshape(1, -1)
    if args.only in ("all", "layers"):
        for buffers in (xs, qs, xh):
            buffers.clear()
        torch.cuda.empty_cache()
        layer_dims = {k: int(v) for k, v in (kv.split("=") for kv in args.layer_dims.split(",") if kv)}
        layers = bench_layers(torch, dev, args.layer_case, args.layer_arm, args.layer_seq, layer_dims)
    stack = None
    if args.only in ("all", "stack"):
        for buffers in (xs, qs, xh):
            buffers.clear()
        torch.cuda.empty_cache()
        stack = bench_stack(torch, dev)

    # ---- CPU baseline: the oracle on the host cores, same tensor --------------------------------
    cpu = None
    if want_cpu:
        from oracle import hyc_oracle as O
        torch.set_num_threads(os.cpu_count() or 1)
        O.decompress(O.compress(x_cpu[:1, :64], s_cpu, QB), s_cpu, QB)      # warm-up
        t0 = time.perf_counter()
        reps = 0
        while reps < 2 or (time.perf_counter() - t0 < 10.0 and reps < 20):
            p = O.compress(x_cpu, s_cpu, QB)
            O.decompress(p, s_cpu, QB)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        cpu = {"value": bytes_round / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
               "sample": f"{reps} x compress+decompress of the full [4,1024,11008] bf16 tensor, q_bit=4 "
                         f"({dt:.2f} s each) with the torch-CPU oracle"}

    line = {
        "metric": "compress+decompress GB/s (% HBM peak); fused LoRA-SiLU fwd+bwd ms per MLP layer",
        "value": out.get("value"),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": out.get("ms_per_step"),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "BASELINE config 2: Llama-2-7B-shaped MLP activations, bf16 [4,1024,11008], "
                               "LoRA r=16, q_bit=4; step = quantise+pack then unpack+dequantise of one activation",
                   "rotating_buffers": NB},
        "pct_of_hbm_peak": None if out.get("value") is None else 100.0 * out["value"] / HBM_PEAK_GBS,
        "wall_ms_per_step": out.get("wall_ms_per_step"),
        "launch_mode": out.get("launch_mode"),
        "roofline": roofline,
        "cpu_baseline": cpu,
        "fused": fused,
        "fused_config4": fused_config4,
        "mlp": mlp,
        "lora": lora,
        "kernels": kernels,
        "layers": layers,
        "stack": stack,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
