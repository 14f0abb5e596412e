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
# HBM bytes per launch of quant_pack_kernel<4,false,false> on the benchmark tensor, measured with
# rocprofv3 --pmc FETCH_SIZE (44 162.3 KiB raw, x1.99948 from the copy-kernel calibration) and
# WRITE_SIZE (22 016 KiB, x1.0): 88 301.6 KiB read + 22 016 KiB written.
MEASURED_TRAFFIC_BYTES = int((44162.3 * 1.99948 + 22016.0) * 1024)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=1000,
                    help="untimed steps; ~50 ms of work lets the GPU reach its steady clocks (20 steps do not)")
    ap.add_argument("--skip-cpu", action="store_true", help="omit the CPU-oracle timing (for profiler runs)")
    ap.add_argument("--only", choices=["all", "roundtrip", "quant", "fused", "lora", "copy", "layers", "stack"], default="all",
                    help="restrict the run to one part (for profiler runs)")
    ap.add_argument("--layer-case", default="", help="with --only layers: run only the cases whose name contains this")
    ap.add_argument("--layer-arm", choices=["both", "plain", "compressed"], default="both",
                    help="with --only layers: run only one arm (for profiler runs)")
    return ap.parse_args()


def bench_layers(torch, dev, only_case="", arm="both"):
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
        y.backward(t.grad)
        for _ in range(warmup):
            fn().backward(t.grad)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn().backward(t.grad)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps, saved

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
        t = make(**dims)
        mask = None if sdpa else torch.full((t.S, t.S), float("-inf"), device=dev).triu(1).to(BF16)[None, None]
        entry, saved_p = {}, 0
        if arm != "compressed":
            ms_p, saved_p = measure(lambda: run_plain(t, mask, sdpa), t)
            entry["bf16_uncompressed"] = {"fwd_bwd_ms": ms_p, "saved_activation_MB": saved_p / 1e6}
            # the reference's own comparison arm: its default layer type, hand-written backward, nothing compressed
            base = llama_flash_attn.FusedLlamaLayerBaseline() if maker is None else maker(cfg("baseline", 0))
            base.set_hyclora_config(cfg("baseline", 0))
            ms_b, saved_b = measure(lambda: run_fused(base, t, mask), t)
            entry["baseline_layer"] = {"fwd_bwd_ms": ms_b, "saved_activation_MB": saved_b / 1e6}
            del base
        for q in (qbits if arm != "plain" else []):
            if maker is None:
                layer = llama_flash_attn.FusedLlamaLayerIntraInter()
                layer.set_hyclora_config(cfg(lt, q))
            else:
                layer = maker(cfg(lt, q))
            for _ in range(3):                       # run past calibration so the steady state is timed
                run_fused(layer, t, mask).backward(t.grad)
            ms_f, saved_f = measure(lambda: run_fused(layer, t, mask), t)
            entry[f"compressed_q{q}"] = {"fwd_bwd_ms": ms_f, "saved_activation_MB": saved_f / 1e6,
                                         "saved_vs_bf16": saved_p / max(saved_f, 1) if saved_p else None}
            del layer
        out[name] = entry
        del t, mask
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
        for _ in range(steps):
            forward(arm).backward()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        out[arm] = {"static_MiB": static, "allocated_after_forward_minus_static_MiB": after,
                    "fwd_bwd_ms": ms, "sequences_per_s": B / (ms * 1e-3)}
    out["activation_memory_ratio"] = out["plain"]["allocated_after_forward_minus_static_MiB"][1] / \
        out["compressed"]["allocated_after_forward_minus_static_MiB"][1]
    return out


def main():
    args = parse()
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

    def timed(fn, steps, warmup):
        """ms per call: `steps` calls between two events on the launching stream, bracketed
        by synchronisation; the host clock around the same region is returned as well."""
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
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
        torch.cuda.synchronize()
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
        ms_q, _ = timed(quant, K, W)
        ms_d, _ = timed(dequant, K, W)
        kernels["quant_pack_q4"] = {"ms": ms_q, "GBps": bytes_quant / ms_q / 1e6}
        kernels["unpack_dequant_q4"] = {"ms": ms_d, "GBps": bytes_quant / ms_d / 1e6}
        roofline = {"bound": "hbm", "kernel": "hyc::quant_pack_kernel<4,false,false>",
                    "achieved": bytes_quant / ms_q / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": bytes_quant / ms_q / 1e6 / HBM_PEAK_GBS,
                    "algorithmic_bytes_per_launch": bytes_quant, "launch_ms": ms_q,
                    "traffic": MEASURED_TRAFFIC_BYTES}
    else:
        roofline = None

    # ---- the other kernels of the path, same shape ---------------------------------------------
    fused = None
    if args.only in ("all", "fused"):
        NF = 3
        sets = []
        for _ in range(NF):
            d = dict(x1=randn(B, M, N), x2=randn(B, M, N), xa1=randn(B, M, R), xa2=randn(B, M, R),
                     b1=randn(R, N, scale=0.05), b2=randn(R, N, scale=0.05), g=randn(B, M, N))
            sets.append(d)
        s1 = cf.get_statistics_only_quant(sets[0]["x1"], QB, 'per-channel')
        s2 = cf.get_statistics_only_quant(sets[0]["x2"], QB, 'per-channel')
        saved = {}

        def f_fwd(i):
            d = sets[i % NF]
            saved[i % NF] = fuse_forward(d["xa1"], d["b1"], d["x1"], s1, d["xa2"], d["b2"], d["x2"], s2, QB)

        def f_bwd(i):
            d = sets[i % NF]
            q1, q2, _ = saved[i % NF]
            fuse_backward(d["xa1"], d["b1"], q1, s1, d["xa2"], d["b2"], q2, s2, d["g"], QB)

        Kf, Wf = max(K // 4, 10), max(W // 4, 3)
        ms_ff, _ = timed(f_fwd, Kf, Wf)
        ms_fb, _ = timed(f_bwd, Kf, Wf)
        bytes_ff = E * (6 + QB / 4) + 2 * T * R * 2 + 2 * R * N * 2 + 4 * N
        bytes_fb = E * (8 + QB / 4) + 2 * T * R * 2 + 2 * R * N * 2 + 4 * N

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
        fused = {"fwd_ms": ms_ff, "bwd_ms": ms_fb, "fwd_bwd_ms": ms_ff + ms_fb,
                 "fwd_GBps": bytes_ff / ms_ff / 1e6, "bwd_GBps": bytes_fb / ms_fb / 1e6,
                 "fwd_frac_of_hbm_peak": bytes_ff / ms_ff / 1e6 / HBM_PEAK_GBS,
                 "bwd_frac_of_hbm_peak": bytes_fb / ms_fb / 1e6 / HBM_PEAK_GBS,
                 "torch_unfused_fwd_ms": ms_tf, "torch_unfused_fwd_bwd_ms": ms_tfb,
                 "speedup_vs_torch_unfused": ms_tfb / (ms_ff + ms_fb),
                 "note": "the fused kernels also produce/consume the 4-bit saved activations; the torch arm keeps bf16"}
        del sets, saved

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
            p1 = torch.empty(R, Nw, device=dev, dtype=BF16)
            p2 = torch.empty(B * M, R, device=dev, dtype=BF16)
            ws_bytes = L.hyc_lora_contract_workspace(T, Nw, R, 1, 1)
            ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
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
                                           p1.data_ptr(), p2.data_ptr(), ws.data_ptr(), ws_bytes, T, Nw, R, st) == 0

            def c_codes(i, st):
                j = i % NBl
                assert L.hyc_lora_contract(None, q_l[j].data_ptr(), s_l.data_ptr(), None, QB, xa.data_ptr(), None, 0,
                                           p1.data_ptr(), None, ws.data_ptr(), ws_bytes, T, Nw, R, st) == 0

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
                e[key] = {"ms": ms, "GBps": nbytes / ms / 1e6}
            for key, fn in (("torch_add_after_lora_gemm", t_add), ("quantiser_alone", t_quant), ("dequantiser_alone", t_dequant),
                            ("torch_both_products", t_both), ("torch_xT_grad_medium", t_xt)):
                fn(0, stream)
                torch.cuda.synchronize()
                e[key] = {"ms": timed_graph(fn, Kl, 200)[0]}
            lora[wname] = e
            del x_l, y_l, q_l, ws

    if args.only == "all":
        Kx, Wx = max(K // 4, 10), max(W // 4, 3)
        NH = 16                                   # 16 x 33.5 MB: past the 256 MiB last-level cache
        x_h = [randn(B, M, H) for _ in range(NH)]
        w_h = torch.ones(H, device=dev, dtype=BF16)
        ms, _ = timed(lambda i: rmsnorm_kernels.rmsnorm_forward(x_h[i % NH], w_h, 1e-5), Kx, Wx)
        kernels["rmsnorm_fwd_4096"] = {"ms": ms, "GBps": T * H * 4 / ms / 1e6}
        y, mean, rstd, bs, nw = rmsnorm_kernels.rmsnorm_forward(x_h[0], w_h, 1e-5)
        ms, _ = timed(lambda i: rmsnorm_kernels.rmsnorm_backward(x_h[(i + 1) % NH], x_h[i % NH], w_h, mean, rstd, True, 1e-5, nw, bs), Kx, Wx)
        kernels["rmsnorm_bwd_4096"] = {"ms": ms, "GBps": T * H * 6 / ms / 1e6}
        ms, _ = timed(lambda i: silu_kernels.silu_backward(xs[i % NB], xs[(i + 1) % NB]), Kx, Wx)
        kernels["silu_bwd"] = {"ms": ms, "GBps": E * 6 / ms / 1e6}
        idx = torch.randperm(H, device=dev)[:20].contiguous()
        _, sc = cf.get_statistics_channel_base(x_h[0], 0.005, QB, 'per-channel')
        ms, _ = timed(lambda i: cf.outlier_subtraction_fuse_compression_quantization(x_h[i % NH], sc, idx, QB), Kx, Wx)
        kernels["quant_pack_q4_outlier_4096"] = {"ms": ms, "GBps": T * H * 2.5 / ms / 1e6}
        sy = cf.get_statistics_only_quant(y, QB, 'per-channel')
        tbl = rmsnorm_kernels.outlier_table(idx, H)
        ms, _ = timed(lambda i: rmsnorm_kernels.rmsnorm_forward_compress(x_h[i % NH], w_h, 1e-5, QB, scale_y=sy, scale_x=sc,
                                                                         outlier_idx=idx, table=tbl), Kx, Wx)
        ms3, _ = timed(lambda i: (rmsnorm_kernels.rmsnorm_forward(x_h[i % NH], w_h, 1e-5),
                                  cf.outlier_subtraction_fuse_compression_quantization(x_h[i % NH], sc, idx, QB),
                                  cf.compression_quantization(x_h[(i + 1) % NH], sy, QB)), Kx, Wx)
        kernels["rmsnorm_fwd_compress_4096"] = {"ms": ms, "GBps": T * H * (4 + 2 * QB / 8) / ms / 1e6,
                                                "three_separate_kernels_ms": ms3}
        ms, _ = timed(lambda i: cf.get_statistics_channel_base(x_h[i % NH], 0.005, QB, 'per-channel'), Kx, Wx)
        kernels["calibration_stats_4096"] = {"ms": ms}
        # norm backward straight from the channel-base compressed input, residual gradient added, against
        # restore + backward with the same add
        xo_h, qx_h = cf.outlier_subtraction_fuse_compression_quantization(x_h[0].clone(), sc, idx, QB)
        ms, _ = timed(lambda i: rmsnorm_kernels.rmsnorm_backward_from_codes(x_h[i % NH], qx_h, sc, xo_h, idx, QB, w_h, rstd,
                                                                            residual=x_h[(i + 1) % NH], table=tbl), Kx, Wx)
        ms2, _ = timed(lambda i: rmsnorm_kernels._backward(
            x_h[i % NH], cf.outlier_addition_fuse_decompression_dequantization(qx_h, sc, xo_h, idx, QB), w_h, rstd,
            want_dw=False, residual=x_h[(i + 1) % NH]), Kx, Wx)
        kernels["rmsnorm_bwd_from_codes_4096"] = {"ms": ms, "GBps": T * H * (6 + QB / 8) / ms / 1e6,
                                                  "restore_then_backward_ms": ms2}
        ms, _ = timed(lambda i: silu_kernels.silu_hadamard_backward(xs[i % NB], xs[(i + 1) % NB], xs[(i + 2) % NB]), Kx, Wx)
        kernels["silu_mul_bwd"] = {"ms": ms, "GBps": E * 10 / ms / 1e6}
        # attention map (configuration 3 shape): compaction, restore, softmax backward
        a = torch.softmax(torch.randn(4, 32, 1024, 1024, generator=gen, device=dev) * 0.707
                          + torch.full((1024, 1024), float("-inf"), device=dev).triu(1), dim=-1).to(BF16)
        g_a = randn(4, 32, 1024, 1024)
        Ea = a.numel()
        thr = cf.get_statistics_softmax(a, 0.05)
        ms, _ = timed(lambda i: cf.get_statistics_softmax(a, 0.05), 5, 2)
        kernels["softmax_threshold_kth"] = {"ms": ms, "GBps": Ea * 2 / ms / 1e6}
        idx_a, val_a, seg_a = cf.compress_attention_map(a, thr)
        nnz = idx_a.numel()
        ms, _ = timed(lambda i: cf.compress_attention_map(a, thr), 5, 2)
        kernels["softmax_compress"] = {"ms": ms, "GBps": (2 * Ea + 10 * nnz) / ms / 1e6, "nnz": nnz,
                                       "note": "includes the host read-back of nnz"}
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
        del a, g_a, idx_a, val_a

    # ---- whole decoder layers (benchmark configurations 2, 4, 5): fwd+bwd ms and saved bytes ----
    layers = None
    want_cpu = args.only == "all" and not args.skip_cpu
    if want_cpu:
        x_cpu, s_cpu = xs[0].cpu(), scale.cpu().reshape(1, -1)
    if args.only in ("all", "layers"):
        for buffers in (xs, qs, xh):
            buffers.clear()
        torch.cuda.empty_cache()
        layers = bench_layers(torch, dev, args.layer_case, args.layer_arm)
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
        "lora": lora,
        "kernels": kernels,
        "layers": layers,
        "stack": stack,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
