#!/usr/bin/env python3
"""Benchmark of the HyC-LoRA activation-compression hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload: BASELINE configuration 2 — the activations of a Llama-2-7B-shaped MLP layer,
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
# rocprofv3 --pmc FETCH_SIZE (44 136 KiB raw, x1.9995 from the copy-kernel calibration) and
# WRITE_SIZE (22 016 KiB, x1.0): 88 248 KiB read + 22 016 KiB written.
MEASURED_TRAFFIC_BYTES = (88248 + 22016) * 1024


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--skip-cpu", action="store_true", help="omit the CPU-oracle timing (for profiler runs)")
    ap.add_argument("--only", choices=["all", "roundtrip", "quant", "fused", "copy"], default="all",
                    help="restrict the run to one part (for profiler runs)")
    return ap.parse_args()


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

    def quant(i):
        j = i % NB
        rc = L.hyc_quant_pack(xs[j].data_ptr(), sp, None, qs[j].data_ptr(), None, 0, None, 0,
                              B, M, N, M * N, N, N, 0, QB, stream)
        assert rc == 0, _lib.error_string(rc)

    def dequant(i):
        j = i % NB
        rc = L.hyc_unpack_dequant(qs[j].data_ptr(), sp, None, xh[j].data_ptr(), None, 0, None,
                                  B, M, N, M * N, N, N, 0, QB, stream)
        assert rc == 0, _lib.error_string(rc)

    def roundtrip(i):
        quant(i)
        dequant(i)

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
        ms_step, wall_step = timed(roundtrip, K, W)
        out["ms_per_step"] = ms_step
        out["value"] = bytes_round / (ms_step * 1e-3) / 1e9
        out["wall_ms_per_step"] = wall_step
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

    if args.only == "all":
        Kx, Wx = max(K // 4, 10), max(W // 4, 3)
        x_h = [randn(B, M, H) for _ in range(4)]
        w_h = torch.ones(H, device=dev, dtype=BF16)
        ms, _ = timed(lambda i: rmsnorm_kernels.rmsnorm_forward(x_h[i % 4], w_h, 1e-5), Kx, Wx)
        kernels["rmsnorm_fwd_4096"] = {"ms": ms, "GBps": T * H * 4 / ms / 1e6}
        y, mean, rstd, bs, nw = rmsnorm_kernels.rmsnorm_forward(x_h[0], w_h, 1e-5)
        ms, _ = timed(lambda i: rmsnorm_kernels.rmsnorm_backward(x_h[(i + 1) % 4], x_h[i % 4], w_h, mean, rstd, True, 1e-5, nw, bs), Kx, Wx)
        kernels["rmsnorm_bwd_4096"] = {"ms": ms, "GBps": T * H * 6 / ms / 1e6}
        ms, _ = timed(lambda i: silu_kernels.silu_backward(xs[i % NB], xs[(i + 1) % NB]), Kx, Wx)
        kernels["silu_bwd"] = {"ms": ms, "GBps": E * 6 / ms / 1e6}
        idx = torch.randperm(H, device=dev)[:20].contiguous()
        _, sc = cf.get_statistics_channel_base(x_h[0], 0.005, QB, 'per-channel')
        ms, _ = timed(lambda i: cf.outlier_subtraction_fuse_compression_quantization(x_h[i % 4], sc, idx, QB), Kx, Wx)
        kernels["quant_pack_q4_outlier_4096"] = {"ms": ms, "GBps": T * H * 2.5 / ms / 1e6}
        ms, _ = timed(lambda i: cf.get_statistics_channel_base(x_h[i % 4], 0.005, QB, 'per-channel'), Kx, Wx)
        kernels["calibration_stats_4096"] = {"ms": ms}
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
        del a, g_a, idx_a, val_a

    # ---- CPU baseline: the oracle on the host cores, same tensor --------------------------------
    cpu = None
    if args.only == "all" and not args.skip_cpu:
        from oracle import hyc_oracle as O
        x_cpu = xs[0].cpu()
        s_cpu = scale.cpu().reshape(1, -1)
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
        "roofline": roofline,
        "cpu_baseline": cpu,
        "fused": fused,
        "kernels": kernels,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
