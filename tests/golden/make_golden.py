"""Writes tests/golden/kat.json: small known-answer vectors for the packed activation format,
computed here with scalar numpy / integer arithmetic only (no torch, no oracle, no kernels), from
the rules the reference's kernels implement:

  code  = clamp(roundf(fp32(x) / fp32(s) [+ z]), -2^(q-1), 2^(q-1)-1) + 2^(q-1), roundf = half away
          from zero                        (operators/compress_function_kernel.py:92-110, :292)
  pack  : byte[p*w + j] = OR_i code[32p + j + i*w] << (q*i), epp = 8/q, w = 32/epp, i < epp   (:77-85, :96-112)
  value = bf16( (code - 2^(q-1) [- z]) * s )                                    (:193-206, :382-388)
  keep  : entries of the flattened map strictly above the threshold, ascending index
                                                   (operators/compress_function.py:309-313)
  steps, zero points and outlier channels of the calibration statistics (:45-105), see main()

bf16 values are stored as their 16-bit patterns.  Run:  python tests/golden/make_golden.py
The vectors pin both the CPU oracle (tests/test_golden.py, CPU) and the kernels (GPU part of it)."""
import json
import math
from pathlib import Path

import numpy as np


def bf16_bits(x: float) -> int:
    """float -> bf16 bit pattern, round to nearest even."""
    u = int(np.array([x], dtype=np.float32).view(np.uint32)[0])
    if (u & 0x7fffffff) > 0x7f800000:                      # NaN
        return (u >> 16) | 0x40
    u += 0x7fff + ((u >> 16) & 1)
    return (u >> 16) & 0xffff


def bf16_val(bits: int) -> float:
    return float(np.array([bits << 16], dtype=np.uint32).view(np.float32)[0])


def roundf(t: np.float32) -> float:
    a = math.floor(abs(float(t)))
    frac = abs(float(t)) - a
    r = a + 1 if frac >= 0.5 else a
    return math.copysign(r, float(t))


def code(x_bits, s_bits, q, z=0):
    x, s = np.float32(bf16_val(x_bits)), np.float32(bf16_val(s_bits))
    with np.errstate(divide="ignore", invalid="ignore"):
        t = np.float32(x / s)
        if z:
            t = np.float32(t + np.float32(z))
    if math.isnan(float(t)):
        return 0
    half = 1 << (q - 1)
    if math.isinf(float(t)):
        r = -half if t < 0 else half - 1
    else:
        r = min(max(roundf(t), -half), half - 1)
    return int(r) + half


def pack_row(codes, q):
    epp, n = 8 // q, len(codes)
    w = 32 // epp
    out = [0] * (n // epp)
    for p in range(n // 32):
        for j in range(w):
            b = 0
            for i in range(epp):
                b |= codes[32 * p + j + i * w] << (q * i)
            out[p * w + j] = b
    return out


def dequant(c, s_bits, q, z=0):
    half = 1 << (q - 1)
    v = bf16_val(bf16_bits(float(c - half)))                # exact small integer
    if z:
        v = bf16_val(bf16_bits(v - bf16_val(bf16_bits(float(z)))))
    return bf16_bits(float(np.float32(v) * np.float32(bf16_val(s_bits))))


def main():
    rng = np.random.default_rng(20240607)
    cases = []
    for q in (2, 4, 8):
        for zp in (False, True):
            n, rows = 64, 4
            half = 1 << (q - 1)
            # steps: powers of two, non-powers, tiny and large; values: exact multiples, ties at k + 0.5,
            # just below / above ties, beyond the clamp, signed zeros, infinities, NaN
            s_vals = [0.5, 0.75, 1.0, 1.5, 0.0999755859375, 3.0, 0.001953125, 17.0]
            s_bits = [bf16_bits(s_vals[c % len(s_vals)]) for c in range(n)]
            z = [int(rng.integers(-half, half)) if zp else 0 for _ in range(n)]
            x_bits = []
            for r in range(rows):
                row = []
                for c in range(n):
                    s = bf16_val(s_bits[c])
                    k = int(rng.integers(-half - 2, half + 2))
                    kind = (r * n + c) % 7
                    if kind == 0:
                        v = k * s
                    elif kind == 1:
                        v = (k + 0.5) * s
                    elif kind == 2:
                        v = (k + 0.49) * s
                    elif kind == 3:
                        v = (k - 0.5) * s
                    elif kind == 4:
                        v = float(rng.normal()) * s * half
                    elif kind == 5:
                        v = [0.0, -0.0, float("inf"), float("-inf"), float("nan")][(r + c) % 5]
                    else:
                        v = (k + 0.51) * s
                    row.append(bf16_bits(v))
                x_bits.append(row)
            codes = [[code(x_bits[r][c], s_bits[c], q, z[c]) for c in range(n)] for r in range(rows)]
            cases.append({
                "q_bit": q, "zero_point": z if zp else None, "scale_bits": s_bits, "x_bits": x_bits,
                "codes": codes, "packed": [pack_row(codes[r], q) for r in range(rows)],
                "dequant_bits": [[dequant(codes[r][c], s_bits[c], q, z[c]) for c in range(n)] for r in range(rows)],
            })
    # compaction: a 2 x 3 x 8 map, threshold in the middle; NaN is kept (NaN * 0 is not zero), zeros are not
    vals = [0.0, 0.25, 0.5, 0.125, 0.75, 0.5, 0.0, 1.0] * 6
    vals[13], vals[30] = float("nan"), -0.0
    thr = 0.5
    keep = [i for i, v in enumerate(vals) if (v > thr or v != v) and v != 0]
    softmax = {"shape": [2, 3, 8], "map_bits": [bf16_bits(v) for v in vals], "threshold": thr,
               "indices": keep, "value_bits": [bf16_bits(vals[i]) for i in keep]}
    # calibration statistics from batch element 0 (operators/compress_function.py:45-105), bf16 after
    # every tensor operation: d = bf16(max - min), s = bf16(fp32(d) / (2^q - 1)); zero point
    # z = int8(bf16(-rne(bf16(min / s)) - 2^(q-1))); channel base: the k = int(N*ratio) channels of
    # largest bf16 norm (ties: lower channel first) are zeroed first, a zero step becomes bf16(0 + 1e-3)
    nb, rows, n = 2, 6, 64
    xs = rng.normal(size=(nb, rows, n))
    xs[:, :, 9] *= 40.0
    xs[:, :, 33] *= 25.0
    xs[:, :, 50] *= 60.0
    xs[:, :, 20] = 0.5                                       # a constant channel: zero step
    xs[1] *= 3.0                                             # batch element 1 must not matter
    xb = [[[bf16_bits(v) for v in row] for row in bt] for bt in xs]
    x0 = [[bf16_val(b) for b in row] for row in xb[0]]
    bf = lambda v: bf16_val(bf16_bits(v))
    stats = {"x_bits": xb, "ratio": 0.05, "only_quant": {}, "zero_point": {}, "channel_base": {}}
    col = lambda c: [x0[r][c] for r in range(rows)]
    for q in (2, 4, 8):
        levels = float((1 << q) - 1)
        half = float(1 << (q - 1))
        sc, zs = [], []
        for c in range(n):
            lo, hi = min(col(c)), max(col(c))
            d = bf(hi - lo)
            sv = bf(float(np.float32(d) / np.float32(levels)))
            sc.append(bf16_bits(sv))
            if sv != 0.0:
                t = bf(float(np.float32(lo) / np.float32(sv)))
                r = float(np.round(np.float32(t)))            # numpy rounds half to even
                zs.append(int(bf(bf(-r) - half)))
            else:
                zs.append(None)                               # 0 / 0: not defined, not compared
        stats["only_quant"][str(q)] = sc
        stats["zero_point"][str(q)] = zs
        norms = [bf(math.sqrt(float(sum(np.float32(v) * np.float32(v) for v in col(c))))) for c in range(n)]
        k = int(n * 0.05)
        idx = sorted(range(n), key=lambda c: (-norms[c], c))[:k]
        sb = []
        for c in range(n):
            vals = [0.0] * rows if c in idx else col(c)
            sv = bf(float(np.float32(bf(max(vals) - min(vals))) / np.float32(levels)))
            if sv == 0.0:
                sv = bf(float(np.float32(sv) + np.float32(1e-3)))
            sb.append(bf16_bits(sv))
        stats["channel_base"][str(q)] = {"outlier_channel_index": idx, "scale_bits": sb}
    out = {"quant": cases, "compaction": softmax, "statistics": stats}
    path = Path(__file__).with_name("kat.json")
    path.write_text(json.dumps(out, separators=(",", ":")))
    print("wrote", path, path.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
