"""The committed known-answer vectors (tests/golden/kat.json, written by tests/golden/make_golden.py
with scalar numpy / integer arithmetic only) against the CPU oracle and, on the GPU, against the
kernels through the operator API: codes, packed bytes, dequantised values, compacted attention
map - all bit-exact."""
import json
from pathlib import Path

import numpy as np
import pytest
import torch

from helpers import BF16, bits, from_bits
from oracle import hyc_oracle as O

KAT = json.loads((Path(__file__).parent / "golden" / "kat.json").read_text())


def _tensors(case):
    x = from_bits(np.array(case["x_bits"], dtype=np.uint16))[None]                 # [1, rows, N]
    s = from_bits(np.array(case["scale_bits"], dtype=np.uint16))[None]             # [1, N]
    z = None if case["zero_point"] is None else torch.tensor(case["zero_point"], dtype=torch.int8)[None]
    return x, s, z


@pytest.mark.parametrize("i", range(len(KAT["quant"])))
def test_oracle_reproduces_the_quantisation_vectors(i):
    case = KAT["quant"][i]
    q = case["q_bit"]
    x, s, z = _tensors(case)
    assert np.array_equal(O.quant_codes(x, s, q, z)[0].numpy(), np.array(case["codes"], dtype=np.uint8))
    packed = O.compress(x, s, q, z)
    assert np.array_equal(packed[0].numpy(), np.array(case["packed"], dtype=np.uint8))
    assert np.array_equal(bits(O.decompress(packed, s, q, z))[0], np.array(case["dequant_bits"], dtype=np.uint16))


def test_oracle_reproduces_the_compaction_vector():
    c = KAT["compaction"]
    a = from_bits(np.array(c["map_bits"], dtype=np.uint16)).reshape(c["shape"])
    idx, val = O.softmax_compress(a, c["threshold"])
    assert idx.tolist() == c["indices"]
    got, want = bits(val), np.array(c["value_bits"], dtype=np.uint16)
    nan = (want & 0x7fff) > 0x7f80
    assert np.array_equal(got[~nan], want[~nan]) and np.all((got[nan] & 0x7fff) > 0x7f80)


@pytest.mark.gpu
@pytest.mark.parametrize("i", range(len(KAT["quant"])))
def test_kernels_reproduce_the_quantisation_vectors(dev, i):
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import compress_function as cf
    case = KAT["quant"][i]
    q = case["q_bit"]
    x, s, z = _tensors(case)
    d = lambda t: None if t is None else t.to(dev)
    if z is None:
        packed = cf.compression_quantization(d(x), d(s), q)
        back = cf.decompression_dequantization(packed, d(s), q)
    else:
        packed = cf.compression_quantization_with_zero_point(d(x), d(s), d(z), q)
        back = cf.decompression_dequantization_with_zero_point(packed, d(s), d(z), q)
    assert np.array_equal(packed[0].cpu().numpy(), np.array(case["packed"], dtype=np.uint8))
    assert np.array_equal(bits(back)[0], np.array(case["dequant_bits"], dtype=np.uint16))


@pytest.mark.gpu
def test_kernels_reproduce_the_compaction_vector(dev):
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import compress_function as cf
    c = KAT["compaction"]
    a = from_bits(np.array(c["map_bits"], dtype=np.uint16)).reshape(c["shape"]).to(dev)
    sp = cf.compression_softmax(a, c["threshold"])
    assert sp.indices().flatten().tolist() == c["indices"]
    got, want = bits(sp.values()), np.array(c["value_bits"], dtype=np.uint16)
    nan = (want & 0x7fff) > 0x7f80
    assert np.array_equal(got[~nan], want[~nan]) and np.all((got[nan] & 0x7fff) > 0x7f80)
    dense = cf.decompression_softmax(sp).reshape(c["shape"])
    keep = np.zeros(a.numel(), dtype=bool)
    keep[c["indices"]] = True
    assert np.array_equal(bits(dense).reshape(-1)[~keep], np.zeros((~keep).sum(), dtype=np.uint16))


def _stat_input():
    st = KAT["statistics"]
    return st, from_bits(np.array(st["x_bits"], dtype=np.uint16))


def _check_stats(st, q, scale, zp_pair, cb_pair):
    assert np.array_equal(bits(scale).reshape(-1), np.array(st["only_quant"][str(q)], dtype=np.uint16))
    s_zp, z = zp_pair
    want_z = st["zero_point"][str(q)]
    defined = np.array([v is not None for v in want_z])
    assert np.array_equal(bits(s_zp).reshape(-1), np.array(st["only_quant"][str(q)], dtype=np.uint16))
    assert np.array_equal(z.reshape(-1).cpu().numpy()[defined], np.array([v for v in want_z if v is not None], dtype=np.int8))
    idx, s_cb = cb_pair
    want = st["channel_base"][str(q)]
    assert idx.reshape(-1).tolist() == want["outlier_channel_index"]
    assert np.array_equal(bits(s_cb).reshape(-1), np.array(want["scale_bits"], dtype=np.uint16))


@pytest.mark.parametrize("q", [2, 4, 8])
def test_oracle_reproduces_the_statistics_vectors(q):
    st, x = _stat_input()
    _check_stats(st, q, O.scale_only_quant(x, q), O.scale_zero_point(x, q), O.channel_stats(x, st["ratio"], q))


@pytest.mark.gpu
@pytest.mark.parametrize("q", [2, 4, 8])
def test_kernels_reproduce_the_statistics_vectors(dev, q):
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import compress_function as cf
    st, x = _stat_input()
    x = x.to(dev)
    _check_stats(st, q, cf.get_statistics_only_quant(x, q, 'per-channel'),
                 cf.get_statistics_only_quant_zero_point(x, q, 'per-channel'),
                 cf.get_statistics_channel_base(x, st["ratio"], q, 'per-channel'))
