"""GPU parity of the NF4 weight dequantisation against the oracle (bit-exact: one fp32 product and
one rounding per element), and a decoder layer running on NF4 frozen weights."""
from types import SimpleNamespace

import pytest
import torch

from helpers import BF16, same_bits
from oracle import hyc_oracle as O

pytestmark = pytest.mark.gpu


def code_book_256():
    """A signed, sorted 256-entry code book for the block statistics (the real one travels inside the
    checkpoint's quant state; any table exercises the same arithmetic)."""
    mag = torch.logspace(-7, 0, 127)
    return torch.cat([-mag.flip(0), torch.zeros(2), mag]).sort().values.float()


@pytest.fixture(scope="module")
def nf4():
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import nf4
    return nf4


@pytest.mark.parametrize("shape", [(256, 128), (11008, 64), (96, 40), (4096, 4096)])
@pytest.mark.parametrize("nested", [False, True])
def test_dequant_bit_exact(nf4, dev, shape, nested):
    g = torch.Generator().manual_seed(shape[0])
    w = torch.randn(*shape, generator=g) * 0.02
    code2 = code_book_256() if nested else None
    packed, absmax, nest = O.nf4_quantize(w, blocksize=64, code2=code2)
    want = O.nf4_dequant(packed, absmax, shape, blocksize=64, nested=nest)
    state2 = None
    offset = None
    if nested:
        state2 = SimpleNamespace(absmax=nest[1].to(dev), code=nest[0].to(dev), blocksize=nest[2])
        offset = nest[3].to(dev)
    qs = nf4.make_quant_state(absmax.to(dev), shape, blocksize=64, code=O.NF4_TABLE.to(dev), offset=offset, state2=state2)
    got = nf4.dequantize_nf4(packed.reshape(-1, 1).to(dev), qs)          # bitsandbytes stores the weight as [n/2, 1]
    assert got.dtype == BF16 and tuple(got.shape) == shape
    assert same_bits(got, want)
    # without an explicit code book the published table is used
    qs.code = None
    assert same_bits(nf4.dequantize_nf4(packed.to(dev), qs), want)


def test_dequant_rejects_bad_states(nf4, dev):
    packed = torch.zeros(64, dtype=torch.uint8, device=dev)
    ok = nf4.make_quant_state(torch.ones(2, device=dev), (128,), blocksize=64)
    assert nf4.dequantize_nf4(packed, ok).shape == (128,)
    with pytest.raises(ValueError):
        nf4.dequantize_nf4(packed, nf4.make_quant_state(torch.ones(2, device=dev), (100,), blocksize=64))   # size mismatch
    with pytest.raises(ValueError):
        nf4.dequantize_nf4(packed, nf4.make_quant_state(torch.ones(1, device=dev), (128,), blocksize=64))   # too few statistics
    bad = nf4.make_quant_state(torch.ones(2, device=dev), (128,), blocksize=64)
    bad.quant_type = "fp4"
    with pytest.raises(NotImplementedError):
        nf4.dequantize_nf4(packed, bad)


def test_decoder_layer_on_nf4_weights(nf4, dev):
    """Frozen weights handed over as packed NF4 + quant state give the same layer output and gradients
    as the same weights handed over dense."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import llama
    from test_gpu_layers import Lin, config, grads_of, make_layer_inputs, run_fused
    t = make_layer_inputs(dev, seed=71)
    code2 = code_book_256()
    packed_P, dense_P = {}, {}
    for n, (base, la, lb) in t.P.items():
        packed, absmax, nest = O.nf4_quantize(base.weight.float().cpu(), blocksize=64, code2=code2)
        state2 = SimpleNamespace(absmax=nest[1].to(dev), code=nest[0].to(dev), blocksize=nest[2])
        qs = nf4.make_quant_state(absmax.to(dev), tuple(base.weight.shape), offset=nest[3].to(dev), state2=state2)
        wq = packed.reshape(-1, 1).to(dev)
        wq.quant_state = qs
        packed_P[n] = (Lin(wq), la, lb)
        dense_P[n] = (Lin(nf4.dequantize_nf4(wq, qs)), la, lb)
    outs = []
    for P in (dense_P, packed_P):
        t.P = P
        layer = llama.make_fused_llama_layer(config("intra_inter_full_fuse", 4))
        out = run_fused(layer, t)
        outs.append((out.detach().clone(), grads_of(t, out)))
    assert torch.equal(outs[0][0], outs[1][0])
    for a, b in zip(outs[0][1], outs[1][1]):
        assert (a is None and b is None) or torch.equal(a, b)


def test_default_code_book_is_uploaded_once(nf4, dev):
    """Without a code book in the quant state the published table is used from a device tensor made once
    per device: a host tensor copied at every call would stall the stream (a pageable copy waits for it)."""
    table = nf4._default_table(torch.device(dev))
    assert table.is_cuda and table.dtype == torch.float32
    assert torch.equal(table.cpu(), torch.tensor(nf4.NF4_TABLE))
    packed = torch.zeros(64, dtype=torch.uint8, device=dev)
    qs = nf4.make_quant_state(torch.ones(2, device=dev), (128,), blocksize=64)
    before = dict(nf4._DEFAULT_TABLE)
    nf4.dequantize_nf4(packed, qs)
    nf4.dequantize_nf4(packed, qs)
    assert nf4._DEFAULT_TABLE == before and nf4._default_table(packed.device) is table
