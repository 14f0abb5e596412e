"""The memory-only probe of the C ABI stores the xor of what it loads (plus the index of the output), for both
access shapes and ragged sizes, and rejects arguments it cannot run."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,rows", [(0, 16), (0, 96), (1, 4), (1, 8)])
@pytest.mark.parametrize("T,N", [(64, 256), (37, 136), (300, 1544)])
def test_stream_probe_copies_what_it_reads(dev, shape, rows, T, N):
    import hyclora_amd  # noqa: F401
    from hyclora_amd import _lib
    L = _lib.lib()
    g = torch.Generator().manual_seed(T + N)
    a = torch.randint(0, 2 ** 31 - 1, (T, N // 2), generator=g, dtype=torch.int32).to(dev)
    b = torch.randint(0, 2 ** 31 - 1, (T, N // 2), generator=g, dtype=torch.int32).to(dev)
    outs = [torch.full_like(a, -1) for _ in range(3)]
    ptrs = lambda ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    st = torch.cuda.current_stream().cuda_stream
    assert L.hyc_stream_probe(ptrs([a, b]), 2, ptrs(outs), 3, T, N, shape, rows, st) == 0
    want = a ^ b
    for k, o in enumerate(outs):
        w = want.clone().view(T, N // 8, 4)
        w[:, :, 0] += sum(range(k + 1))                 # every 16-byte chunk's first word counts the outputs written
        assert torch.equal(o.view(T, N // 8, 4), w), f"output {k}"
    assert L.hyc_stream_probe(ptrs([a]), 1, ptrs(outs), 4, T, N, shape, rows, st) == -8
    assert L.hyc_stream_probe(ptrs([a]), 1, ptrs(outs), 1, T, N, shape, rows + 1, st) == -8
    assert L.hyc_stream_probe(ptrs([a]), 1, ptrs(outs), 1, T, N + 4, shape, rows, st) == -3
    torch.cuda.synchronize()
