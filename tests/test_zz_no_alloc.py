"""The entry point that allocates nothing (hyc_rmsnorm_bwd_static: RMSNorm backward with the weight
gradient, its partial rows in a file-scope device array of the library) against the entry point it
is a variant of (hyc_rmsnorm_bwd with a caller workspace): dx and dw bit for bit, on two calls in a
row, the second with a smaller input, so that what the first call left in the array must not leak
into the second."""
import ctypes

import pytest
import torch

from helpers import BF16

pytestmark = pytest.mark.gpu


def _case(dev, rows, n, seed, wdtype):
    g = torch.Generator(device=dev).manual_seed(seed)
    x = (torch.randn(rows, n, generator=g, device=dev) * 2).to(BF16)
    dy = torch.randn(rows, n, generator=g, device=dev).to(BF16)
    w = (1 + 0.1 * torch.randn(n, generator=g, device=dev)).to(wdtype)
    rstd = torch.rsqrt(x.float().pow(2).mean(-1) + 1e-5)
    return x, dy, w, rstd


def _with_workspace(L, x, dy, w, rstd):
    rows, n = x.shape
    dx, dw = torch.empty_like(dy), torch.empty_like(w)
    nbytes = L.lib().hyc_rmsnorm_bwd_workspace(rows, n)
    ws = torch.full((nbytes // 4,), float("nan"), device=x.device)
    L.call("hyc_rmsnorm_bwd", dy.data_ptr(), x.data_ptr(), w.data_ptr(), int(w.dtype == torch.float32),
           rstd.data_ptr(), dx.data_ptr(), dw.data_ptr(), ws.data_ptr(), nbytes, rows, n, L.stream_of(x))
    return dx, dw


def _static(L, x, dy, w, rstd):
    rows, n = x.shape
    dx, dw = torch.empty_like(dy), torch.empty_like(w)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    L.call("hyc_rmsnorm_bwd_static", dy.data_ptr(), x.data_ptr(), w.data_ptr(), int(w.dtype == torch.float32),
           rstd.data_ptr(), dx.data_ptr(), dw.data_ptr(), rows, n, L.stream_of(x))
    assert torch.cuda.memory_allocated() == before
    return dx, dw


@pytest.mark.parametrize("wdtype", [BF16, torch.float32])
def test_static_scratch_entry_point_matches_workspace_entry_point(dev, wdtype):
    import hyclora_amd  # noqa: F401
    from hyclora_amd import _lib as L
    from hyclora_amd.operators import rmsnorm_kernels
    assert L.lib().hyc_rmsnorm_bwd_static_max_bytes() == 512 * 8192 * 4
    # first a launch that fills all 512 partial rows at the widest row, then smaller ones
    for rows, n, seed in ((8192 + 37, 8192, 1), (300, 4096, 2), (5, 96, 3), (4096, 4096, 4)):
        x, dy, w, rstd = _case(dev, rows, n, seed, wdtype)
        want_dx, want_dw = _with_workspace(L, x, dy, w, rstd)
        got_dx, got_dw = _static(L, x, dy, w, rstd)
        assert torch.equal(got_dx, want_dx), f"dx differs at {rows} x {n}"
        assert torch.equal(got_dw, want_dw), f"dw differs at {rows} x {n}"
        assert bool(torch.isfinite(got_dw.float()).all())
    # the Python wrapper goes the same way and allocates nothing either
    dx, dw = torch.empty_like(dy), torch.empty_like(w)
    rmsnorm_kernels.rmsnorm_backward_into(dy, x, w, rstd, dx, dw)
    assert torch.equal(dx, want_dx) and torch.equal(dw, want_dw)
    with pytest.raises(ValueError):
        rmsnorm_kernels.rmsnorm_backward_into(dy, x, w, rstd.double(), dx, dw)


def test_static_scratch_entry_point_rejects_oversized_rows(dev):
    import hyclora_amd  # noqa: F401
    from hyclora_amd import _lib as L
    fake = ctypes.c_void_p(0x1000)          # never dereferenced: the size check comes first
    h = L.lib()
    assert h.hyc_rmsnorm_bwd_static(fake, fake, fake, 0, fake, fake, fake, 16, 8200, None) == -7
    assert h.hyc_rmsnorm_bwd_static(fake, fake, fake, 0, fake, fake, fake, 16, 16384, None) == -7
    assert h.hyc_rmsnorm_bwd_static(fake, fake, fake, 0, fake, fake, fake, 16, 100, None) == -3
    assert h.hyc_rmsnorm_bwd_static(fake, fake, fake, 0, fake, fake, None, 16, 64, None) == -1
    assert h.hyc_rmsnorm_bwd_static(None, None, None, 0, None, None, None, 0, 64, None) == 0
    assert "workspace" in L.error_string(-7)
