"""Pins of the oracle's RMSNorm backward that need no GPU.

The reference's RMSNorm backward (operators/rmsnorm_kernels.py:92-100) is LayerNorm's formula with
mean(x) taken as 0: dx = (w*dy - (x^*c1 + c2)) * rstd with c1 = mean(x^ * w*dy), c2 = mean(w*dy).
The c2 term is NOT part of the derivative of a true RMSNorm, so autograd of RMSNorm cannot pin it.
On rows whose mean is exactly zero, mean(x^2) is the variance, RMSNorm(x) is LayerNorm(x) without
bias, and the reference formula is exactly LayerNorm's backward (operators/layernorm_kernels.py:92-104)
- a library routine with its own autograd.  The rows are built as (v | -v) so that their sum
cancels exactly, and dy is given a non-zero mean so that c2 is large: a dropped, halved or
sign-flipped c2 fails the first assertion, and the second shows that the case can tell."""
import pytest
import torch
import torch.nn.functional as F

from helpers import BF16, assert_close_bf16, rel_err_and_cos
from oracle import hyc_oracle as O

EPS = 1e-5


def zero_mean_case(n, rows, seed):
    """x bf16 [rows, n] with every row (v | -v), dy with mean ~0.5, w around 1."""
    g = torch.Generator().manual_seed(seed)
    v = (torch.randn(rows, n // 2, generator=g) * 2).to(BF16)
    x = torch.cat([v, -v], dim=-1)
    perm = torch.randperm(n, generator=g)           # mix the halves; the row sum stays exactly 0
    x = x[:, perm].contiguous()
    dy = (torch.randn(rows, n, generator=g) + 0.5).to(BF16)
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(BF16)
    assert float(x.double().sum(-1).abs().max()) == 0.0
    return x, dy, w


def layernorm_autograd_dx(x, dy, w):
    xd = x.double().requires_grad_()
    F.layer_norm(xd, (x.shape[-1],), w.double(), None, EPS).backward(dy.double())
    return xd.grad


def rmsnorm_autograd_dx(x, dy, w):
    xd = x.double().requires_grad_()
    (xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + EPS) * w.double()).backward(dy.double())
    return xd.grad


@pytest.mark.parametrize("n,rows", [(512, 7), (4096, 5), (96, 33)])
def test_rmsnorm_bwd_is_layernorm_backward_on_zero_mean_rows(n, rows):
    x, dy, w = zero_mean_case(n, rows, seed=n + rows)
    y, rstd = O.rmsnorm_fwd(x, w, EPS)
    # the forward agrees with the library LayerNorm on these rows (mean = 0, variance = mean square)
    assert_close_bf16(y, F.layer_norm(x.double(), (n,), w.double(), None, EPS), what="rmsnorm_fwd vs layer_norm")
    dx, _ = O.rmsnorm_bwd(dy, x, w, rstd)
    assert_close_bf16(dx, layernorm_autograd_dx(x, dy, w), what="rmsnorm_bwd vs autograd of layer_norm")
    # ... and is NOT the derivative of a true RMSNorm: the two differ by c2 * rstd
    true_rms = rmsnorm_autograd_dx(x, dy, w)
    rel, _ = rel_err_and_cos(dx, true_rms)
    assert rel > 5e-2, "the case does not exercise the mean term"
    c2 = (w.double() * dy.double()).mean(-1, keepdim=True) * rstd.double().reshape(-1, 1)
    assert_close_bf16(dx, true_rms - c2, what="difference to true RMSNorm is c2 * rstd")


def test_rmsnorm_bwd_variants_of_the_mean_term_fail_the_pin():
    """What the pin is for: the same formula with the mean term dropped or its sign flipped is far
    outside the tolerance on the zero-mean case."""
    n, rows = 512, 7
    x, dy, w = zero_mean_case(n, rows, seed=1)
    _, rstd = O.rmsnorm_fwd(x, w, EPS)
    ref = layernorm_autograd_dx(x, dy, w)
    xhat = x.double() * rstd.double().reshape(-1, 1)
    wdy = w.double() * dy.double()
    c1 = (xhat * wdy).mean(-1, keepdim=True)
    c2 = wdy.mean(-1, keepdim=True)
    for sign in (0.0, -1.0):
        wrong = (wdy - (xhat * c1 + sign * c2)) * rstd.double().reshape(-1, 1)
        rel, _ = rel_err_and_cos(wrong, ref)
        assert rel > 5e-2


def test_rmsnorm_bwd_dw_is_the_weight_gradient():
    x, dy, w = zero_mean_case(256, 9, seed=3)
    _, rstd = O.rmsnorm_fwd(x, w, EPS)
    _, dw = O.rmsnorm_bwd(dy, x, w, rstd)
    wd = w.double().requires_grad_()
    F.layer_norm(x.double(), (256,), wd, None, EPS).backward(dy.double())
    assert_close_bf16(dw, wd.grad, what="dw vs autograd of layer_norm")
