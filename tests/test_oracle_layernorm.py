"""Pins the oracle's LayerNorm (operators/layernorm_kernels.py:27-56, :92-104) against torch's own
layer_norm and its autograd, evaluated in float64."""
import torch
import torch.nn.functional as F

from helpers import BF16, rel_err_and_cos
from oracle import hyc_oracle as O


def _case(seed, shape):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(*shape, generator=g) * 2 + 0.5).to(BF16)
    w = (1 + 0.2 * torch.randn(shape[-1], generator=g)).to(BF16)
    b = (0.1 * torch.randn(shape[-1], generator=g)).to(BF16)
    dy = torch.randn(*shape, generator=g).to(BF16)
    return x, w, b, dy


def test_forward_against_library_layer_norm():
    for shape in [(3, 7, 768), (2, 5, 96), (1, 1, 1024)]:
        x, w, b, _ = _case(shape[-1], shape)
        y, mean, rstd = O.layernorm_fwd(x, w, b, 1e-5)
        ref = F.layer_norm(x.double(), (shape[-1],), w.double(), b.double(), 1e-5)
        rel, cos = rel_err_and_cos(y, ref)
        assert rel <= 1e-2 and cos >= 0.9999
        assert torch.allclose(mean.double(), x.double().mean(-1).flatten(), atol=1e-6)
        assert torch.allclose(rstd.double(), 1 / torch.sqrt(x.double().var(-1, unbiased=False) + 1e-5).flatten(), rtol=1e-5)
    # a constant row: variance 0, output = bias
    x = torch.full((1, 2, 64), 3.0).to(BF16)
    w, b = torch.ones(64).to(BF16), torch.full((64,), 0.25).to(BF16)
    y, mean, rstd = O.layernorm_fwd(x, w, b, 1e-5)
    assert torch.equal(y.float(), torch.full((1, 2, 64), 0.25)) and mean.tolist() == [3.0, 3.0]


def test_backward_against_autograd():
    for shape in [(3, 7, 768), (2, 5, 96)]:
        x, w, b, dy = _case(shape[-1] + 1, shape)
        _, mean, rstd = O.layernorm_fwd(x, w, b, 1e-5)
        dx = O.layernorm_bwd(dy, x, w, mean, rstd)
        xd = x.double().requires_grad_()
        F.layer_norm(xd, (shape[-1],), w.double(), b.double(), 1e-5).backward(dy.double())
        rel, cos = rel_err_and_cos(dx, xd.grad)
        assert rel <= 1e-2 and cos >= 0.9999
        # the input gradient of a LayerNorm is orthogonal to the constant vector
        assert dx.float().sum(-1).abs().max() <= 2e-2 * dx.float().abs().sum(-1).max()
