"""The torch-side glue of the layers (reference: models/utils/compute_utils.py:7-51) on the GPU:
lora_forward / lora_backward against the reference's expressions evaluated in float64, with and
without the kernels' extra arguments, and the attention products on hidden-layout views."""
import math

import numpy as np
import pytest
import torch

from helpers import BF16, assert_close_bf16, bits
from oracle import hyc_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def CU():
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import compute_utils
    return compute_utils


def lora_case(dev, seed, B=2, M=48, n_in=256, n_out=384, R=16, dtype=BF16):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(n_out, n_in, generator=g) * 0.05).to(dtype).to(dev)
    a_w = torch.empty(R, n_in)
    torch.nn.init.kaiming_uniform_(a_w, a=math.sqrt(5), generator=g)
    a_w = a_w.to(dtype).to(dev)                              # lora_A.weight [R, in]
    b_w = (torch.randn(n_out, R, generator=g) * 0.05).to(dtype).to(dev)     # lora_B.weight [out, R]
    bias = (torch.randn(n_out, generator=g) * 0.1).to(dtype).to(dev)
    x = torch.randn(B, M, n_in, generator=g).to(dtype).to(dev)
    gy = torch.randn(B, M, n_out, generator=g).to(dtype).to(dev)
    return w, a_w, b_w, bias, x, gy


@pytest.mark.parametrize("dtype", [BF16, torch.float32])
@pytest.mark.parametrize("with_bias", [False, True])
def test_lora_forward_and_backward_match_the_reference_expressions(CU, dev, dtype, with_bias):
    w, a_w, b_w, bias, x, gy = lora_case(dev, 1, dtype=dtype)
    bias = bias if with_bias else None
    y, main, xa = CU.lora_forward(w, None, a_w.T, b_w.T, bias, x)
    X, Wd, A, Bm = x.double(), w.double(), a_w.double(), b_w.double()
    main_ref = X @ Wd.T + (bias.double() if with_bias else 0.0)
    assert_close_bf16(main, main_ref, what="frozen part")
    assert_close_bf16(xa, X @ A.T, what="x @ A")
    assert_close_bf16(y, main_ref + (X @ A.T) @ Bm.T, what="projection output")
    ga, gb, gx = CU.lora_backward(w, None, a_w.T, b_w.T, x, xa, gy)
    G = gy.double()
    gm = G @ Bm
    ga_ref = torch.einsum("bmi,bmr->ir", X, gm)
    gb_ref = torch.einsum("bmr,bmo->ro", xa.double(), G)
    # the torch path returns one gradient per batch element (autograd sums them), the kernels the sum
    ga = ga if ga.dim() == 2 else ga.sum(0)
    gb = gb if gb.dim() == 2 else gb.sum(0)
    assert ga.shape == (x.shape[-1], 16) and gb.shape == (16, gy.shape[-1])
    assert_close_bf16(ga, ga_ref, what="grad lora_A")
    assert_close_bf16(gb, gb_ref, what="grad lora_B")
    assert_close_bf16(gx, G @ Wd + gm @ A, what="grad x")


@pytest.mark.parametrize("q_bit", [2, 4, 8])
def test_lora_backward_from_codes_residual_and_accumulate(CU, dev, q_bit):
    from hyclora_amd.operators import compress_function as cf
    w, a_w, b_w, _, x, gy = lora_case(dev, 2 + q_bit)
    s = cf.get_statistics_only_quant(x, q_bit, 'per-channel')
    q = cf.compression_quantization(x, s, q_bit)
    x_hat = cf.decompression_dequantization(q, s, q_bit)
    xa = x @ a_w.T
    acc = torch.randn_like(x)
    ga0, gb0, gx0 = CU.lora_backward(w, None, a_w.T, b_w.T, x_hat, xa, gy)
    ga1, gb1, gx1 = CU.lora_backward(w, None, a_w.T, b_w.T, None, xa, gy, x_codes=(q, s, None, q_bit),
                                     accumulate=acc.clone())
    assert np.array_equal(bits(ga0), bits(ga1)), "codes path == dequantise first"
    assert np.array_equal(bits(gb0), bits(gb1))
    assert np.array_equal(bits(gx1), bits(acc + gx0)), "accumulate == add afterwards"
    res = torch.randn_like(gy)
    y0, _, _ = CU.lora_forward(w, None, a_w.T, b_w.T, None, x)
    y1, _, _ = CU.lora_forward(w, None, a_w.T, b_w.T, None, x, residual=res)
    assert np.array_equal(bits(y1), bits(res + y0))


@pytest.mark.parametrize("B", [2, 17])
@pytest.mark.parametrize("n_rep", [1, 4])
def test_attention_products_on_hidden_layout_views(CU, dev, B, n_rep):
    """heads_matmul == torch.matmul on [B, S, H*D] tensors seen as [B, H, S, D]; with out_hidden the
    result already lies in hidden layout.  B = 17 takes the plain matmul (more batch elements than
    the per-batch loop is used for)."""
    S, H, D = 24, 8, 16
    KV = H // n_rep
    g = torch.Generator().manual_seed(B)
    q = CU.hidden_to_head_shape(torch.randn(B, S, H * D, generator=g).to(BF16).to(dev), H)
    k = CU.repeat_kv(CU.hidden_to_head_shape(torch.randn(B, S, KV * D, generator=g).to(BF16).to(dev), KV), n_rep)
    v = CU.repeat_kv(CU.hidden_to_head_shape(torch.randn(B, S, KV * D, generator=g).to(BF16).to(dev), KV), n_rep)
    s = CU.heads_matmul(q, k.transpose(-2, -1))
    assert s.shape == (B, H, S, S) and s.is_contiguous()
    assert_close_bf16(s, q.double() @ k.double().transpose(-2, -1), what="q k^T")
    a = torch.softmax(s.float(), dim=-1).to(BF16)
    o = CU.heads_matmul(a, v, out_hidden=True)
    assert o.shape == (B, H, S, D) and o.transpose(1, 2).is_contiguous(), "result lies in [B, S, H, D] memory"
    assert_close_bf16(o, a.double() @ v.double(), what="a v")
    hid = CU.head_to_hidden_shape(o)
    assert hid.data_ptr() == o.data_ptr() and hid.shape == (B, S, H * D), "head_to_hidden_shape is then free"
    # grads of k, v summed over the query heads that share them, on the strided view
    gk = CU.heads_matmul(s.transpose(-2, -1), q, out_hidden=True)
    want = (s.double().transpose(-2, -1) @ q.double()).reshape(B, KV, n_rep, S, D).sum(2)
    assert_close_bf16(CU.repeat_kv_backward(gk, n_rep), want, what="repeat_kv_backward on a strided view")
