"""CPU checks of the oracle's LoRA helpers against explicit loops: which operand is transposed,
which index is contracted, and where the bf16 rounding falls."""
import torch

from helpers import BF16, same_bits
from oracle import hyc_oracle as O


def test_lora_add_rounds_the_product_before_the_add():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 5, 32, generator=g).to(BF16)
    xa = torch.randn(2, 5, 4, generator=g).to(BF16)
    b = torch.randn(4, 32, generator=g).to(BF16)
    want = torch.empty_like(x)
    for bi in range(2):
        for t in range(5):
            for n in range(32):
                dot = sum(float(xa[bi, t, r]) * float(b[r, n]) for r in range(4))
                lora = torch.tensor(dot, dtype=torch.float32).to(BF16)               # first rounding
                want[bi, t, n] = (x[bi, t, n].float() + lora.float()).to(BF16)       # second rounding
    assert same_bits(O.lora_add(x, xa, b), want)
    # a case where rounding once instead of twice gives another result: 1 + (2^-8 + 2^-16) in bf16
    one = torch.ones(1, 1, 32, dtype=BF16)
    xa1 = torch.tensor([[[1.0, 1.0]]], dtype=BF16)
    b1 = torch.zeros(2, 32, dtype=BF16)
    b1[0, 0], b1[1, 0] = 2.0 ** -8, 2.0 ** -16
    y = O.lora_add(one, xa1, b1)
    assert float(y[0, 0, 0]) == 1.0                        # product rounds to 2^-8, 1 + 2^-8 ties to even = 1
    assert float(torch.tensor(1.0 + 2.0 ** -8 + 2.0 ** -16).to(BF16)) == 1.0078125   # single rounding would go up


def test_lora_products_contract_the_right_index():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(3, 4, 32, generator=g).to(BF16)
    u = torch.randn(3, 4, 2, generator=g).to(BF16)
    v = torch.randn(2, 32, generator=g).to(BF16)
    p1, p2 = O.lora_products(x, u, v)
    assert p1.shape == (2, 32) and p2.shape == (3, 4, 2)
    w1 = torch.zeros(2, 32, dtype=torch.float64)
    w2 = torch.zeros(3, 4, 2, dtype=torch.float64)
    for bi in range(3):
        for t in range(4):
            for n in range(32):
                for r in range(2):
                    w1[r, n] += float(u[bi, t, r]) * float(x[bi, t, n])      # rows (batch and sequence) contracted
                    w2[bi, t, r] += float(x[bi, t, n]) * float(v[r, n])      # columns contracted
    assert same_bits(p1, w1.to(BF16)) and same_bits(p2, w2.to(BF16))
    assert O.lora_products(x, u)[1] is None and O.lora_products(x, v=v)[0] is None
