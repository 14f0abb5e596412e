"""A short LoRA fine-tuning run through a stack of fused layers: the loss of the run that keeps compressed
activations must follow the loss of the same run with plain torch autograd (uncompressed), through the
calibration steps and after the statistics are frozen.  A sanity check of the whole path at once - the
parity bars are in the operator and layer tests."""
import math
from types import SimpleNamespace

import pytest
import torch
import torch.nn.functional as F

from helpers import BF16
from test_gpu_layers import Lin, RefRMSNorm, config

pytestmark = pytest.mark.gpu

VOCAB, HIDDEN, HEADS, INTER, RANK, LAYERS, B, S = 97, 256, 2, 512, 16, 2, 4, 64


def build(dev, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    rn = lambda *s, sc=1.0: (torch.randn(*s, generator=g, device=dev) * sc).to(BF16)
    dims = dict(q=(HIDDEN, HIDDEN), k=(HIDDEN, HIDDEN), v=(HIDDEN, HIDDEN), o=(HIDDEN, HIDDEN),
                gate=(INTER, HIDDEN), up=(INTER, HIDDEN), down=(HIDDEN, INTER))
    layers = []
    for _ in range(LAYERS):
        P = {}
        for n, (out_f, in_f) in dims.items():
            P[n] = (Lin(rn(out_f, in_f, sc=1.0 / math.sqrt(in_f))),
                    Lin(rn(RANK, in_f, sc=1.0 / math.sqrt(in_f)).float().requires_grad_()),     # fp32 master adapters
                    Lin(torch.zeros(out_f, RANK, device=dev).requires_grad_()))                 # LoRA-B starts at zero
        layers.append(SimpleNamespace(P=P, nw1=torch.ones(HIDDEN, device=dev, dtype=BF16),
                                      nw2=torch.ones(HIDDEN, device=dev, dtype=BF16)))
    emb = rn(VOCAB, HIDDEN)
    head = rn(VOCAB, HIDDEN, sc=1.0 / math.sqrt(HIDDEN))
    hd = HIDDEN // HEADS
    pos = torch.arange(S, device=dev, dtype=torch.float32)
    inv = 1.0 / (1e4 ** (torch.arange(0, hd, 2, device=dev, dtype=torch.float32) / hd))
    ang = torch.cat([pos[:, None] * inv[None, :]] * 2, dim=-1)
    cos, sin = ang.cos().to(BF16)[None], ang.sin().to(BF16)[None]
    mask = torch.full((S, S), float("-inf"), device=dev).triu(1).to(BF16)[None, None]
    # a learnable toy language: the next token is a fixed function of the current one
    perm = torch.randperm(VOCAB, generator=g, device=dev)
    start = torch.randint(0, VOCAB, (64, B, 1), generator=g, device=dev)
    seqs = [start]
    for _ in range(S):
        seqs.append(perm[seqs[-1]])
    tokens = torch.cat(seqs, dim=-1)                   # [steps, B, S + 1]
    return SimpleNamespace(layers=layers, emb=emb, head=head, cos=cos, sin=sin, mask=mask, tokens=tokens, hd=hd)


def adapters(m):
    return [mod.weight for L in m.layers for n in L.P for mod in L.P[n][1:]]


def plain_layer(m, L, x):
    from hyclora_amd.models.compute_utils import head_to_hidden_shape, hidden_to_head_shape
    from oracle import hyc_oracle as O

    def proj(n, inp):
        base, la, lb = L.P[n]
        return inp @ base.weight.t() + (inp @ la.weight.to(BF16).t()) @ lb.weight.to(BF16).t()
    xn = RefRMSNorm.apply(x, L.nw1)
    q, k, v = (hidden_to_head_shape(proj(n, xn), HEADS) for n in ("q", "k", "v"))
    q = O.rope(q.transpose(1, 2), m.cos, m.sin).transpose(1, 2)
    k = O.rope(k.transpose(1, 2), m.cos, m.sin).transpose(1, 2)
    a = torch.softmax(q @ k.transpose(-2, -1) / math.sqrt(m.hd) + m.mask, dim=-1, dtype=BF16)
    xm = x + proj("o", head_to_hidden_shape(a @ v))
    xn2 = RefRMSNorm.apply(xm, L.nw2)
    return xm + proj("down", F.silu(proj("gate", xn2)) * proj("up", xn2))


def fused_layer(m, layer, L, x):
    # adapters are kept in fp32 by the optimiser and handed over in bf16, as a mixed-precision trainer does
    cast = lambda mod: Lin(mod.weight.to(BF16))
    args = [x, L.nw1, None, m.cos, m.sin]
    for n in ("q", "k", "v", "o"):
        args += [L.P[n][0], cast(L.P[n][1]), cast(L.P[n][2])]
    args += [L.nw2, None]
    for n in ("gate", "up", "down"):
        args += [L.P[n][0], cast(L.P[n][1]), cast(L.P[n][2])]
    return layer(*args, m.mask, HEADS, m.hd, HEADS)


def run(dev, arm, layer_type="intra_inter_full_fuse", q_bit=8, steps=40):
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import llama
    m = build(dev, seed=11)
    fused = [llama.make_fused_llama_layer(config(layer_type, q_bit, sm_ratio=0.2, thr=5)) for _ in m.layers] \
        if arm == "fused" else None
    opt = torch.optim.AdamW(adapters(m), lr=2e-3, weight_decay=0.0)
    losses = []
    for it in range(steps):
        tok = m.tokens[it % m.tokens.shape[0]]
        x = m.emb[tok[:, :-1]]
        for i, L in enumerate(m.layers):
            x = fused_layer(m, fused[i], L, x) if fused else plain_layer(m, L, x)
        logits = (x @ m.head.t()).float()
        loss = F.cross_entropy(logits.reshape(-1, VOCAB), tok[:, 1:].reshape(-1))
        opt.zero_grad(set_to_none=True)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    return losses, fused


@pytest.mark.parametrize("layer_type, q_bit, tol", [("intra_inter_full_fuse", 8, 0.02), ("intra_inter", 8, 0.02),
                                                   ("intra", 8, 0.02), ("intra_inter_full_fuse", 4, 0.02),
                                                   ("intra_inter_full_fuse", 2, 0.15)])
def test_compressed_fine_tuning_follows_the_uncompressed_run(dev, layer_type, q_bit, tol):
    ref, _ = run(dev, "plain")
    got, fused = run(dev, "fused", layer_type, q_bit)
    assert ref[-1] < 0.7 * ref[0], f"the toy task is not being learnt: {ref[0]:.3f} -> {ref[-1]:.3f}"
    assert all(layer.iteration == len(got) for layer in fused)
    assert fused[0].static_value["gate"]["scale"] is not None          # statistics were gathered, then frozen
    # gap of the two loss curves, step by step, as a share of the loss the runs start from (the toy task is learnt
    # almost perfectly, so a gap relative to the current loss would compare noise with noise at the end)
    worst = max(abs(a - b) for a, b in zip(got, ref)) / ref[0]
    print(f"{layer_type} q{q_bit}: loss {ref[0]:.3f} -> {ref[-1]:.4f} (plain), {got[-1]:.4f} (compressed), worst gap {worst:.3%} of the initial loss")
    assert worst <= tol, f"{layer_type} q{q_bit}: loss curves differ by {worst:.2%} of the initial loss (last losses {got[-5:]} vs {ref[-5:]})"
    assert got[-1] < 0.7 * got[0]
