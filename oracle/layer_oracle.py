"""Oracle restatement of one fused decoder layer: forward, what is saved (compressed), and the
hand-written backward that recomputes from the compressed activations.  TEST INFRASTRUCTURE ONLY.

Follows models/llama/fused_llama_layer_intra_inter_full_fuse.py:95-285 (forward) and :358-494
(backward), fused_llama_layer_intra_inter.py:352-383 and fused_llama_layer_intra.py:373-455 for the
other two layer types, using only plain torch operations and the element-level oracle functions of
hyc_oracle.py (device-agnostic: runs wherever the input tensors live).  One deviation, shared with
the implementation under test: the input-norm outliers are restored with the input-norm channel list
(the reference's intra_inter/full_fuse files pass the post-attention list, :484);
`as_reference_restores_x=True` restores them as the reference's text does.

The map-free variant (attention="flash") follows models/llama_flash_attn/fused_llama_layer_intra_inter.py:
zero-point codes for q and k (:128-139), causal attention through the flash kernel with its row log-sum-exps
kept (:156-180), and the kernel's backward formula applied to the rebuilt q, k, v and the dequantised output
(:450-468) - restated here with dense fp32 matrices.

Calibration is always "fresh" (iteration < threshold): statistics are computed from the tensors at hand.

Forward and backward are separate functions joined by a dict `saved` whose keys are the reference's names in
its ctx.save_for_backward lists (…full_fuse.py:254-285, fused_llama_layer_intra.py:267-300,
llama_flash_attn/fused_llama_layer_intra_inter.py:252-270) plus the ctx attributes backward reads (the two
channel lists, the map's shape, the flash kernel's log-sum-exps); the sparse map `a_o` is its (indices,
values) pair.  So the backward can also be run from saved state that something else produced.

Pinning (tests/test_oracle_layer.py, CPU):
  * with IdentityCodec (every compress call keeps the tensor as it is, the map keeps every entry) forward and
    backward of all three layer types x {map, flash} x {MHA, GQA} equal float64 autograd of the plain layer,
    whose only non-autograd piece is the mean term the reference's RMSNorm backward keeps; variants of the
    backward with one term dropped or one operand swapped fail that test;
  * the saved set per layer type equals the reference's save list written out by hand (names, shapes, dtypes).
The compress calls themselves are the element functions of hyc_oracle.py, pinned there.
"""
import math

import torch
import torch.nn.functional as F

from . import hyc_oracle as O


def _heads(x, h):
    b, s, d = x.shape
    return x.reshape(b, s, h, d // h).transpose(1, 2)


def _hidden(x):
    b, _, s, _ = x.shape
    return x.transpose(1, 2).reshape(b, s, -1).contiguous()


def _repeat(x, n):
    if n == 1:
        return x
    b, kv, s, d = x.shape
    return x[:, :, None].expand(b, kv, n, s, d).reshape(b, kv * n, s, d)


def _repeat_bwd(g, n):
    if n == 1:
        return g
    b, h, s, d = g.shape
    return g.reshape(b, h // n, n, s, d).sum(dim=2)


def _rope(x, cos, sin, sign=1.0):
    # operators/rope_kernels.py:56-78: first-half cos/sin, rotate the two halves; backward = -sin
    cos, sin = cos.squeeze(), sin.squeeze()
    seq, half = x.shape[1], x.shape[-1] // 2
    c = cos[:seq, :half][None, :, None, :]
    s = sin[:seq, :half][None, :, None, :] * sign
    x1, x2 = x[..., :half].to(s.dtype), x[..., half:].to(s.dtype)
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1).to(x.dtype)


def _flash_forward(q, k, v, scale):
    """Causal attention as the flash kernels define it (llama_flash_attn/fused_llama_layer_intra_inter.py:156-180,
    flash_attn 2.5.8 `_flash_attn_varlen_forward`, causal=True, no dropout): fp32 scores (float64 for float64
    operands), row log-sum-exps kept, output rounded once.  -> (o [B,H,S,D] in q's dtype, lse [B,H,S])."""
    f = torch.promote_types(q.dtype, torch.float32)
    s = (q.to(f) @ k.to(f).transpose(-2, -1)) * scale
    n = s.shape[-1]
    s = s + torch.full((n, n), float("-inf"), device=s.device, dtype=f).triu(1)
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse.unsqueeze(-1))
    return (p @ v.to(f)).to(q.dtype), lse


def _flash_backward(g_o, q, k, v, out, lse, scale):
    """What `_flash_attn_varlen_backward` computes from the tensors it is GIVEN (…intra_inter.py:450-468: q, k, v
    rebuilt from their codes and `out` dequantised, `softmax_lse` the one saved in forward): the probabilities are
    recomputed from q, k and the saved log-sum-exps, the row term is sum(dO * out) of the given output.
    -> (grad_q, grad_k, grad_v)."""
    f = torch.promote_types(q.dtype, torch.float32)
    s = (q.to(f) @ k.to(f).transpose(-2, -1)) * scale
    n = s.shape[-1]
    s = s + torch.full((n, n), float("-inf"), device=s.device, dtype=f).triu(1)
    p = torch.exp(s - lse.to(f).unsqueeze(-1))
    gof = g_o.to(f)
    d_p = gof @ v.to(f).transpose(-2, -1)
    delta = (gof * out.to(f)).sum(dim=-1, keepdim=True)
    d_s = p * (d_p - delta)
    g_q = (d_s @ k.to(f)) * scale
    g_k = (d_s.transpose(-2, -1) @ q.to(f)) * scale
    g_v = p.transpose(-2, -1) @ gof
    return g_q.to(q.dtype), g_k.to(q.dtype), g_v.to(q.dtype)


class ReferenceCodec:
    """The compress / decompress calls of the reference's layers, calibrating (statistics from the tensor at
    hand): compression_pack_quant_base, compression_pack_quant_zp_base, compression_pack_channel_base,
    compression_pack_softmax_base and their inverses (operators/compress_function.py:346-379, :147-174,
    :214-241, :278-306, :316-317), and the two fused kernels of the full_fuse layer type."""

    def __init__(self, q_bit, softmax_ratio, layernorm_ratio):
        self.q_bit, self.softmax_ratio, self.layernorm_ratio = q_bit, softmax_ratio, layernorm_ratio

    def quant(self, t):
        s = O.scale_only_quant(t, self.q_bit)
        return O.compress(t, s, self.q_bit), s

    def quant_zp(self, t):
        s, z = O.scale_zero_point(t, self.q_bit)
        return O.compress(t, s, self.q_bit, z), s, z

    def dequant(self, q, s, z=None, is_head=False, num_heads=1):
        return O.decompress(q, s, self.q_bit, z, is_head=is_head, num_heads=num_heads)

    def channel_base(self, t):
        idx, s = O.channel_stats(t, self.layernorm_ratio, self.q_bit)
        xo, q = O.compress_channel_base(t, s, idx, self.q_bit)
        return xo, q, idx, s

    def channel_base_restore(self, xo, q, idx, s):
        return O.decompress_channel_base(q, s, xo, idx, self.q_bit)

    def prune_map(self, a):
        thr = O.softmax_threshold(a, self.softmax_ratio)
        return O.softmax_compress(a, thr) + (thr,)

    def restore_map(self, idx, val, shape):
        return O.softmax_restore(idx, val, shape)

    def fused_forward(self, xa1, b1, x1, xa2, b2, x2):
        s1, s2 = O.scale_only_quant(x1, self.q_bit), O.scale_only_quant(x2, self.q_bit)
        q1, q2, had = O.fused_fwd(xa1, b1, x1, s1, xa2, b2, x2, s2, self.q_bit)
        return q1, s1, q2, s2, had

    def fused_backward(self, xa1, b1, q1, s1, xa2, b2, q2, s2, g):
        return O.fused_bwd(xa1, b1, q1, s1, xa2, b2, q2, s2, g, self.q_bit)


class IdentityCodec:
    """For pinning the layer logic only: every compress call keeps its tensor as it is (the "codes" are the
    tensor, scale and zero point are None) and the attention map keeps every entry; the channel-base calls
    still split off int(N * layernorm_ratio) outlier channels - exactly, the remainder is kept with those
    columns zeroed - so that the channel lists still matter.  What is saved under which name, what is
    recomputed from what and in which order stay as they are, so forward + backward must then be the gradient
    of the plain layer."""

    def __init__(self, layernorm_ratio=0.0):
        self.layernorm_ratio = layernorm_ratio

    def quant(self, t):
        return t, None

    def quant_zp(self, t):
        return t, None, None

    def dequant(self, q, s, z=None, is_head=False, num_heads=1):
        return _heads(q, num_heads) if is_head and q.dim() == 3 else q

    def channel_base(self, t):
        idx = O.outlier_channels(t, self.layernorm_ratio)
        rest = t.clone()
        rest[..., idx] = 0
        return t[..., idx], rest, idx, None

    def channel_base_restore(self, xo, q, idx, s):
        x = q.clone()
        x[..., idx] = xo
        return x

    def prune_map(self, a):
        return O.softmax_compress(a, float("-inf")) + (None,)

    def restore_map(self, idx, val, shape):
        return O.softmax_restore(idx, val, shape)

    def fused_forward(self, xa1, b1, x1, xa2, b2, x2):
        had = O.silu_mul(O.lora_add(x1, xa1, b1), O.lora_add(x2, xa2, b2))
        return x1, None, x2, None, had

    def fused_backward(self, xa1, b1, q1, s1, xa2, b2, q2, s2, g):
        return O.fused_bwd_dense(xa1, b1, q1, xa2, b2, q2, g)


def _transposed(weights):
    return ({n: w[0].t() for n, w in weights.items()},       # [in, out]
            {n: w[1].t() for n, w in weights.items()},       # [in, r]
            {n: w[2].t() for n, w in weights.items()})       # [r, out]


def layer_forward(x, nw1, nw2, cos, sin, weights, mask, heads, kv_heads, *, mode, q_bit, softmax_ratio,
                  layernorm_ratio, eps=1e-5, attention="map", codec=None):
    """-> (x_out, saved).  weights: name -> (W [out,in], A [r,in], B [out,r]) for q,k,v,o,gate,up,down (plain
    tensors).  attention="flash": the map-free variant (models/llama_flash_attn/fused_llama_layer_intra_inter.py):
    causal attention without a saved map, q and k compressed with a zero point (:128-139); `mask` is not used."""
    C = codec or ReferenceCodec(q_bit, softmax_ratio, layernorm_ratio)
    hd = x.shape[-1] // heads
    n_rep = heads // kv_heads
    Wt, At, Bt = _transposed(weights)
    flash = attention == "flash"
    S = {}

    def lora_fwd(n, inp):                                # compute_utils.py:18-25
        main = inp @ Wt[n]
        xa = inp @ At[n]
        return main + xa @ Bt[n], main, xa

    def keep(name, t):                                   # compression_pack_quant_base
        S[name + "_q"], S[name + "_scale"] = C.quant(t)

    def keep_zp(name, t):                                # compression_pack_quant_zp_base
        S[name + "_q"], S[name + "_scale"], S[name + "_zero_point"] = C.quant_zp(t)

    def keep_channel_base(name, t):                      # compression_pack_channel_base
        S[name + "_o"], S[name + "_q"], S[name + "_channel_idx"], S[name + "_scale"] = C.channel_base(t)

    keep_qk = keep_zp if flash else keep                 # q and k: with a zero point in the map-free variant

    xn1, S["rstd_1"] = O.rmsnorm_fwd(x, nw1, eps)
    keep_channel_base("x", x)
    q, q_main, S["q_lora_a"] = lora_fwd("q", xn1)
    k, k_main, S["k_lora_a"] = lora_fwd("k", xn1)
    v, v_main, S["v_lora_a"] = lora_fwd("v", xn1)
    keep("x_norm_1", xn1)
    if mode != "intra":
        keep_qk("q_main", q_main), keep_qk("k_main", k_main), keep("v_main", v_main)
    q, k, v = _heads(q, heads), _heads(k, kv_heads), _heads(v, kv_heads)
    q = _rope(q.transpose(1, 2), cos, sin).transpose(1, 2)
    k = _rope(k.transpose(1, 2), cos, sin).transpose(1, 2)
    k, v = _repeat(k, n_rep), _repeat(v, n_rep)
    if mode == "intra":
        keep_qk("q", q), keep_qk("k", k), keep("v", v)  # 4-D inputs are read as [B, S, H*D]
    if flash:
        o, S["softmax_lse"] = _flash_forward(q, k, v, 1.0 / math.sqrt(hd))
        o = _hidden(o)
    else:
        s = q @ k.transpose(-2, -1) / math.sqrt(hd)
        if mask is not None:
            s = s + mask
        a = torch.softmax(s, dim=-1, dtype=v.dtype)
        S["a_o_indices"], S["a_o_values"], S["a_threshold"] = C.prune_map(a)
        S["a_shape"] = tuple(a.shape)
        o = _hidden(a @ v)
    o_final, _, S["o_final_lora_a"] = lora_fwd("o", o)
    keep("o", o)
    xm = x + o_final
    xn2, S["rstd_2"] = O.rmsnorm_fwd(xm, nw2, eps)
    keep_channel_base("x_medium", xm)
    if mode == "intra_inter_full_fuse":
        gate_main, up_main = xn2 @ Wt["gate"], xn2 @ Wt["up"]
        S["gate_lora_a"], S["up_lora_a"] = xn2 @ At["gate"], xn2 @ At["up"]
        S["gate_main_q"], S["gate_main_scale"], S["up_main_q"], S["up_main_scale"], had = C.fused_forward(
            S["gate_lora_a"], Bt["gate"], gate_main, S["up_lora_a"], Bt["up"], up_main)
        had = had.to(x.device)
    else:
        gate, gate_main, S["gate_lora_a"] = lora_fwd("gate", xn2)
        up, up_main, S["up_lora_a"] = lora_fwd("up", xn2)
        if mode == "intra_inter":
            keep("gate_main", gate_main), keep("up_main", up_main)
            had = O.silu_mul(gate, up)
        else:
            fn = F.silu(gate)
            keep("gate", gate)
            had = up * fn
            keep("up", up), keep("fn", fn)
    keep("x_norm_2", xn2)
    down, _, S["down_lora_a"] = lora_fwd("down", had)
    if mode == "intra":
        keep("hadamard", had)
    return xm + down, S


def layer_backward(S, grad_out, nw1, nw2, cos, sin, weights, heads, kv_heads, *, mode, q_bit, attention="map",
                   codec=None, as_reference_restores_x=False):
    """Gradients from the saved state `S` of layer_forward (or of anything that saves the same things):
    {'x': .., 'nw1': .., 'nw2': .., (name,'A'): .., (name,'B'): ..}; the LoRA gradients keep the batch axis
    (sum over it for the parameter's gradient).  as_reference_restores_x: the input-norm outliers are put back
    at the post-attention norm's channels, as …full_fuse.py:484 / fused_llama_layer_intra_inter.py:494 write it
    (layer types intra_inter and intra_inter_full_fuse only; 'intra' passes the right list, :492)."""
    C = codec or ReferenceCodec(q_bit, 0.0, 0.0)
    hd = nw1.numel() // heads
    n_rep = heads // kv_heads
    Wt, At, Bt = _transposed(weights)
    flash = attention == "flash"
    dev = grad_out.device
    G = {}

    def lora_bwd(n, inp, xa, gy):                        # compute_utils.py:28-36
        gmid = gy @ Bt[n].mT
        ga = inp.mT @ gmid
        gb = xa.mT @ gy
        gx = gy @ Wt[n].T
        gx = gx + gmid @ At[n].T
        return ga, gb, gx

    def dq(name, **kw):
        return C.dequant(S[name + "_q"], S[name + "_scale"], S.get(name + "_zero_point"), **kw).to(dev, grad_out.dtype)

    go = grad_out
    if mode == "intra_inter_full_fuse":
        G[("down", "B")] = S["down_lora_a"].mT @ go
        g_down = go @ Wt["down"].T
        g_mid = go @ Bt["down"].T
        g_down = g_down + g_mid @ At["down"].T
        had_r, g_fn, g_h2 = C.fused_backward(S["gate_lora_a"], Bt["gate"], S["gate_main_q"], S["gate_main_scale"],
                                             S["up_lora_a"], Bt["up"], S["up_main_q"], S["up_main_scale"], g_down)
        had_r, g_fn, g_h2 = had_r.to(dev), g_fn.to(dev), g_h2.to(dev)
        G[("down", "A")] = had_r.mT @ g_mid
    else:
        if mode == "intra_inter":
            gate = dq("gate_main") + S["gate_lora_a"] @ Bt["gate"]
            up = dq("up_main") + S["up_lora_a"] @ Bt["up"]
            fn = F.silu(gate)
            had_r = up * fn
        else:
            had_r, up, fn, gate = dq("hadamard"), dq("up"), dq("fn"), dq("gate")
        G[("down", "A")], G[("down", "B")], g_down = lora_bwd("down", had_r, S["down_lora_a"], go)
        g_h1, g_h2 = g_down * up, g_down * fn
        g_fn = O.silu_bwd(gate, g_h1)
    xn2_r = dq("x_norm_2")
    G[("gate", "A")], G[("gate", "B")], g1 = lora_bwd("gate", xn2_r, S["gate_lora_a"], g_fn)
    G[("up", "A")], G[("up", "B")], g2 = lora_bwd("up", xn2_r, S["up_lora_a"], g_h2)
    g_gate_up = g2 + g1
    xm_r = C.channel_base_restore(S["x_medium_o"], S["x_medium_q"], S["x_medium_channel_idx"], S["x_medium_scale"]).to(dev)
    g_norm2, G["nw2"] = O.rmsnorm_bwd(g_gate_up, xm_r, nw2, S["rstd_2"])
    g_medium = g_norm2 + go
    o_r = dq("o")
    G[("o", "A")], G[("o", "B")], g_o = lora_bwd("o", o_r, S["o_final_lora_a"], g_medium)
    g_o = _heads(g_o, heads)
    if mode == "intra":
        q_r, k_r, v_r = (dq(n, is_head=True, num_heads=heads) for n in ("q", "k", "v"))
    else:
        v_r = _repeat(_heads(dq("v_main") + S["v_lora_a"] @ Bt["v"], kv_heads), n_rep)
        q_r = _heads(dq("q_main") + S["q_lora_a"] @ Bt["q"], heads)
        q_r = _rope(q_r.transpose(1, 2), cos, sin).transpose(1, 2)
        k_r = _heads(dq("k_main") + S["k_lora_a"] @ Bt["k"], kv_heads)
        k_r = _repeat(_rope(k_r.transpose(1, 2), cos, sin).transpose(1, 2), n_rep)
    if flash:
        g_q, g_k, g_v = _flash_backward(g_o, q_r, k_r, v_r, _heads(o_r, heads), S["softmax_lse"], 1.0 / math.sqrt(hd))
        g_k, g_v = _repeat_bwd(g_k, n_rep), _repeat_bwd(g_v, n_rep)
    else:
        a_r = C.restore_map(S["a_o_indices"], S["a_o_values"], S["a_shape"]).to(dev)
        g_v = a_r.transpose(-2, -1) @ g_o
        g_a = g_o @ v_r.transpose(-2, -1)
        g_v = _repeat_bwd(g_v, n_rep)
        g_s = O.softmax_bwd(a_r, g_a) / math.sqrt(hd)
        g_k = _repeat_bwd(g_s.transpose(-2, -1) @ q_r, n_rep)
        g_q = g_s @ k_r
    g_q = _rope(g_q.transpose(1, 2), cos, sin, -1.0).transpose(1, 2)
    g_k = _rope(g_k.transpose(1, 2), cos, sin, -1.0).transpose(1, 2)
    g_q, g_k, g_v = _hidden(g_q), _hidden(g_k), _hidden(g_v)
    xn1_r = dq("x_norm_1")
    G[("q", "A")], G[("q", "B")], gx = lora_bwd("q", xn1_r, S["q_lora_a"], g_q)
    G[("k", "A")], G[("k", "B")], gt = lora_bwd("k", xn1_r, S["k_lora_a"], g_k)
    gx = gx + gt
    G[("v", "A")], G[("v", "B")], gt = lora_bwd("v", xn1_r, S["v_lora_a"], g_v)
    gx = gx + gt
    x_list = S["x_medium_channel_idx"] if as_reference_restores_x and mode != "intra" else S["x_channel_idx"]
    x_r = C.channel_base_restore(S["x_o"], S["x_q"], x_list, S["x_scale"]).to(dev)
    g_norm1, G["nw1"] = O.rmsnorm_bwd(gx, x_r, nw1, S["rstd_1"])
    G["x"] = g_norm1 + g_medium
    return G


def layer_forward_backward(x, nw1, nw2, cos, sin, weights, mask, heads, kv_heads, grad_out, *, mode, q_bit,
                           softmax_ratio, layernorm_ratio, eps=1e-5, attention="map", codec=None,
                           as_reference_restores_x=False):
    """layer_forward, then layer_backward from what it saved.  Returns (x_out, grads)."""
    x_out, S = layer_forward(x, nw1, nw2, cos, sin, weights, mask, heads, kv_heads, mode=mode, q_bit=q_bit,
                             softmax_ratio=softmax_ratio, layernorm_ratio=layernorm_ratio, eps=eps,
                             attention=attention, codec=codec)
    G = layer_backward(S, grad_out, nw1, nw2, cos, sin, weights, heads, kv_heads, mode=mode, q_bit=q_bit,
                       attention=attention, codec=codec, as_reference_restores_x=as_reference_restores_x)
    return x_out, G


def roberta_layer_forward(x, weights, ln1, ln2, mask, heads, *, mode, q_bit, softmax_ratio, layernorm_ratio,
                          eps=1e-5, codec=None):
    """Encoder (post-LayerNorm, GELU) layer forward: models/roberta/fused_roberta_layer_intra_inter.py:86-200 and
    fused_roberta_layer_intra.py:86-205.  weights: name -> (W [out,in], bias [out] or None, A [r,in], B [out,r])
    for q,k,v,o,up,down; ln1 / ln2: (weight, bias).  -> (x_out, saved), saved named as the reference's save
    list names its entries (fused_roberta_layer_intra_inter.py:202-232)."""
    C = codec or ReferenceCodec(q_bit, softmax_ratio, layernorm_ratio)
    hd = x.shape[-1] // heads
    Wt = {n: w[0].t() for n, w in weights.items()}
    bias = {n: w[1] for n, w in weights.items()}
    At = {n: w[2].t() for n, w in weights.items()}
    Bt = {n: w[3].t() for n, w in weights.items()}
    S = {}

    def lora_fwd(n, inp):
        main = inp @ Wt[n]
        if bias[n] is not None:
            main = main + bias[n]
        xa = inp @ At[n]
        return main + xa @ Bt[n], main, xa

    def keep(name, t):
        S[name + "_q"], S[name + "_scale"] = C.quant(t)

    def keep_channel_base(name, t):
        S[name + "_o"], S[name + "_q"], S[name + "_channel_idx"], S[name + "_scale"] = C.channel_base(t)

    q, q_main, S["q_lora_a"] = lora_fwd("q", x)
    k, k_main, S["k_lora_a"] = lora_fwd("k", x)
    v, v_main, S["v_lora_a"] = lora_fwd("v", x)
    keep("x", x)
    if mode == "intra_inter":
        keep("q_main", q_main), keep("k_main", k_main), keep("v_main", v_main)
    q, k, v = _heads(q, heads), _heads(k, heads), _heads(v, heads)
    if mode == "intra":
        keep("q", q), keep("k", k)
    a = O.softmax_fwd(q @ k.transpose(-2, -1), 1.0 / math.sqrt(hd), mask)
    o = a @ v
    S["a_o_indices"], S["a_o_values"], S["a_threshold"] = C.prune_map(a)
    S["a_shape"] = tuple(a.shape)
    if mode == "intra":
        keep("v", v)
    o = _hidden(o)
    o_final, _, S["o_final_lora_a"] = lora_fwd("o", o)
    keep("o", o)
    o_final = o_final + x
    x_medium, S["mean_1"], S["rstd_1"] = O.layernorm_fwd(o_final, ln1[0], ln1[1], eps)
    keep_channel_base("o_final", o_final)
    up, up_main, S["up_lora_a"] = lora_fwd("up", x_medium)
    keep("x_medium", x_medium)
    if mode == "intra_inter":
        keep("up_main", up_main)
    fn = F.gelu(up)
    if mode == "intra":
        keep("up", up)
    down, _, S["down_lora_a"] = lora_fwd("down", fn)
    down = down + x_medium
    if mode == "intra":
        keep("fn", fn)
    x_out, S["mean_2"], S["rstd_2"] = O.layernorm_fwd(down, ln2[0], ln2[1], eps)
    keep_channel_base("down", down)
    return x_out, S


def roberta_layer_backward(S, grad_out, weights, ln1, ln2, heads, *, mode, q_bit, codec=None):
    """Backward of the encoder layer from its saved state: fused_roberta_layer_intra_inter.py:362-455 and
    fused_roberta_layer_intra.py:373-440.  Gradients as layer_backward returns them (no norm-weight ones)."""
    C = codec or ReferenceCodec(q_bit, 0.0, 0.0)
    hd = ln1[0].numel() // heads
    Wt = {n: w[0].t() for n, w in weights.items()}
    At = {n: w[2].t() for n, w in weights.items()}
    Bt = {n: w[3].t() for n, w in weights.items()}
    dev = grad_out.device
    G = {}

    def lora_bwd(n, inp, xa, gy):
        gmid = gy @ Bt[n].mT
        ga = inp.mT @ gmid
        gb = xa.mT @ gy
        gx = gy @ Wt[n].T
        gx = gx + gmid @ At[n].T
        return ga, gb, gx

    def dq(name, **kw):
        return C.dequant(S[name + "_q"], S[name + "_scale"], **kw).to(dev, grad_out.dtype)

    def restored(name):
        return C.channel_base_restore(S[name + "_o"], S[name + "_q"], S[name + "_channel_idx"], S[name + "_scale"]).to(dev)

    g_ln2 = O.layernorm_bwd(grad_out, restored("down"), ln2[0], S["mean_2"], S["rstd_2"])
    if mode == "intra":
        fn_r, up_r = dq("fn"), dq("up")
    else:
        up_r = dq("up_main") + S["up_lora_a"] @ Bt["up"]
        fn_r = F.gelu(up_r)
    G[("down", "A")], G[("down", "B")], g_down = lora_bwd("down", fn_r, S["down_lora_a"], g_ln2)
    g_fn = O.gelu_bwd(up_r, g_down)
    G[("up", "A")], G[("up", "B")], g_up = lora_bwd("up", dq("x_medium"), S["up_lora_a"], g_fn)
    g_medium = g_ln2 + g_up
    g_ln1 = O.layernorm_bwd(g_medium, restored("o_final"), ln1[0], S["mean_1"], S["rstd_1"])
    G[("o", "A")], G[("o", "B")], g_o = lora_bwd("o", dq("o"), S["o_final_lora_a"], g_ln1)
    g_o = _heads(g_o, heads)
    a_r = C.restore_map(S["a_o_indices"], S["a_o_values"], S["a_shape"]).to(dev)
    if mode == "intra":
        q_r, k_r, v_r = (dq(n, is_head=True, num_heads=heads) for n in ("q", "k", "v"))
    else:
        v_r = _heads(dq("v_main") + S["v_lora_a"] @ Bt["v"], heads)
        q_r = _heads(dq("q_main") + S["q_lora_a"] @ Bt["q"], heads)
        k_r = _heads(dq("k_main") + S["k_lora_a"] @ Bt["k"], heads)
    g_v = a_r.transpose(-2, -1) @ g_o
    g_a = g_o @ v_r.transpose(-2, -1)
    g_s = O.softmax_bwd(a_r, g_a) / math.sqrt(hd)
    g_k = g_s.transpose(-2, -1) @ q_r
    g_q = g_s @ k_r
    g_q, g_k, g_v = _hidden(g_q), _hidden(g_k), _hidden(g_v)
    x_r = dq("x")
    G[("q", "A")], G[("q", "B")], gx = lora_bwd("q", x_r, S["q_lora_a"], g_q)
    G[("k", "A")], G[("k", "B")], gt = lora_bwd("k", x_r, S["k_lora_a"], g_k)
    gx = gx + gt
    G[("v", "A")], G[("v", "B")], gt = lora_bwd("v", x_r, S["v_lora_a"], g_v)
    gx = gx + gt
    G["x"] = gx + g_ln1
    return G


def roberta_layer_forward_backward(x, weights, ln1, ln2, mask, heads, grad_out, *, mode, q_bit, softmax_ratio,
                                   layernorm_ratio, eps=1e-5, codec=None):
    """roberta_layer_forward, then roberta_layer_backward from what it saved.  Returns (x_out, grads)."""
    x_out, S = roberta_layer_forward(x, weights, ln1, ln2, mask, heads, mode=mode, q_bit=q_bit,
                                     softmax_ratio=softmax_ratio, layernorm_ratio=layernorm_ratio, eps=eps, codec=codec)
    return x_out, roberta_layer_backward(S, grad_out, weights, ln1, ln2, heads, mode=mode, q_bit=q_bit, codec=codec)
