"""Oracle restatement of one fused decoder layer: forward, what is saved (compressed), and the
hand-written backward that recomputes from the compressed activations.  TEST INFRASTRUCTURE ONLY.

Follows models/llama/fused_llama_layer_intra_inter_full_fuse.py:95-285 (forward) and :358-494
(backward), fused_llama_layer_intra_inter.py:352-383 and fused_llama_layer_intra.py:373-455 for the
other two layer types, using only plain torch operations and the element-level oracle functions of
hyc_oracle.py (device-agnostic: runs wherever the input tensors live).  One deviation, shared with
the implementation under test: the input-norm outliers are restored with the input-norm channel list
(the reference's intra_inter/full_fuse files pass the post-attention list, :484).

The map-free variant (attention="flash") follows models/llama_flash_attn/fused_llama_layer_intra_inter.py:
zero-point codes for q and k (:128-139), causal attention through the flash kernel with its row log-sum-exps
kept (:156-180), and the kernel's backward formula applied to the rebuilt q, k, v and the dequantised output
(:450-468) - restated here with dense fp32 matrices.

Calibration is always "fresh" (iteration < threshold): statistics are computed from the tensors at hand.
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
    flash_attn 2.5.8 `_flash_attn_varlen_forward`, causal=True, no dropout): fp32 scores, row log-sum-exps kept,
    output rounded once.  -> (o [B,H,S,D] in q's dtype, lse fp32 [B,H,S])."""
    s = (q.float() @ k.float().transpose(-2, -1)) * scale
    n = s.shape[-1]
    s = s + torch.full((n, n), float("-inf"), device=s.device).triu(1)
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse.unsqueeze(-1))
    return (p @ v.float()).to(q.dtype), lse


def _flash_backward(g_o, q, k, v, out, lse, scale):
    """What `_flash_attn_varlen_backward` computes from the tensors it is GIVEN (…intra_inter.py:450-468: q, k, v
    rebuilt from their codes and `out` dequantised, `softmax_lse` the one saved in forward): the probabilities are
    recomputed from q, k and the saved log-sum-exps, the row term is sum(dO * out) of the given output.
    -> (grad_q, grad_k, grad_v)."""
    s = (q.float() @ k.float().transpose(-2, -1)) * scale
    n = s.shape[-1]
    s = s + torch.full((n, n), float("-inf"), device=s.device).triu(1)
    p = torch.exp(s - lse.unsqueeze(-1))
    gof = g_o.float()
    d_p = gof @ v.float().transpose(-2, -1)
    delta = (gof * out.float()).sum(dim=-1, keepdim=True)
    d_s = p * (d_p - delta)
    g_q = (d_s @ k.float()) * scale
    g_k = (d_s.transpose(-2, -1) @ q.float()) * scale
    g_v = p.transpose(-2, -1) @ gof
    return g_q.to(q.dtype), g_k.to(q.dtype), g_v.to(q.dtype)


def layer_forward_backward(x, nw1, nw2, cos, sin, weights, mask, heads, kv_heads, grad_out, *, mode, q_bit,
                           softmax_ratio, layernorm_ratio, eps=1e-5, attention="map"):
    """weights: name -> (W [out,in], A [r,in], B [out,r]) for q,k,v,o,gate,up,down (plain tensors).
    Returns (x_out, grads) with grads = {'x': .., (name,'A'): .., (name,'B'): ..}.
    attention="flash": the map-free variant (models/llama_flash_attn/fused_llama_layer_intra_inter.py): causal
    attention without a saved map, q and k compressed with a zero point (:128-139), backward through the flash
    kernel's formula on the rebuilt q, k, v and the dequantised output (:450-468); `mask` is not used."""
    hd = x.shape[-1] // heads
    n_rep = heads // kv_heads
    At = {n: w[1].t() for n, w in weights.items()}      # [in, r]
    Bt = {n: w[2].t() for n, w in weights.items()}      # [r, out]
    Wt = {n: w[0].t() for n, w in weights.items()}      # [in, out]

    def lora_fwd(n, inp):                                # compute_utils.py:18-25
        main = inp @ Wt[n]
        xa = inp @ At[n]
        return main + xa @ Bt[n], main, xa

    def lora_bwd(n, inp, xa, gy):                        # compute_utils.py:28-36
        gmid = gy @ Bt[n].mT
        ga = inp.mT @ gmid
        gb = xa.mT @ gy
        gx = gy @ Wt[n].T
        gx = gx + gmid @ At[n].T
        return ga, gb, gx

    def cq(t):                                           # compression_pack_quant_base, calibrating
        s = O.scale_only_quant(t, q_bit)
        return O.compress(t, s, q_bit), s

    def cqz(t):                                          # compression_pack_quant_zp_base, calibrating
        s, z = O.scale_zero_point(t, q_bit)
        return O.compress(t, s, q_bit, z), s, z

    flash = attention == "flash"
    cqk = cqz if flash else cq                           # q and k: with a zero point in the map-free variant

    def ccb(t):                                          # compression_pack_channel_base, calibrating
        idx, s = O.channel_stats(t, layernorm_ratio, q_bit)
        xo, q = O.compress_channel_base(t, s, idx, q_bit)
        return xo, q, idx, s

    # ------------------------------ forward ------------------------------
    xn1, rstd1 = O.rmsnorm_fwd(x, nw1, eps)
    x_sv = ccb(x)
    q, q_main, q_xa = lora_fwd("q", xn1)
    k, k_main, k_xa = lora_fwd("k", xn1)
    v, v_main, v_xa = lora_fwd("v", xn1)
    xn1_sv = cq(xn1)
    if mode != "intra":
        q_sv, k_sv, v_sv = cqk(q_main), cqk(k_main), cq(v_main)
    q, k, v = _heads(q, heads), _heads(k, kv_heads), _heads(v, kv_heads)
    q = _rope(q.transpose(1, 2), cos, sin).transpose(1, 2)
    k = _rope(k.transpose(1, 2), cos, sin).transpose(1, 2)
    k, v = _repeat(k, n_rep), _repeat(v, n_rep)
    if mode == "intra":
        q_sv, k_sv, v_sv = cqk(q), cqk(k), cq(v)         # 4-D inputs are read as [B, S, H*D]
    if flash:
        o, lse = _flash_forward(q, k, v, 1.0 / math.sqrt(hd))
        o = _hidden(o)
    else:
        s = q @ k.transpose(-2, -1) / math.sqrt(hd)
        if mask is not None:
            s = s + mask
        a = torch.softmax(s, dim=-1, dtype=v.dtype)
        thr = O.softmax_threshold(a, softmax_ratio)
        a_idx, a_val = O.softmax_compress(a, thr)
        a_shape = a.shape
        o = _hidden(a @ v)
    o_final, _, o_xa = lora_fwd("o", o)
    o_sv = cq(o)
    xm = x + o_final
    xn2, rstd2 = O.rmsnorm_fwd(xm, nw2, eps)
    xm_sv = ccb(xm)
    if mode == "intra_inter_full_fuse":
        gate_main, up_main = xn2 @ Wt["gate"], xn2 @ Wt["up"]
        gate_xa, up_xa = xn2 @ At["gate"], xn2 @ At["up"]
        gs, us = O.scale_only_quant(gate_main, q_bit), O.scale_only_quant(up_main, q_bit)
        gq, uq, had = O.fused_fwd(gate_xa, Bt["gate"], gate_main, gs, up_xa, Bt["up"], up_main, us, q_bit)
        had = had.to(x.device)
    else:
        gate, gate_main, gate_xa = lora_fwd("gate", xn2)
        up, up_main, up_xa = lora_fwd("up", xn2)
        if mode == "intra_inter":
            gate_sv, up_sv = cq(gate_main), cq(up_main)
            had = O.silu_mul(gate, up)
        else:
            fn = F.silu(gate)
            gate_sv = cq(gate)
            had = up * fn
            up_sv, fn_sv = cq(up), cq(fn)
    xn2_sv = cq(xn2)
    down, _, down_xa = lora_fwd("down", had)
    if mode == "intra":
        had_sv = cq(had)
    x_out = xm + down

    # ------------------------------ backward ------------------------------
    G = {}
    dq = lambda sv, **kw: O.decompress(sv[0], sv[1], q_bit, **kw).to(x.device)
    go = grad_out
    if mode == "intra_inter_full_fuse":
        G[("down", "B")] = down_xa.mT @ go
        g_down = go @ Wt["down"].T
        g_mid = go @ Bt["down"].T
        g_down = g_down + g_mid @ At["down"].T
        had_r, g_fn, g_h2 = O.fused_bwd(gate_xa, Bt["gate"], gq, gs, up_xa, Bt["up"], uq, us, g_down, q_bit)
        G[("down", "A")] = had_r.mT @ g_mid
    else:
        if mode == "intra_inter":
            gate = dq(gate_sv) + gate_xa @ Bt["gate"]
            up = dq(up_sv) + up_xa @ Bt["up"]
            fn = F.silu(gate)
            had_r = up * fn
        else:
            had_r, up, fn, gate = dq(had_sv), dq(up_sv), dq(fn_sv), dq(gate_sv)
        G[("down", "A")], G[("down", "B")], g_down = lora_bwd("down", had_r, down_xa, go)
        g_h1, g_h2 = g_down * up, g_down * fn
        g_fn = O.silu_bwd(gate, g_h1)
    xn2_r = dq(xn2_sv)
    G[("gate", "A")], G[("gate", "B")], g1 = lora_bwd("gate", xn2_r, gate_xa, g_fn)
    G[("up", "A")], G[("up", "B")], g2 = lora_bwd("up", xn2_r, up_xa, g_h2)
    g_gate_up = g2 + g1
    xm_r = O.decompress_channel_base(xm_sv[1], xm_sv[3], xm_sv[0], xm_sv[2], q_bit)
    g_norm2, G["nw2"] = O.rmsnorm_bwd(g_gate_up, xm_r, nw2, rstd2)
    g_medium = g_norm2 + go
    o_r = dq(o_sv)
    G[("o", "A")], G[("o", "B")], g_o = lora_bwd("o", o_r, o_xa, g_medium)
    g_o = _heads(g_o, heads)
    dqk = (lambda sv, **kw: O.decompress(sv[0], sv[1], q_bit, sv[2], **kw).to(x.device)) if flash else dq
    if mode == "intra":
        q_r, k_r = (dqk(sv, is_head=True, num_heads=heads) for sv in (q_sv, k_sv))
        v_r = dq(v_sv, is_head=True, num_heads=heads)
    else:
        v_r = _repeat(_heads(dq(v_sv) + v_xa @ Bt["v"], kv_heads), n_rep)
        q_r = _heads(dqk(q_sv) + q_xa @ Bt["q"], heads)
        q_r = _rope(q_r.transpose(1, 2), cos, sin).transpose(1, 2)
        k_r = _heads(dqk(k_sv) + k_xa @ Bt["k"], kv_heads)
        k_r = _repeat(_rope(k_r.transpose(1, 2), cos, sin).transpose(1, 2), n_rep)
    if flash:
        g_q, g_k, g_v = _flash_backward(g_o, q_r, k_r, v_r, _heads(o_r, heads), lse, 1.0 / math.sqrt(hd))
        g_k, g_v = _repeat_bwd(g_k, n_rep), _repeat_bwd(g_v, n_rep)
    else:
        a_r = O.softmax_restore(a_idx, a_val, a_shape)
        g_v = a_r.transpose(-2, -1) @ g_o
        g_a = g_o @ v_r.transpose(-2, -1)
        g_v = _repeat_bwd(g_v, n_rep)
        g_s = O.softmax_bwd(a_r, g_a) / math.sqrt(hd)
        g_k = _repeat_bwd(g_s.transpose(-2, -1) @ q_r, n_rep)
        g_q = g_s @ k_r
    g_q = _rope(g_q.transpose(1, 2), cos, sin, -1.0).transpose(1, 2)
    g_k = _rope(g_k.transpose(1, 2), cos, sin, -1.0).transpose(1, 2)
    g_q, g_k, g_v = _hidden(g_q), _hidden(g_k), _hidden(g_v)
    xn1_r = dq(xn1_sv)
    G[("q", "A")], G[("q", "B")], gx = lora_bwd("q", xn1_r, q_xa, g_q)
    G[("k", "A")], G[("k", "B")], gt = lora_bwd("k", xn1_r, k_xa, g_k)
    gx = gx + gt
    G[("v", "A")], G[("v", "B")], gt = lora_bwd("v", xn1_r, v_xa, g_v)
    gx = gx + gt
    x_r = O.decompress_channel_base(x_sv[1], x_sv[3], x_sv[0], x_sv[2], q_bit)
    g_norm1, G["nw1"] = O.rmsnorm_bwd(gx, x_r, nw1, rstd1)
    G["x"] = g_norm1 + g_medium
    return x_out, G


def roberta_layer_forward_backward(x, weights, ln1, ln2, mask, heads, grad_out, *, mode, q_bit, softmax_ratio,
                                   layernorm_ratio, eps=1e-5):
    """Encoder (post-LayerNorm, GELU) layer: models/roberta/fused_roberta_layer_intra_inter.py:86-200
    (forward), :362-455 (backward) and fused_roberta_layer_intra.py:86-205, :373-440.
    weights: name -> (W [out,in], bias [out] or None, A [r,in], B [out,r]) for q,k,v,o,up,down;
    ln1 / ln2: (weight, bias).  Returns (x_out, grads) like layer_forward_backward."""
    hd = x.shape[-1] // heads
    Wt = {n: w[0].t() for n, w in weights.items()}
    bias = {n: w[1] for n, w in weights.items()}
    At = {n: w[2].t() for n, w in weights.items()}
    Bt = {n: w[3].t() for n, w in weights.items()}

    def lora_fwd(n, inp):
        main = inp @ Wt[n]
        if bias[n] is not None:
            main = main + bias[n]
        xa = inp @ At[n]
        return main + xa @ Bt[n], main, xa

    def lora_bwd(n, inp, xa, gy):
        gmid = gy @ Bt[n].mT
        ga = inp.mT @ gmid
        gb = xa.mT @ gy
        gx = gy @ Wt[n].T
        gx = gx + gmid @ At[n].T
        return ga, gb, gx

    def cq(t):
        s = O.scale_only_quant(t, q_bit)
        return O.compress(t, s, q_bit), s

    def ccb(t):
        idx, s = O.channel_stats(t, layernorm_ratio, q_bit)
        xo, q = O.compress_channel_base(t, s, idx, q_bit)
        return xo, q, idx, s

    dq = lambda sv, **kw: O.decompress(sv[0], sv[1], q_bit, **kw).to(x.device)

    # ------------------------------ forward ------------------------------
    q, q_main, q_xa = lora_fwd("q", x)
    k, k_main, k_xa = lora_fwd("k", x)
    v, v_main, v_xa = lora_fwd("v", x)
    x_sv = cq(x)
    if mode == "intra_inter":
        q_sv, k_sv, v_sv = cq(q_main), cq(k_main), cq(v_main)
    q, k, v = _heads(q, heads), _heads(k, heads), _heads(v, heads)
    if mode == "intra":
        q_sv, k_sv = cq(q), cq(k)
    a = O.softmax_fwd(q @ k.transpose(-2, -1), 1.0 / math.sqrt(hd), mask)
    o = a @ v
    thr = O.softmax_threshold(a, softmax_ratio)
    a_idx, a_val = O.softmax_compress(a, thr)
    a_shape = a.shape
    if mode == "intra":
        v_sv = cq(v)
    o = _hidden(o)
    o_final, _, o_xa = lora_fwd("o", o)
    o_sv = cq(o)
    o_final = o_final + x
    x_medium, mean1, rstd1 = O.layernorm_fwd(o_final, ln1[0], ln1[1], eps)
    of_sv = ccb(o_final)
    up, up_main, up_xa = lora_fwd("up", x_medium)
    xm_sv = cq(x_medium)
    if mode == "intra_inter":
        up_sv = cq(up_main)
    fn = F.gelu(up)
    if mode == "intra":
        up_sv = cq(up)
    down, _, down_xa = lora_fwd("down", fn)
    down = down + x_medium
    if mode == "intra":
        fn_sv = cq(fn)
    x_out, mean2, rstd2 = O.layernorm_fwd(down, ln2[0], ln2[1], eps)
    down_sv = ccb(down)

    # ------------------------------ backward ------------------------------
    G = {}
    go = grad_out
    down_r = O.decompress_channel_base(down_sv[1], down_sv[3], down_sv[0], down_sv[2], q_bit)
    g_ln2 = O.layernorm_bwd(go, down_r, ln2[0], mean2, rstd2)
    if mode == "intra":
        fn_r, up_r = dq(fn_sv), dq(up_sv)
    else:
        up_r = dq(up_sv) + up_xa @ Bt["up"]
        fn_r = F.gelu(up_r)
    G[("down", "A")], G[("down", "B")], g_down = lora_bwd("down", fn_r, down_xa, g_ln2)
    g_fn = O.gelu_bwd(up_r, g_down)
    G[("up", "A")], G[("up", "B")], g_up = lora_bwd("up", dq(xm_sv), up_xa, g_fn)
    g_medium = g_ln2 + g_up
    of_r = O.decompress_channel_base(of_sv[1], of_sv[3], of_sv[0], of_sv[2], q_bit)
    g_ln1 = O.layernorm_bwd(g_medium, of_r, ln1[0], mean1, rstd1)
    G[("o", "A")], G[("o", "B")], g_o = lora_bwd("o", dq(o_sv), o_xa, g_ln1)
    g_o = _heads(g_o, heads)
    a_r = O.softmax_restore(a_idx, a_val, a_shape)
    if mode == "intra":
        v_r = dq(v_sv, is_head=True, num_heads=heads)
        q_r, k_r = dq(q_sv, is_head=True, num_heads=heads), dq(k_sv, is_head=True, num_heads=heads)
    else:
        v_r = _heads(dq(v_sv) + v_xa @ Bt["v"], heads)
        q_r = _heads(dq(q_sv) + q_xa @ Bt["q"], heads)
        k_r = _heads(dq(k_sv) + k_xa @ Bt["k"], heads)
    g_v = a_r.transpose(-2, -1) @ g_o
    g_a = g_o @ v_r.transpose(-2, -1)
    g_s = O.softmax_bwd(a_r, g_a) / math.sqrt(hd)
    g_k = g_s.transpose(-2, -1) @ q_r
    g_q = g_s @ k_r
    g_q, g_k, g_v = _hidden(g_q), _hidden(g_k), _hidden(g_v)
    x_r = dq(x_sv)
    G[("q", "A")], G[("q", "B")], gx = lora_bwd("q", x_r, q_xa, g_q)
    G[("k", "A")], G[("k", "B")], gt = lora_bwd("k", x_r, k_xa, g_k)
    gx = gx + gt
    G[("v", "A")], G[("v", "B")], gt = lora_bwd("v", x_r, v_xa, g_v)
    gx = gx + gt
    G["x"] = gx + g_ln1
    return x_out, G
