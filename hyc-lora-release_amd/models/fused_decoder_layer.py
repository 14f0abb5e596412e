"""A LoRA decoder layer (RMSNorm - attention - RMSNorm - gated MLP) as one autograd.Function that
saves *compressed* activations for backward.

Restates what the reference spreads over twelve near-identical files
(models/{llama,mistral,llama_flash_attn}/fused_*_layer_{baseline,intra,intra_inter,intra_inter_full_fuse}.py)
as one function with three switches:

  mode        'baseline'              nothing is compressed: the same tensors 'intra' saves are kept
                                      as they are and no statistics are gathered - the reference's
                                      default layer type and the uncompressed arm of its memory /
                                      throughput comparison          (fused_llama_layer_baseline.py:147-235)
              'intra'                 every saved activation is quantised as is; q, k (after RoPE) and
                                      v are saved in head shape; silu(gate) and the gated product are
                                      saved too                      (fused_llama_layer_intra.py:95-310)
              'intra_inter'           only the frozen-weight outputs (x@W, "main") are quantised; the
                                      LoRA part is recomputed from the saved x@A in backward
                                                                     (fused_llama_layer_intra_inter.py)
              'intra_inter_full_fuse' as above, with the gate/up quantisation, LoRA add, SiLU and
                                      product in one fused kernel each way
                                                      (fused_llama_layer_intra_inter_full_fuse.py:218-235,359-371)
  attention   'map'   softmax map is materialised, thresholded and saved sparse (:159-176,414-432)
              'sdpa'  no map is saved; the flash kernel's log-sum-exps are, and its backward gets the
                      dequantised attention output; q/k main use a zero point
                      (llama_flash_attn/fused_llama_layer_intra_inter.py:118-180, :450-468 - the
                      flash-attn kernels themselves are replaced by the ones behind torch's
                      scaled_dot_product_attention)
  norm weights receive gradients when they require grad (rmsnorm_updatable_kernels.py:173-220).

Deliberate differences from the reference:
  * the activations handed to the channel-base compressor are not cloned first (the kernels do not
    modify their input);
  * backward restores the input-norm outliers with the *input-norm* channel list; the reference's
    intra_inter / full_fuse files pass the post-attention list there
    (fused_llama_layer_intra_inter_full_fuse.py:484), which its own 'intra' file does not (:492) and
    which is not the gradient of the layer; `reference_outlier_list=True` reproduces that statement;
  * RMSNorm eps is a parameter (default 1e-5, the value the reference hard-codes, :99,203).
"""
from __future__ import annotations

import math
import weakref
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from ..operators.compress_function import (compress_attention_map, compression_pack_channel_base,
                                           compression_pack_quant_base, compression_pack_quant_zp_base,
                                           decompression_dequantization,
                                           decompression_dequantization_with_zero_point,
                                           get_statistics_only_quant, get_statistics_only_quant_zero_point,
                                           get_statistics_softmax,
                                           outlier_addition_fuse_decompression_dequantization,
                                           update_dict, validate_channel_list)
from ..operators.rmsnorm_kernels import _backward as _rmsnorm_backward
from ..operators.rmsnorm_kernels import (backward_from_codes_supported, lora_a_supported, rmsnorm_backward_from_codes, rmsnorm_forward,
                                         rmsnorm_forward_compress)
from ..operators.silu_kernels import silu_backward, silu_hadamard, silu_hadamard_backward, silu_once_hadamard
from ..operators.softmax_kernels import softmax_backward, softmax_backward_from_compressed, softmax_forward
from ..operators.triton_fuse_lora_silu_hadamard_backward_kernels import triton_fuse_silu_backward
from ..operators.triton_fuse_lora_silu_hadamard_forward_kernels import triton_fuse_silu_forward
from ..operators import lora_kernels
from .compute_utils import (head_to_hidden_shape, heads_matmul, hidden_to_head_shape, lora_backward, lora_forward, lora_input_sum, lora_parts,
                            repeat_kv, repeat_kv_backward, rope_backward, rope_forward)

MODES = ("baseline", "intra", "intra_inter", "intra_inter_full_fuse")
# Map-free attention keeps the flash kernel's row log-sum-exps for backward, whose kernel is then
# handed the *dequantised* attention output - the reference's scheme
# (llama_flash_attn/fused_llama_layer_intra_inter.py:450-468).  False recomputes the attention in
# backward instead: one more attention forward per step, gradients free of that output's
# quantisation error (q/k LoRA gradients: cosine 0.99 -> 1.0 against the uncompressed layer at 8
# bits).  Recomputation is also what happens with an explicit mask, or where the flash kernel does not
# take the operands.
KEEP_ATTENTION_LSE = True


@dataclass(frozen=True)
class LayerSpec:
    mode: str = "intra_inter_full_fuse"
    attention: str = "map"          # 'map' | 'sdpa'
    eps: float = 1e-5
    # True: backward puts the input-norm outliers back at the post-attention norm's channels, as the
    # reference's intra_inter / full_fuse files are written (…full_fuse.py:484 passes
    # ctx.post_layernorm_channel); False: at their own channels, as its 'intra' file does (:492)
    reference_outlier_list: bool = False

    def __post_init__(self):
        if self.mode not in MODES:
            raise ValueError(f"layer_type must be one of {MODES}, got {self.mode!r}")
        if self.attention not in ("map", "sdpa"):
            raise ValueError(f"attention must be 'map' or 'sdpa', got {self.attention!r}")

    def stat_slots(self):
        """(static_value key, field) of every calibration statistic the layer returns, in order."""
        if self.mode == "baseline":
            return []
        slots = [("x", "outlier_channel_index"), ("x", "scale"), ("x_norm_1", "scale"),
                 ("q", "scale"), ("k", "scale"), ("v", "scale")]
        if self.attention == "map":
            slots.append(("a", "outlier"))
        else:
            slots += [("q", "zero_point"), ("k", "zero_point")]
        slots += [("o", "scale"), ("x_medium", "outlier_channel_index"), ("x_medium", "scale"),
                  ("x_norm_2", "scale"), ("gate", "scale"), ("up", "scale")]
        if self.mode == "intra":
            slots += [("fn", "scale"), ("hadamard", "scale")]
        return slots

    def empty_static_value(self):
        sv = {}
        for key, field in self.stat_slots():
            sv.setdefault(key, {})[field] = None
        return sv


_PROJ = ("q", "k", "v", "o", "gate", "up", "down")

_ALL_KEPT = {}      # id(mask tensor) -> (weak reference to it, its version, whether every position is kept)


def _nothing_padded(mask2d):
    """Whether a [B, S] key-padding mask keeps every position.  The answer needs one read-back from the
    device; it is kept with the mask tensor (weakly, and only while the tensor is not modified in place),
    because every layer of a model is handed the same mask object in a step."""
    key = id(mask2d)
    hit = _ALL_KEPT.get(key)
    if hit is not None and hit[0]() is mask2d and hit[1] == mask2d._version:
        return hit[2]
    full = bool((mask2d != 0).all().item())
    _ALL_KEPT[key] = (weakref.ref(mask2d, lambda _r, k=key: _ALL_KEPT.pop(k, None)), mask2d._version, full)
    return full


def key_padding_attention_mask(mask2d, dtype):
    """The map-free layers of the reference take a key-padding mask [B, S] (non-zero = a real token) and run
    the varlen flash kernel, causal, on the unpadded tokens; the attention output of padded positions is zero
    (llama_flash_attn/fused_llama_layer_intra_inter.py:160-178).  -> (None, None) when nothing is padded -
    the plain causal kernel is that computation - else (additive mask [B, 1, S, S]: 0 where query i may look
    at key j <= i of a real token or at itself, -inf elsewhere; keep [B, 1, S, 1] in `dtype`, by which the
    attention output is multiplied)."""
    if mask2d.dim() != 2:
        raise ValueError(f"a key-padding mask is [batch, seq], got shape {tuple(mask2d.shape)}")
    if _nothing_padded(mask2d):
        return None, None
    keep = mask2d != 0
    s = keep.shape[1]
    causal = torch.ones(s, s, dtype=torch.bool, device=keep.device).tril()
    allowed = (causal[None] & keep[:, None, :]) | torch.eye(s, dtype=torch.bool, device=keep.device)[None]
    additive = torch.zeros(allowed.shape, dtype=dtype, device=keep.device).masked_fill_(~allowed, float("-inf"))
    return additive[:, None], keep[:, None, :, None].to(dtype)


class FusedDecoderLayerFunc(torch.autograd.Function):
    """Inputs follow the reference's Func.apply order (…full_fuse.py:31-93) with the LayerSpec appended."""

    @staticmethod
    def forward(ctx, x, norm_weight_1, norm_bias_1, cos, sin,
                w_q, b_q, qs_q, a_q, bb_q, w_k, b_k, qs_k, a_k, bb_k,
                w_v, b_v, qs_v, a_v, bb_v, w_o, b_o, qs_o, a_o, bb_o,
                norm_weight_2, norm_bias_2,
                w_gate, b_gate, qs_gate, a_gate, bb_gate, w_up, b_up, qs_up, a_up, bb_up,
                w_down, b_down, qs_down, a_down, bb_down,
                attention_mask, num_heads, head_dim, num_key_value_heads,
                iteration, iteration_threshold, static_value, softmax_outlier_ratio,
                layernorm_outlier_ratio, q_bit, spec, host_state=None):
        W = dict(q=(w_q, b_q, qs_q, a_q, bb_q), k=(w_k, b_k, qs_k, a_k, bb_k), v=(w_v, b_v, qs_v, a_v, bb_v),
                 o=(w_o, b_o, qs_o, a_o, bb_o), gate=(w_gate, b_gate, qs_gate, a_gate, bb_gate),
                 up=(w_up, b_up, qs_up, a_up, bb_up), down=(w_down, b_down, qs_down, a_down, bb_down))
        it, thd, sv = iteration, iteration_threshold, static_value
        calib = it < thd
        n_rep = num_heads // num_key_value_heads
        stats, saved = {}, {}
        raw = spec.mode == "baseline"                   # keep activations as they are
        whole = spec.mode in ("baseline", "intra")      # save whole activations, not the frozen-weight parts

        xa_ready = {}           # projection name -> x @ A formed by the norm kernel that produced x

        def proj(name, inp, residual=None):
            w, b, qs, la, lb = W[name]
            return lora_forward(w, qs, la, lb, b, inp, residual=residual, x_lora_a=xa_ready.pop(name, None))

        def proj_quant_group(names, inp, zp=(), rotate=()):
            """Projections `names` of inp with their frozen parts quantised on the way:
            -> {name: (output, x @ A, whether the output is already rotated)}.  One kernel reads a frozen
            part once, writes its codes, adds the LoRA product and - for the names in `rotate`, with heads of
            128 dims - applies the rotary embedding; the reference quantises `*_main`, adds and rotates in
            separate passes (…full_fuse.py:105-152).  The members that share a kind of code (with / without a
            zero point) go into one launch."""
            out, ready = {}, []
            for name in names:
                w, b, qs, la, lb = W[name]
                main, xa = lora_parts(w, qs, la, b, inp, xa_ready.pop(name, None))
                lb = lb.to(main.dtype)
                with_zp = name in zp
                if not (lora_kernels.supported(main, xa, lb) and main.dim() == 3):
                    (quant_zp if with_zp else quant)(name + "_main", main, name)
                    out[name] = (main + xa @ lb, xa, False)
                    continue
                rope = (cos, sin) if name in rotate and head_dim == lora_kernels.ROPE_HEAD_DIM else None
                if with_zp:
                    s_, z_ = get_statistics_only_quant_zero_point(main, q_bit, 'per-channel') if calib else \
                        (sv[name]['scale'], sv[name]['zero_point'])
                    stats[(name, "zero_point")] = saved[name + "_main_z"] = z_
                else:
                    s_, z_ = get_statistics_only_quant(main, q_bit, 'per-channel') if calib else sv[name]['scale'], None
                stats[(name, "scale")] = saved[name + "_main_s"] = s_
                ready.append((name, dict(x_main=main, xa=xa, b=lb, scale=s_, zero_point=z_, rope=rope)))
            for with_zp in (True, False):
                group = [(n, it) for n, it in ready if (it["zero_point"] is not None) == with_zp]
                for g0 in range(0, len(group), lora_kernels.GROUP_MAX):
                    part = group[g0:g0 + lora_kernels.GROUP_MAX]
                    results = lora_kernels.lora_add_quant_group([it for _, it in part], q_bit, inplace=True)
                    for (n, it), (q_, y_) in zip(part, results):
                        saved[n + "_main_q"] = q_
                        out[n] = (y_, it["xa"], it["rope"] is not None)
            return out

        def quant(name, t, key=None):
            if raw:
                saved[name + "_raw"] = t
                return
            q, s = compression_pack_quant_base(t, q_bit, 'per-channel', it, thd, sv[key or name])
            stats[(key or name, "scale")] = s
            saved[name + "_q"], saved[name + "_s"] = q, s

        def quant_zp(name, t, key):
            if raw:
                saved[name + "_raw"] = t
                return
            q, s, z = compression_pack_quant_zp_base(t, q_bit, 'per-channel', it, thd, sv[key])
            stats[(key, "scale")], stats[(key, "zero_point")] = s, z
            saved[name + "_q"], saved[name + "_s"], saved[name + "_z"] = q, s, z

        def channel_base(name, t):
            if raw:
                saved[name + "_raw"] = t
                return
            o, q, idx, s = compression_pack_channel_base(t, layernorm_outlier_ratio, q_bit, 'per-channel', it, thd,
                                                         sv[name])
            stats[(name, "outlier_channel_index")], stats[(name, "scale")] = idx, s
            saved[name + "_o"], saved[name + "_q"], saved[name + "_s"], saved[name + "_idx"] = o, q, s, idx

        def norm_block(xname, nname, t, w, consumers):
            """RMSNorm of t plus the compressed copies of t (channel base) and of the output.  With
            frozen statistics all three come out of one pass over t; while calibrating the steps of
            the output depend on the output, so the separate operators run (returns done=False and
            the caller quantises the output itself).  Where the kernel takes the shape, the same pass
            also forms `output @ lora_A` for the projections `consumers` that read the output
            (…full_fuse.py:111-117, :218-226 do one GEMM each): calibrating or not, so that both give
            the same bits."""
            n = t.shape[-1]
            adapters = [W[c][3] for c in consumers]
            with_xa = lora_a_supported(t, w, adapters) and all(W[c][0].dtype == torch.bfloat16 or W[c][2] is not None
                                                               for c in consumers)
            if raw or calib or t.dtype != torch.bfloat16 or t.dim() != 3 or n % 32 or n > 8192:
                if with_xa:
                    y, rstd, _, _, _, xas = rmsnorm_forward_compress(t, w, spec.eps, q_bit or 8, lora_a=adapters)
                    xa_ready.update(zip(consumers, xas))
                else:
                    y, _, rstd, _, _ = rmsnorm_forward(t, w, spec.eps)
                channel_base(xname, t)
                return y, rstd, False
            idx, sx, sn = sv[xname]['outlier_channel_index'], sv[xname]['scale'], sv[nname]['scale']
            y, rstd, q_y, q_x, x_out, *xas = rmsnorm_forward_compress(t, w, spec.eps, q_bit, scale_y=sn, scale_x=sx,
                                                                      outlier_idx=idx, lora_a=adapters if with_xa else None)
            if with_xa:
                xa_ready.update(zip(consumers, xas[0]))
            stats[(xname, "outlier_channel_index")], stats[(xname, "scale")], stats[(nname, "scale")] = idx, sx, sn
            saved[xname + "_o"], saved[xname + "_q"], saved[xname + "_s"], saved[xname + "_idx"] = x_out, q_x, sx, idx
            saved[nname + "_q"], saved[nname + "_s"] = q_y, sn
            return y, rstd, True

        # ---- attention block -------------------------------------------------------------------
        x_norm_1, saved["rstd_1"], norm_1_done = norm_block("x", "x_norm_1", x, norm_weight_1, ("q", "k", "v"))
        q_rotated = k_rotated = False
        if whole:
            q, _, saved["q_lora_a"] = proj("q", x_norm_1)
            k, _, saved["k_lora_a"] = proj("k", x_norm_1)
            v, _, saved["v_lora_a"] = proj("v", x_norm_1)
        else:
            qkv = proj_quant_group(("q", "k", "v"), x_norm_1, zp=("q", "k") if spec.attention == "sdpa" else (),
                                   rotate=("q", "k"))
            q, saved["q_lora_a"], q_rotated = qkv["q"]
            k, saved["k_lora_a"], k_rotated = qkv["k"]
            v, saved["v_lora_a"], _ = qkv["v"]
            del qkv
        if not norm_1_done:
            quant("x_norm_1", x_norm_1)
        del x_norm_1

        q = hidden_to_head_shape(q, num_heads)
        k = hidden_to_head_shape(k, num_key_value_heads)
        v = hidden_to_head_shape(v, num_key_value_heads)
        if not q_rotated:
            q = rope_forward(q.transpose(1, 2), cos, sin).transpose(1, 2)
        if not k_rotated:
            k = rope_forward(k.transpose(1, 2), cos, sin).transpose(1, 2)
        k = repeat_kv(k, n_rep)
        v = repeat_kv(v, n_rep)
        if whole:
            (quant_zp if spec.attention == "sdpa" else quant)("q_rope", q, "q")
            (quant_zp if spec.attention == "sdpa" else quant)("k_rope", k, "k")
            quant("v_rep", v, "v")

        map_pending = None
        if spec.attention == "map":
            s = heads_matmul(q, k.transpose(-2, -1))
            del q, k
            # scale, mask and softmax in one pass over the scores, in place; once the threshold is
            # frozen the same pass also counts the entries the compaction keeps
            m = attention_mask
            if m is not None and not (m.dim() == 4 and m.shape[1] == 1 and m.shape[0] in (1, s.shape[0])
                                      and tuple(m.shape[2:]) == tuple(s.shape[2:])):
                m = m.expand(s.shape[0], 1, *s.shape[2:]) if m.dim() == 4 and m.shape[1] == 1 else None
            seg = None
            if s.dtype == torch.bfloat16 and s.shape[-1] % 8 == 0 and s.shape[-1] <= 8192 and \
                    (attention_mask is None or m is not None):
                if calib or raw:
                    a = softmax_forward(s, 1.0 / math.sqrt(head_dim), m, inplace=True)
                else:
                    a, seg = softmax_forward(s, 1.0 / math.sqrt(head_dim), m, threshold=sv['a']['outlier'], inplace=True)
            else:
                s = s / math.sqrt(head_dim)
                if attention_mask is not None:
                    s = s + attention_mask
                a = torch.softmax(s, dim=-1, dtype=v.dtype)
            del s
            if raw:
                saved["a_raw"] = a
            else:
                thr = get_statistics_softmax(a, softmax_outlier_ratio) if calib else sv['a']['outlier']
                stats[("a", "outlier")] = thr
                capacity = None if (calib or host_state is None) else host_state.get("map_capacity")
                if capacity is None:
                    # sizes the lists from nnz read back from the device, as to_sparse() does
                    saved["a_idx"], saved["a_val"], saved["a_seg"] = compress_attention_map(a, thr, seg)
                    if host_state is not None:
                        _note_map_entries(host_state, saved["a_idx"].numel())
                else:
                    # frozen threshold: the lists get room for a little more than the recent steps
                    # needed and nothing is read back here; whether they fitted is looked at after the
                    # o projection has been enqueued (the map is kept until then)
                    saved["a_idx"], saved["a_val"], saved["a_seg"], count = compress_attention_map(a, thr, seg, capacity=capacity)
                    map_pending = (a, thr, count, capacity)
            o = heads_matmul(a, v, out_hidden=True)
            del a, v
        else:
            # causal attention without a map: the flash kernel behind torch's SDPA, called through its
            # aten entry point so that the row log-sum-exps come back and backward needs no second
            # forward (the reference keeps flash-attn's softmax_lse the same way,
            # llama_flash_attn/fused_llama_layer_intra_inter.py:169-180, :459-468)
            ctx.flash = None
            query_keep = ctx.key_padding = None
            if attention_mask is not None and attention_mask.dim() == 2:      # the reference's key-padding mask
                key_padding = attention_mask if attention_mask.device == q.device else attention_mask.to(q.device)
                attention_mask, query_keep = key_padding_attention_mask(key_padding, q.dtype)
                if query_keep is not None:
                    ctx.key_padding = key_padding      # backward builds the [B, 1, S, S] mask again instead of keeping it
            if KEEP_ATTENTION_LSE and attention_mask is None and q.is_cuda:
                try:
                    res = torch.ops.aten._scaled_dot_product_flash_attention(q, k, v, 0.0, True, False)
                    o, saved["sdpa_lse"] = res[0], res[1]
                    saved["sdpa_rng"], saved["sdpa_unused"] = res[6], res[7]
                    ctx.flash = tuple(res[2:6])
                except RuntimeError:
                    ctx.flash = None
            if ctx.flash is None:
                o = F.scaled_dot_product_attention(q, k, v, attn_mask=attention_mask, is_causal=attention_mask is None)
                if query_keep is not None:
                    o = o * query_keep
            del q, k, v
        o = head_to_hidden_shape(o)
        x_medium, _, saved["o_lora_a"] = proj("o", o, residual=x)       # x + o_proj(o) in the projection's add pass
        quant("o", o)
        del o
        if map_pending is not None:
            # The dense map (B*H*S*S bf16, 537 MB at 2 x 32 x 2048^2) is let go before the MLP block allocates
            # its gate / up tensors.  The wait is for the compaction only, which was enqueued before the two
            # attention products and the o projection the device still has to run.
            a, thr, count, capacity = map_pending
            nnz = count.value()
            if nnz > capacity:                    # did not fit: write the lists again at their exact size
                saved["a_idx"], saved["a_val"], saved["a_seg"] = compress_attention_map(a, thr, saved["a_seg"])
            _note_map_entries(host_state, nnz)
            del a, map_pending
            map_pending = None

        # ---- MLP block ---------------------------------------------------------------------------
        x_norm_2, saved["rstd_2"], norm_2_done = norm_block("x_medium", "x_norm_2", x_medium, norm_weight_2, ("gate", "up"))
        if spec.mode == "intra_inter_full_fuse":
            from .compute_utils import dense_weight
            wg, wu = dense_weight(w_gate, qs_gate).t(), dense_weight(w_up, qs_up).t()
            x_norm_2 = x_norm_2.to(wg.dtype)
            gate_main = x_norm_2 @ wg if b_gate is None else x_norm_2 @ wg + b_gate.to(wg.dtype)
            up_main = x_norm_2 @ wu if b_up is None else x_norm_2 @ wu + b_up.to(wu.dtype)
            gate_lora_a = xa_ready.pop("gate", None)
            up_lora_a = xa_ready.pop("up", None)
            if gate_lora_a is None:
                gate_lora_a = x_norm_2 @ a_gate.to(wg.dtype)
            if up_lora_a is None:
                up_lora_a = x_norm_2 @ a_up.to(wu.dtype)
            if calib:
                gate_s = get_statistics_only_quant(gate_main, q_bit, 'per-channel')
                up_s = get_statistics_only_quant(up_main, q_bit, 'per-channel')
            else:
                gate_s, up_s = sv['gate']['scale'], sv['up']['scale']
            stats[("gate", "scale")], stats[("up", "scale")] = gate_s, up_s
            gate_q, up_q, hadamard = triton_fuse_silu_forward(gate_lora_a, bb_gate, gate_main, gate_s,
                                                              up_lora_a, bb_up, up_main, up_s, q_bit)
            saved.update(gate_main_q=gate_q, gate_main_s=gate_s, up_main_q=up_q, up_main_s=up_s)
            del gate_main, up_main
        else:
            if spec.mode == "intra_inter":
                gu = proj_quant_group(("gate", "up"), x_norm_2)
                (gate, gate_lora_a, _), (up, up_lora_a, _) = gu["gate"], gu["up"]
                del gu
                hadamard = silu_hadamard(gate, up)
            else:                                           # 'intra' and 'baseline'
                gate, _, gate_lora_a = proj("gate", x_norm_2)
                up, _, up_lora_a = proj("up", x_norm_2)
                fn = F.silu(gate)
                quant("gate", gate)
                hadamard = up * fn
                quant("up", up)
                quant("fn", fn)
                del fn
            del gate, up
        saved["gate_lora_a"], saved["up_lora_a"] = gate_lora_a, up_lora_a
        if not norm_2_done:
            quant("x_norm_2", x_norm_2)
        del x_norm_2
        x_out, _, saved["down_lora_a"] = proj("down", hadamard, residual=x_medium)
        if whole:
            quant("hadamard", hadamard)
        del hadamard

        ctx.names = list(saved.keys())
        ctx.save_for_backward(*saved.values(), cos, sin, norm_weight_1, norm_weight_2,
                              *(t for n in _PROJ for t in (W[n][0], W[n][1], W[n][3], W[n][4])))
        ctx.quant_states = {n: W[n][2] for n in _PROJ}
        ctx.spec, ctx.q_bit = spec, q_bit
        ctx.num_heads, ctx.num_key_value_heads, ctx.head_dim = num_heads, num_key_value_heads, head_dim
        ctx.has_mask = attention_mask is not None
        ctx.attention_mask = None if spec.attention == "sdpa" and ctx.key_padding is not None else attention_mask
        ctx.norm_grads = (norm_weight_1.requires_grad, norm_weight_2.requires_grad)
        out_stats = tuple(stats[slot] for slot in spec.stat_slots())
        ctx.mark_non_differentiable(*[t for t in out_stats if torch.is_tensor(t)])
        ctx.set_materialize_grads(False)         # no zero-filled gradients for the statistics outputs
        return (x_out,) + out_stats

    @staticmethod
    def backward(ctx, grad_output, *_unused):
        spec, q_bit = ctx.spec, ctx.q_bit
        if grad_output is None:
            return (None,) * 54
        tensors = list(ctx.saved_tensors)
        ns = len(ctx.names)
        S = dict(zip(ctx.names, tensors[:ns]))
        cos, sin, norm_weight_1, norm_weight_2 = tensors[ns:ns + 4]
        rest = tensors[ns + 4:]
        W = {n: (rest[4 * i], rest[4 * i + 1], ctx.quant_states[n], rest[4 * i + 2], rest[4 * i + 3])
             for i, n in enumerate(_PROJ)}
        H, KV, D = ctx.num_heads, ctx.num_key_value_heads, ctx.head_dim
        n_rep = H // KV
        G = {}                                           # LoRA gradients

        def deq(name, **kw):
            if name + "_raw" in S:
                return S[name + "_raw"]
            if name + "_z" in S:
                return decompression_dequantization_with_zero_point(S[name + "_q"], S[name + "_s"], S[name + "_z"],
                                                                    q_bit, **kw)
            return decompression_dequantization(S[name + "_q"], S[name + "_s"], q_bit, **kw)

        def back(name, inp, inp_lora_a, grad_y, accumulate=None, defer_input=False):
            """Backward of projection `name`.  `inp` is its input, or the name under which the layer
            saved that input: a compressed one is then read from its codes, not dequantised.  With
            `defer_input` the input gradient comes back as its terms, for lora_input_sum."""
            w, _, qs, la, lb = W[name]
            codes = None
            if isinstance(inp, str):
                if inp + "_raw" in S:
                    inp = S[inp + "_raw"]
                else:
                    codes, inp = (S[inp + "_q"], S[inp + "_s"], S.get(inp + "_z"), q_bit), None
            ga, gb, gx = lora_backward(w, qs, la, lb, inp, inp_lora_a, grad_y, x_codes=codes, accumulate=accumulate,
                                       defer_input=defer_input)
            G[name] = (ga, gb)
            return gx

        def rebuilt_hidden_group(names, rotate=()):
            """Outputs of projections `names` as forward produced them, from the codes of their frozen parts
            and the saved x @ A: dequantise + LoRA add (+ the rotary embedding for the names in `rotate`, with
            heads of 128 dims) in one kernel, the members with the same kind of code in one launch
            (…full_fuse.py:416-417,439-452).  -> {name: (tensor, rotated or not)}."""
            out, ready = {}, []
            for name in names:
                xa, lb = S[name + "_lora_a"], W[name][4]
                lb = lb.to(xa.dtype)
                q_, s_, z_ = S[name + "_main_q"], S[name + "_main_s"], S.get(name + "_main_z")
                if lora_kernels.supported_restore(q_, xa, lb):
                    rope = (cos, sin) if name in rotate and D == lora_kernels.ROPE_HEAD_DIM else None
                    ready.append((name, dict(q=q_, scale=s_, xa=xa, b=lb, zero_point=z_, rope=rope)))
                else:
                    main = deq(name + "_main")
                    out[name] = (main + (xa @ lb).to(main.dtype), False)
            for with_zp in (True, False):
                group = [(n, it) for n, it in ready if (it["zero_point"] is not None) == with_zp]
                for g0 in range(0, len(group), lora_kernels.GROUP_MAX):
                    part = group[g0:g0 + lora_kernels.GROUP_MAX]
                    results = lora_kernels.lora_add_restore_group([it for _, it in part], q_bit)
                    for (n, it), y_ in zip(part, results):
                        out[n] = (y_, it["rope"] is not None)
            return out

        def channel_base_restored(name, channels):
            if name + "_raw" in S:
                return S[name + "_raw"]
            return outlier_addition_fuse_decompression_dequantization(
                S[name + "_q"], S[name + "_s"], S[name + "_o"], S[channels + "_idx"], q_bit)

        def norm_backward(dy, name, weight, rstd, want_dw, residual, channels=None):
            """Backward of the norm whose input the layer saved under `name`, plus the gradient of the
            residual connection (`grad_norm + residual` in the reference, …full_fuse.py:386-393,486-493).
            A compressed input is read from its codes where the kernel takes the shape; otherwise it
            is restored first.  The residual is added inside the kernel where it can be."""
            channels = channels or name
            fused_add = residual.dtype == dy.dtype == torch.bfloat16 and residual.shape == dy.shape
            if name + "_raw" not in S and fused_add and backward_from_codes_supported(dy, dy.shape[-1], want_dw):
                dx = rmsnorm_backward_from_codes(dy, S[name + "_q"], S[name + "_s"], S[name + "_o"], S[channels + "_idx"],
                                                 q_bit, weight, rstd, residual=residual)
                return dx, None
            xin = channel_base_restored(name, channels)
            if fused_add:
                return _rmsnorm_backward(dy, xin, weight, rstd, want_dw=want_dw, residual=residual)
            dx, dw = _rmsnorm_backward(dy, xin, weight, rstd, want_dw=want_dw)
            return dx + residual, dw

        # ---- MLP block ---------------------------------------------------------------------------
        if spec.mode == "intra_inter_full_fuse":
            from .compute_utils import dense_weight
            w, _, qs, la, lb = W["down"]
            wd = dense_weight(w, qs)
            la, lb = la.to(wd.dtype), lb.to(wd.dtype)
            g = grad_output.to(wd.dtype)
            r = lb.shape[0]
            fast = lora_kernels.contract_supported(g, g.shape[-1], r) and S["down_lora_a"].dtype == g.dtype
            if fast:                      # both rank-R products of grad_output from one pass over it
                grad_b_down, grad_mid = lora_kernels.lora_products(g, u=S["down_lora_a"], v=lb, p1_transposed=True)
                grad_b_down = grad_b_down.t()         # [R, N] view of the [N, R] result, as in lora_backward
            else:
                grad_b_down = S["down_lora_a"].to(wd.dtype).mT @ g
                grad_mid = g @ lb.mT
            grad_down = g @ wd
            if lora_kernels.supported(grad_down, grad_mid, la.mT):
                grad_down = lora_kernels.lora_add(grad_down, grad_mid, la.mT, inplace=True)
            else:
                grad_down += grad_mid @ la.mT
            hadamard, grad_fn, grad_h2 = triton_fuse_silu_backward(
                S["gate_lora_a"], W["gate"][4], S["gate_main_q"], S["gate_main_s"],
                S["up_lora_a"], W["up"][4], S["up_main_q"], S["up_main_s"], grad_down, q_bit)
            if fast and lora_kernels.contract_supported(hadamard, hadamard.shape[-1], r):
                G["down"] = (lora_kernels.lora_products(hadamard, u=grad_mid)[0].t(), grad_b_down)
            else:
                G["down"] = (hadamard.to(wd.dtype).mT @ grad_mid, grad_b_down)
            del hadamard, grad_down
        else:
            fn = None
            if spec.mode == "intra_inter":
                gu = rebuilt_hidden_group(("gate", "up"))
                gate, up = gu["gate"][0], gu["up"][0]
                del gu
                if gate.dtype == up.dtype == torch.bfloat16:
                    hadamard = silu_once_hadamard(gate, up)   # up * F.silu(gate), as the reference recomputes it
                else:
                    hadamard = up * F.silu(gate)
            else:
                hadamard, up, fn, gate = deq("hadamard"), deq("up"), deq("fn"), deq("gate")
            grad_down = back("down", hadamard, S["down_lora_a"], grad_output)
            del hadamard
            if fn is None and grad_down.dtype == gate.dtype == torch.bfloat16:
                # grad_down * up, silu_backward of it, and grad_down * silu(gate): one pass
                grad_fn, grad_h2 = silu_hadamard_backward(gate, up, grad_down)
            else:
                if fn is None:
                    fn = F.silu(gate)
                grad_h1 = grad_down * up
                grad_h2 = grad_down * fn
                grad_fn = silu_backward(gate, grad_h1)
                del grad_h1
            del grad_down, up, fn, gate
        # gate and up share their input: their input gradients are added up in one pass (`grad_x += grad_x_temp`)
        grad_x2 = lora_input_sum([back("gate", "x_norm_2", S["gate_lora_a"], grad_fn, defer_input=True),
                                  back("up", "x_norm_2", S["up_lora_a"], grad_h2, defer_input=True)])
        del grad_fn, grad_h2
        grad_medium, grad_nw2 = norm_backward(grad_x2, "x_medium", norm_weight_2, S["rstd_2"], ctx.norm_grads[1], grad_output)
        del grad_x2

        # ---- attention block -------------------------------------------------------------------
        grad_o = back("o", "o", S["o_lora_a"], grad_medium)
        grad_o = hidden_to_head_shape(grad_o, H)

        if spec.mode in ("baseline", "intra"):
            q, k, v = (deq(n, is_head=True, num_heads=H) for n in ("q_rope", "k_rope", "v_rep"))
        else:
            qkv = rebuilt_hidden_group(("q", "k", "v"), rotate=("q", "k"))

            def rebuilt(name, heads):
                """q/k/v in head shape as the forward attention saw them (before repeat_kv)."""
                t, rotated = qkv[name]
                t = hidden_to_head_shape(t, heads)
                if name != "v" and not rotated:
                    t = rope_forward(t.transpose(1, 2), cos, sin).transpose(1, 2)
                return t
            q, k, v = rebuilt("q", H), repeat_kv(rebuilt("k", KV), n_rep), repeat_kv(rebuilt("v", KV), n_rep)
            del qkv

        if spec.attention == "map":
            # grad_a first, then the restored map and the softmax backward come out of one pass over
            # the compressed map (the reference restores, then reads the dense map twice more)
            grad_a = heads_matmul(grad_o, v.transpose(-2, -1))
            del v
            if "a_raw" in S:
                a = S["a_raw"]
                grad_s = softmax_backward(a, grad_a) / math.sqrt(D)
            else:
                a, grad_s = softmax_backward_from_compressed(S["a_idx"], S["a_val"], S["a_seg"], grad_a,
                                                             out_scale=1.0 / math.sqrt(D))
            del grad_a
            grad_v = heads_matmul(a.transpose(-2, -1), grad_o, out_hidden=True)
            del a, grad_o
            grad_k = heads_matmul(grad_s.transpose(-2, -1), q, out_hidden=True)
            grad_q = heads_matmul(grad_s, k, out_hidden=True)
            del grad_s, q, k
        elif ctx.flash is not None:
            # the attention output handed to the backward kernel is the dequantised one, as in the
            # reference (…intra_inter.py:450-461)
            out = hidden_to_head_shape(deq("o"), H)
            cum_q, cum_k, max_q, max_k = ctx.flash
            grad_q, grad_k, grad_v = torch.ops.aten._scaled_dot_product_flash_attention_backward(
                grad_o, q, k, v, out, S["sdpa_lse"], cum_q, cum_k, max_q, max_k, 0.0, True,
                S["sdpa_rng"], S["sdpa_unused"])
            del q, k, v, out, grad_o
        else:
            with torch.enable_grad():
                q_, k_, v_ = (t.detach().requires_grad_() for t in (q, k, v))
                mask, query_keep = ctx.attention_mask, None
                if ctx.key_padding is not None:
                    mask, query_keep = key_padding_attention_mask(ctx.key_padding, q.dtype)
                o_ = F.scaled_dot_product_attention(q_, k_, v_, attn_mask=mask, is_causal=not ctx.has_mask)
                if query_keep is not None:
                    o_ = o_ * query_keep
                grad_q, grad_k, grad_v = torch.autograd.grad(o_, (q_, k_, v_), grad_o)
            del q, k, v, q_, k_, v_, o_, grad_o
        grad_v = repeat_kv_backward(grad_v, n_rep)
        grad_k = repeat_kv_backward(grad_k, n_rep)
        grad_q = rope_backward(grad_q.transpose(1, 2), cos, sin).transpose(1, 2)
        grad_k = rope_backward(grad_k.transpose(1, 2), cos, sin).transpose(1, 2)
        grad_q, grad_k, grad_v = (head_to_hidden_shape(t) for t in (grad_q, grad_k, grad_v))

        grad_x = lora_input_sum([back("q", "x_norm_1", S["q_lora_a"], grad_q, defer_input=True),
                                 back("k", "x_norm_1", S["k_lora_a"], grad_k, defer_input=True),
                                 back("v", "x_norm_1", S["v_lora_a"], grad_v, defer_input=True)])
        del grad_q, grad_k, grad_v
        as_reference = spec.reference_outlier_list and spec.mode in ("intra_inter", "intra_inter_full_fuse")
        grad_input, grad_nw1 = norm_backward(grad_x, "x", norm_weight_1, S["rstd_1"], ctx.norm_grads[0], grad_medium,
                                             channels="x_medium" if as_reference else "x")

        def lora_grads(name):
            return (None, None, None) + G[name]

        return ((grad_input, grad_nw1, None, None, None)
                + lora_grads("q") + lora_grads("k") + lora_grads("v") + lora_grads("o")
                + (grad_nw2, None)
                + lora_grads("gate") + lora_grads("up") + lora_grads("down")
                + (None,) * 12)


MAP_HISTORY = 8            # steps whose kept-entry counts size the next step's attention-map lists
MAP_HEADROOM = 1.0 / 16    # room beyond the largest of them


def _note_map_entries(host_state, nnz):
    """Records the kept-entry count of a step and sets the capacity of the next step's lists."""
    history = host_state.setdefault("map_history", [])
    history.append(int(nnz))
    del history[:-MAP_HISTORY]
    top = max(history)
    host_state["map_capacity"] = top + int(top * MAP_HEADROOM) + 64


def _weight_of(module):
    """Weight of a LoRA adapter container (`module.default.weight`, PEFT) or of a plain Linear."""
    inner = getattr(module, "default", module)
    return inner.weight


class FusedDecoderLayer(torch.nn.Module):
    """Module wrapper: owns the calibration state (`iteration`, `static_value`) and feeds the
    Function.  Same call signature as the reference's modules (…full_fuse.py:582-614)."""

    layer_type = "intra_inter_full_fuse"
    attention = "map"

    def __init__(self, eps: float = 1e-5, reference_outlier_list: bool = False):
        super().__init__()
        self.spec = LayerSpec(self.layer_type, self.attention, eps, reference_outlier_list)
        self.iteration = 0
        self.static_value = self.spec.empty_static_value()
        # host-side bookkeeping that is not part of the calibration state (not checkpointed): the
        # recent kept-entry counts of the attention map, from which the next step's lists are sized
        # without reading the count back first
        self.host_state = {}
        self.use_hyclora = False

    def set_hyclora_config(self, hyclora_config):
        self.hyclora_config = hyclora_config
        self.use_hyclora = hyclora_config.use_hyclora
        # the uncompressed layer reads none of the compression settings
        # (fused_llama_layer_baseline.py:443-445 keeps only use_hyclora and the config itself)
        self.iteration_threshold = getattr(hyclora_config, "iteration_threshold", 0)
        self.softmax_outlier_ratio = getattr(hyclora_config, "softmax_outlier_ratio", 0.0)
        self.layernorm_outlier_ratio = getattr(hyclora_config, "layernorm_outlier_ratio", 0.0)
        self.q_bit = getattr(hyclora_config, "q_bit", 0)

    # The reference keeps `iteration` and `static_value` as plain attributes (…full_fuse.py:574-580),
    # so a checkpoint taken after calibration restarts calibrating.  Here they travel with
    # state_dict() as the module's extra state: ints, None and tensors only, loadable with
    # torch.load(weights_only=True).
    def get_extra_state(self):
        return {"iteration": int(self.iteration),
                "static_value": {key: {f: (v.detach().clone() if torch.is_tensor(v) else v) for f, v in fields.items()}
                                 for key, fields in self.static_value.items()}}

    def set_extra_state(self, state):
        if not state:
            return
        want = self.spec.empty_static_value()
        got = state["static_value"]
        if set(got) != set(want) or any(set(got[k]) != set(want[k]) for k in want):
            raise ValueError(f"calibration state of another layer type: has {sorted(got)}, "
                             f"{self.spec.mode}/{self.spec.attention} needs {sorted(want)}")
        for key, fields in got.items():
            channel, scale = fields.get("outlier_channel_index"), fields.get("scale")
            if torch.is_tensor(channel) and torch.is_tensor(scale):
                validate_channel_list(channel, scale.numel())
        self.iteration = int(state["iteration"])
        self.static_value = {key: {f: (v.detach().clone() if torch.is_tensor(v) else v) for f, v in fields.items()}
                             for key, fields in got.items()}

    def _apply(self, fn, *args, **kwargs):
        # .to(device)/.cuda() move the statistics with the module; their dtypes are part of the
        # format (bf16 steps, fp32 threshold, int64 channels) and survive .half()/.float()
        super()._apply(fn, *args, **kwargs)
        for fields in self.static_value.values():
            for f, v in fields.items():
                if torch.is_tensor(v):
                    fields[f] = fn(v).to(v.dtype)
        return self

    def forward(self, input, norm_weight_1, norm_bias_1, cos, sin,
                q_proj_base, q_proj_lora_a, q_proj_lora_b, k_proj_base, k_proj_lora_a, k_proj_lora_b,
                v_proj_base, v_proj_lora_a, v_proj_lora_b, o_proj_base, o_proj_lora_a, o_proj_lora_b,
                norm_weight_2, norm_bias_2,
                gate_proj_base, gate_proj_lora_a, gate_proj_lora_b, up_proj_base, up_proj_lora_a, up_proj_lora_b,
                down_proj_base, down_proj_lora_a, down_proj_lora_b,
                attention_mask, num_heads, head_dim, num_key_value_heads=None):
        # the reference's map-free modules are called without num_key_value_heads
        # (llama_flash_attn/modeling_llama.py:620-653): as many key / value heads as query heads
        if num_key_value_heads is None:
            num_key_value_heads = num_heads

        def five(base, la, lb):
            w = base.weight
            return (w, getattr(base, "bias", None), getattr(w, "quant_state", None),
                    _weight_of(la).T, _weight_of(lb).T)

        outs = FusedDecoderLayerFunc.apply(
            input, norm_weight_1, norm_bias_1, cos, sin,
            *five(q_proj_base, q_proj_lora_a, q_proj_lora_b), *five(k_proj_base, k_proj_lora_a, k_proj_lora_b),
            *five(v_proj_base, v_proj_lora_a, v_proj_lora_b), *five(o_proj_base, o_proj_lora_a, o_proj_lora_b),
            norm_weight_2, norm_bias_2,
            *five(gate_proj_base, gate_proj_lora_a, gate_proj_lora_b), *five(up_proj_base, up_proj_lora_a, up_proj_lora_b),
            *five(down_proj_base, down_proj_lora_a, down_proj_lora_b),
            attention_mask, num_heads, head_dim, num_key_value_heads,
            self.iteration, self.iteration_threshold, self.static_value,
            self.softmax_outlier_ratio, self.layernorm_outlier_ratio, self.q_bit, self.spec, self.host_state)
        y, stat_values = outs[0], outs[1:]
        if self.iteration < self.iteration_threshold:
            fresh = {}
            for (key, field), value in zip(self.spec.stat_slots(), stat_values):
                fresh.setdefault(key, {})[field] = value
            for key, fields in fresh.items():
                self.static_value[key] = update_dict(self.static_value[key], fields, self.iteration)
        self.iteration += 1
        return y


def lora_linear_parts(linear):
    """(base_layer, lora_A, lora_B) of a PEFT-style LoRA linear.  The layers compute `x @ W^T + (x @ A^T) @ B^T`
    without a scaling factor, like the reference, whose scripts refuse lora_alpha != rank (run_gsm8k.py:373-374):
    a wrapper that carries another scaling is refused here."""
    scaling = getattr(linear, "scaling", None)
    values = list(scaling.values()) if isinstance(scaling, dict) else ([] if scaling is None else [scaling])
    if any(float(v) != 1.0 for v in values):
        raise ValueError(f"LoRA scaling {values} is not supported: the fused layers apply none (lora_alpha must equal the rank)")
    return linear.base_layer, linear.lora_A, linear.lora_B


def call_from_decoder_layer(fused_layer, decoder_layer, hidden_states, attention_mask, cos, sin, num_key_value_heads=None):
    """The call the reference's decoder layers make while training (models/llama/modeling_llama.py:745-786,
    models/mistral/modeling_mistral.py:611-646): hands the fused layer the norm weights and, for each of the seven
    projections, the frozen `base_layer` and the `lora_A` / `lora_B` containers of a PEFT-wrapped linear, taken
    from a decoder layer with the stock attribute names (`input_layernorm`, `self_attn.{q,k,v,o}_proj`,
    `post_attention_layernorm`, `mlp.{gate,up,down}_proj`).  Head counts come from the layer's attention config."""
    attn, mlp = decoder_layer.self_attn, decoder_layer.mlp
    cfg = getattr(attn, "config", None)
    num_heads = getattr(attn, "num_heads", None) or getattr(attn, "num_attention_heads", None) or cfg.num_attention_heads
    head_dim = getattr(attn, "head_dim", None) or cfg.hidden_size // num_heads
    if num_key_value_heads is None:
        num_key_value_heads = getattr(attn, "num_key_value_heads", None) or getattr(cfg, "num_key_value_heads", num_heads)

    def parts(linear):
        return lora_linear_parts(linear)
    return fused_layer(hidden_states, decoder_layer.input_layernorm.weight, None, cos, sin,
                       *parts(attn.q_proj), *parts(attn.k_proj), *parts(attn.v_proj), *parts(attn.o_proj),
                       decoder_layer.post_attention_layernorm.weight, None,
                       *parts(mlp.gate_proj), *parts(mlp.up_proj), *parts(mlp.down_proj),
                       attention_mask, num_heads, head_dim, num_key_value_heads)
