"""RoBERTa encoder layers (post-LayerNorm, GELU MLP) with compressed saved activations; class names,
argument order and calibration behaviour of the reference
(models/roberta/fused_roberta_layer_{baseline,intra,intra_inter}.py).

One autograd.Function serves the layer types:
  baseline     keeps the tensors 'intra' keeps, uncompressed, and gathers no statistics
               (…baseline.py: the reference's default layer type);
  intra        keeps the quantised tensors the backward needs as they are (q, k, v in head shape after
               the LoRA add, up, gelu(up));
  intra_inter  keeps only the frozen-weight parts of q, k, v, up and rebuilds the rest in backward
               from the saved LoRA-A products (…intra_inter.py:90-121, :367-371, :411-423).
"""
import math

import torch

from ...operators.compress_function import (compress_attention_map, compression_pack_channel_base,
                                           compression_pack_quant_base, decompression_dequantization,
                                           get_statistics_only_quant, get_statistics_softmax,
                                           outlier_addition_fuse_decompression_dequantization, update_dict,
                                           validate_channel_list)
from ...operators.gelu_kernels import gelu_backward
from ...operators.layernorm_kernels import layernorm_backward, layernorm_forward
from ...operators.softmax_kernels import softmax_backward, softmax_backward_from_compressed, softmax_forward
from ...operators import lora_kernels
from ..compute_utils import (head_to_hidden_shape, heads_matmul, hidden_to_head_shape, lora_backward, lora_forward, lora_input_sum,
                            lora_parts)
from ..fused_decoder_layer import _note_map_entries, lora_linear_parts

MODES = ("baseline", "intra", "intra_inter")
_PROJ = ("q", "k", "v", "o", "up", "down")
_EPS = 1e-5


def stat_slots(mode):
    """(static_value key, field) of every calibration statistic the layer returns, in the reference's
    order (…intra_inter.py:277-282; the intra file adds gelu(up), :296)."""
    if mode == "baseline":
        return []
    slots = [("x", "scale"), ("q", "scale"), ("k", "scale"), ("v", "scale"), ("a", "outlier"), ("o", "scale"),
             ("o_final", "outlier_channel_index"), ("o_final", "scale"), ("x_medium", "scale"), ("up", "scale")]
    if mode == "intra":
        slots.append(("fn", "scale"))
    return slots + [("down", "outlier_channel_index"), ("down", "scale")]


def _weight_of(lora_linear):
    inner = getattr(lora_linear, "default", lora_linear)       # peft wraps adapters in a ModuleDict
    return inner.weight


class FusedRobertaLayerFunc(torch.autograd.Function):
    """Inputs follow the reference's Func.apply order (…intra_inter.py:26-85) with the mode appended."""

    @staticmethod
    def forward(ctx, x,
                w_q, b_q, qs_q, a_q, bb_q, w_k, b_k, qs_k, a_k, bb_k, w_v, b_v, qs_v, a_v, bb_v,
                w_o, b_o, qs_o, a_o, bb_o, norm_weight_1, norm_bias_1,
                w_up, b_up, qs_up, a_up, bb_up, w_down, b_down, qs_down, a_down, bb_down,
                norm_weight_2, norm_bias_2, attention_mask, num_heads, head_dim,
                iteration, iteration_threshold, static_value, softmax_outlier_ratio, layernorm_outlier_ratio,
                q_bit, mode, host_state=None):
        if mode not in MODES:
            raise ValueError(f"layer_type must be one of {MODES}, got {mode!r}")
        W = dict(q=(w_q, b_q, qs_q, a_q, bb_q), k=(w_k, b_k, qs_k, a_k, bb_k), v=(w_v, b_v, qs_v, a_v, bb_v),
                 o=(w_o, b_o, qs_o, a_o, bb_o), up=(w_up, b_up, qs_up, a_up, bb_up),
                 down=(w_down, b_down, qs_down, a_down, bb_down))
        it, thd, sv = iteration, iteration_threshold, static_value
        calib = it < thd
        saved, stats = {}, {}
        raw = mode == "baseline"
        whole = mode in ("baseline", "intra")

        def proj(name, inp, residual=None):
            w, b, qs, la, lb = W[name]
            return lora_forward(w, qs, la, lb, b, inp, residual=residual)

        def proj_quant(name, inp):
            """Projection with the frozen part quantised on the way, one kernel for codes + LoRA add
            (the reference: separate passes, …intra_inter.py:90-121) -> (output, x @ A)."""
            w, b, qs, la, lb = W[name]
            main, xa = lora_parts(w, qs, la, b, inp)
            lb = lb.to(main.dtype)
            if not (lora_kernels.supported(main, xa, lb) and main.dim() == 3):
                quant(name + "_main", main, name)
                return main + xa @ lb, xa
            s_ = get_statistics_only_quant(main, q_bit, 'per-channel') if calib else sv[name]['scale']
            stats[(name, "scale")] = saved[name + "_main_s"] = s_
            saved[name + "_main_q"], y = lora_kernels.lora_add_quant(main, xa, lb, s_, None, q_bit, inplace=True)
            return y, xa

        def quant(name, t, key=None):
            if raw:
                saved[name + "_raw"] = t
                return
            q, s = compression_pack_quant_base(t, q_bit, 'per-channel', it, thd, sv[key or name])
            stats[(key or name, "scale")] = s
            saved[name + "_q"], saved[name + "_s"] = q, s

        def channel_base(name, t):
            if raw:
                saved[name + "_raw"] = t
                return
            o, q, idx, s = compression_pack_channel_base(t, layernorm_outlier_ratio, q_bit, 'per-channel', it, thd,
                                                         sv[name])
            stats[(name, "outlier_channel_index")], stats[(name, "scale")] = idx, s
            saved[name + "_o"], saved[name + "_q"], saved[name + "_s"], saved[name + "_idx"] = o, q, s, idx

        # ---- attention block -------------------------------------------------------------------
        if whole:
            q, _, saved["q_lora_a"] = proj("q", x)
            k, _, saved["k_lora_a"] = proj("k", x)
            v, _, saved["v_lora_a"] = proj("v", x)
        else:
            q, saved["q_lora_a"] = proj_quant("q", x)
            k, saved["k_lora_a"] = proj_quant("k", x)
            v, saved["v_lora_a"] = proj_quant("v", x)
        quant("x", x)
        q, k, v = (hidden_to_head_shape(t, num_heads) for t in (q, k, v))
        if whole:
            quant("q", q)
            quant("k", k)
        s = heads_matmul(q, k.transpose(-2, -1))
        del q, k
        m = attention_mask
        fits = m is None or (m.dim() == 4 and m.shape[1] == 1 and m.shape[0] in (1, s.shape[0]) and
                             m.shape[-1] == s.shape[-1] and m.shape[2] in (1, s.shape[2]))
        if s.dtype == torch.bfloat16 and s.shape[-1] % 8 == 0 and s.shape[-1] <= 8192 and fits:
            if m is not None and m.shape[2] == 1:                # padding mask [B,1,1,S]: one row for all queries
                m = m.expand(m.shape[0], 1, s.shape[2], s.shape[3])
            seg = None
            if calib or raw:
                a = softmax_forward(s, 1.0 / math.sqrt(head_dim), m, inplace=True)
            else:
                a, seg = softmax_forward(s, 1.0 / math.sqrt(head_dim), m, threshold=sv['a']['outlier'], inplace=True)
        else:
            seg = None
            s = s / math.sqrt(head_dim)
            if attention_mask is not None:
                s = s + attention_mask
            a = torch.softmax(s, dim=-1, dtype=v.dtype)
        del s
        o = heads_matmul(a, v, out_hidden=True)
        map_pending = None
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
                # frozen threshold: lists with room for a little more than the recent steps needed, nothing read
                # back here; whether they fitted is looked at once the o projection has been enqueued
                saved["a_idx"], saved["a_val"], saved["a_seg"], count = compress_attention_map(a, thr, seg, capacity=capacity)
                map_pending = (a, thr, count, capacity)
        del a
        if whole:
            quant("v", v)
        del v
        o = head_to_hidden_shape(o)
        o_final, _, saved["o_lora_a"] = proj("o", o, residual=x)        # o_proj(o) + x in the projection's add pass
        quant("o", o)
        del o
        if map_pending is not None:
            a, thr, count, capacity = map_pending
            nnz = count.value()                   # waits for the compaction only, enqueued before the projection
            if nnz > capacity:                    # did not fit: write the lists again at their exact size
                saved["a_idx"], saved["a_val"], saved["a_seg"] = compress_attention_map(a, thr, saved["a_seg"])
            _note_map_entries(host_state, nnz)
            del a, map_pending

        # ---- first LayerNorm (post-norm: on the residual sum) ----------------------------------
        x_medium, saved["mean_1"], saved["rstd_1"], _, _ = layernorm_forward(o_final, norm_weight_1, norm_bias_1, _EPS)
        channel_base("o_final", o_final)
        del o_final

        # ---- MLP block ---------------------------------------------------------------------------
        if whole:
            up, _, saved["up_lora_a"] = proj("up", x_medium)
        else:
            up, saved["up_lora_a"] = proj_quant("up", x_medium)
        quant("x_medium", x_medium)
        fn = torch.nn.functional.gelu(up)
        if whole:
            quant("up", up)
        del up
        down, _, saved["down_lora_a"] = proj("down", fn, residual=x_medium)
        if whole:
            quant("fn", fn)
        del fn, x_medium
        x_out, saved["mean_2"], saved["rstd_2"], block_size, num_warps = layernorm_forward(down, norm_weight_2, norm_bias_2, _EPS)
        channel_base("down", down)
        del down

        ctx.names = list(saved.keys())
        ctx.save_for_backward(*saved.values(), norm_weight_1, norm_bias_1, norm_weight_2, norm_bias_2,
                              *(t for n in _PROJ for t in (W[n][0], W[n][3], W[n][4])))
        ctx.quant_states = {n: W[n][2] for n in _PROJ}
        ctx.mode, ctx.q_bit, ctx.num_heads, ctx.head_dim = mode, q_bit, num_heads, head_dim
        ctx.block_size, ctx.num_warps = block_size, num_warps
        out_stats = tuple(stats[slot] for slot in stat_slots(mode))
        ctx.mark_non_differentiable(*[t for t in out_stats if torch.is_tensor(t)])
        ctx.set_materialize_grads(False)         # no zero-filled gradients for the statistics outputs
        return (x_out,) + out_stats

    @staticmethod
    def backward(ctx, grad_output, *_unused):
        mode, q_bit, H, D = ctx.mode, ctx.q_bit, ctx.num_heads, ctx.head_dim
        tensors = list(ctx.saved_tensors)
        ns = len(ctx.names)
        S = dict(zip(ctx.names, tensors[:ns]))
        nw1, nb1, nw2, nb2 = tensors[ns:ns + 4]
        rest = tensors[ns + 4:]
        W = {n: (rest[3 * i], ctx.quant_states[n], rest[3 * i + 1], rest[3 * i + 2]) for i, n in enumerate(_PROJ)}
        G = {}

        def deq(name, **kw):
            if name + "_raw" in S:
                return S[name + "_raw"]
            return decompression_dequantization(S[name + "_q"], S[name + "_s"], q_bit, **kw)

        def deq_cb(name):
            if name + "_raw" in S:
                return S[name + "_raw"]
            return outlier_addition_fuse_decompression_dequantization(S[name + "_q"], S[name + "_s"], S[name + "_o"],
                                                                      S[name + "_idx"], q_bit)

        def back(name, inp, inp_lora_a, grad_y, accumulate=None, defer_input=False):
            """Backward of projection `name`; `inp` is its input or the name the layer saved it under
            (a compressed input is then read from its codes, not dequantised)."""
            w, qs, la, lb = W[name]
            codes = None
            if isinstance(inp, str):
                if inp + "_raw" in S:
                    inp = S[inp + "_raw"]
                else:
                    codes, inp = (S[inp + "_q"], S[inp + "_s"], None, q_bit), None
            G[name + "_a"], G[name + "_b"], gx = lora_backward(w, qs, la, lb, inp, inp_lora_a, grad_y, x_codes=codes,
                                                                 accumulate=accumulate, defer_input=defer_input)
            return gx

        def rebuilt(name):
            xa, lb = S[name + "_lora_a"], W[name][3]
            lb = lb.to(xa.dtype)
            if lora_kernels.supported_restore(S[name + "_main_q"], xa, lb):
                return lora_kernels.lora_add_restore(S[name + "_main_q"], S[name + "_main_s"], xa, lb, None, q_bit)
            main = deq(name + "_main")
            return main + xa.to(main.dtype) @ lb.to(main.dtype)

        if grad_output is None:
            return (None,) * 45
        grad_output = grad_output.to(torch.bfloat16)
        grad_ln2, _, _ = layernorm_backward(grad_output, deq_cb("down"), nw2, nb2, S["mean_2"], S["rstd_2"], True, _EPS,
                                            ctx.num_warps, ctx.block_size)
        whole = mode in ("baseline", "intra")
        if whole:
            fn, up = deq("fn"), deq("up")
        else:
            up = rebuilt("up")
            fn = torch.nn.functional.gelu(up)
        grad_down = back("down", fn, S["down_lora_a"], grad_ln2)
        del fn
        grad_fn = gelu_backward(up, grad_down)
        del up, grad_down
        grad_up = back("up", "x_medium", S["up_lora_a"], grad_fn)
        grad_medium = grad_ln2 + grad_up
        del grad_ln2, grad_up, grad_fn
        grad_ln1, _, _ = layernorm_backward(grad_medium, deq_cb("o_final"), nw1, nb1, S["mean_1"], S["rstd_1"], True, _EPS,
                                            ctx.num_warps, ctx.block_size)
        del grad_medium
        grad_o = hidden_to_head_shape(back("o", "o", S["o_lora_a"], grad_ln1), H)

        if whole:
            v = deq("v", is_head=True, num_heads=H)
        else:
            v = hidden_to_head_shape(rebuilt("v"), H)
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
        if whole:
            q, k = deq("q", is_head=True, num_heads=H), deq("k", is_head=True, num_heads=H)
        else:
            q, k = hidden_to_head_shape(rebuilt("q"), H), hidden_to_head_shape(rebuilt("k"), H)
        grad_k = heads_matmul(grad_s.transpose(-2, -1), q, out_hidden=True)
        grad_q = heads_matmul(grad_s, k, out_hidden=True)
        del grad_s, q, k
        grad_q, grad_k, grad_v = (head_to_hidden_shape(t) for t in (grad_q, grad_k, grad_v))

        # q, k and v share their input: their input gradients are added up in one pass
        grad_x = lora_input_sum([back("q", "x", S["q_lora_a"], grad_q, defer_input=True),
                                 back("k", "x", S["k_lora_a"], grad_k, defer_input=True),
                                 back("v", "x", S["v_lora_a"], grad_v, defer_input=True)])
        grad_input = grad_x + grad_ln1

        def five(n):
            return (None, None, None, G[n + "_a"], G[n + "_b"])
        return (grad_input, *five("q"), *five("k"), *five("v"), *five("o"), None, None,
                *five("up"), *five("down"), None, None) + (None,) * 11


class _FusedRobertaLayerBase(torch.nn.Module):
    """Module wrapper: owns the calibration state and feeds the Function.  Same call signature as the
    reference's modules (…intra_inter.py:538-568); the state travels with state_dict()."""

    layer_type = "intra_inter"

    def __init__(self):
        super().__init__()
        self.iteration = 0
        self.static_value = self._empty()
        # host-side bookkeeping outside the calibration state (not checkpointed): recent kept-entry counts of
        # the attention map, from which the next step's lists are sized without reading the count back first
        self.host_state = {}
        self.use_hyclora = False

    def _empty(self):
        sv = {}
        for key, field in stat_slots(self.layer_type):
            sv.setdefault(key, {})[field] = None
        return sv

    def set_hyclora_config(self, hyclora_config):
        self.hyclora_config = hyclora_config
        self.use_hyclora = hyclora_config.use_hyclora
        # the uncompressed layer reads none of the compression settings (…baseline.py keeps only
        # use_hyclora and the config itself)
        self.iteration_threshold = getattr(hyclora_config, "iteration_threshold", 0)
        self.softmax_outlier_ratio = getattr(hyclora_config, "softmax_outlier_ratio", 0.0)
        self.layernorm_outlier_ratio = getattr(hyclora_config, "layernorm_outlier_ratio", 0.0)
        self.q_bit = getattr(hyclora_config, "q_bit", 0)

    def get_extra_state(self):
        return {"iteration": int(self.iteration),
                "static_value": {key: {f: (v.detach().clone() if torch.is_tensor(v) else v) for f, v in fields.items()}
                                 for key, fields in self.static_value.items()}}

    def set_extra_state(self, state):
        if not state:
            return
        want, got = self._empty(), state["static_value"]
        if set(got) != set(want) or any(set(got[k]) != set(want[k]) for k in want):
            raise ValueError(f"calibration state of another layer type: has {sorted(got)}, needs {sorted(want)}")
        for fields in got.values():
            channel, scale = fields.get("outlier_channel_index"), fields.get("scale")
            if torch.is_tensor(channel) and torch.is_tensor(scale):
                validate_channel_list(channel, scale.numel())
        self.iteration = int(state["iteration"])
        self.static_value = {key: {f: (v.detach().clone() if torch.is_tensor(v) else v) for f, v in fields.items()}
                             for key, fields in got.items()}

    def _apply(self, fn, *args, **kwargs):
        super()._apply(fn, *args, **kwargs)
        for fields in self.static_value.values():
            for f, v in fields.items():
                if torch.is_tensor(v):
                    fields[f] = fn(v).to(v.dtype)
        return self

    def forward(self, input,
                q_proj_base, q_proj_lora_a, q_proj_lora_b, k_proj_base, k_proj_lora_a, k_proj_lora_b,
                v_proj_base, v_proj_lora_a, v_proj_lora_b, o_proj_base, o_proj_lora_a, o_proj_lora_b,
                norm_weight_1, norm_bias_1,
                up_proj_base, up_proj_lora_a, up_proj_lora_b, down_proj_base, down_proj_lora_a, down_proj_lora_b,
                norm_weight_2, norm_bias_2, attention_mask, num_heads, head_dim):
        def five(base, la, lb):
            w = base.weight
            return (w, getattr(base, "bias", None), getattr(w, "quant_state", None), _weight_of(la).T, _weight_of(lb).T)

        outs = FusedRobertaLayerFunc.apply(
            input, *five(q_proj_base, q_proj_lora_a, q_proj_lora_b), *five(k_proj_base, k_proj_lora_a, k_proj_lora_b),
            *five(v_proj_base, v_proj_lora_a, v_proj_lora_b), *five(o_proj_base, o_proj_lora_a, o_proj_lora_b),
            norm_weight_1, norm_bias_1,
            *five(up_proj_base, up_proj_lora_a, up_proj_lora_b), *five(down_proj_base, down_proj_lora_a, down_proj_lora_b),
            norm_weight_2, norm_bias_2, attention_mask, num_heads, head_dim,
            self.iteration, self.iteration_threshold, self.static_value,
            self.softmax_outlier_ratio, self.layernorm_outlier_ratio, self.q_bit, self.layer_type, self.host_state)
        y, stat_values = outs[0], outs[1:]
        if self.iteration < self.iteration_threshold:
            fresh = {}
            for (key, field), value in zip(stat_slots(self.layer_type), stat_values):
                fresh.setdefault(key, {})[field] = value
            for key, fields in fresh.items():
                self.static_value[key] = update_dict(self.static_value[key], fields, self.iteration)
        self.iteration += 1
        return y


class FusedRobertaLayer(_FusedRobertaLayerBase):
    """The uncompressed layer; the reference gives it the bare name (fused_roberta_layer_baseline.py)."""
    layer_type = "baseline"


FusedRobertaLayerBaseline = FusedRobertaLayer


class FusedRobertaLayerIntra(_FusedRobertaLayerBase):
    layer_type = "intra"


class FusedRobertaLayerIntraInter(_FusedRobertaLayerBase):
    layer_type = "intra_inter"


LAYER_TYPES = {"baseline": FusedRobertaLayer, "intra": FusedRobertaLayerIntra,
               "intra_inter": FusedRobertaLayerIntraInter}


def make_fused_roberta_layer(hyclora_config):
    """Pick the class by `layer_type` and configure it (what the reference's model file does per
    encoder layer)."""
    try:
        layer = LAYER_TYPES[hyclora_config.layer_type]()
    except KeyError:
        raise ValueError(f"Unknown layer type: {hyclora_config.layer_type}") from None
    layer.set_hyclora_config(hyclora_config)
    return layer


def set_fused_roberta_layer(model, hyclora_config):
    """RobertaForSequenceClassification.set_fused_roberta_layer of the reference as a function of the model
    (models/roberta/modeling_roberta.py:982-1009): a configured fused layer per encoder layer in
    `model.roberta.encoder.layer`, as `fused_roberta_layer`."""
    if hyclora_config.layer_type not in LAYER_TYPES:
        raise ValueError(f"Unknown layer type: {hyclora_config.layer_type} (available: {sorted(LAYER_TYPES)})")
    model.hyclora_config = hyclora_config
    for layer in model.roberta.encoder.layer:
        layer.fused_roberta_layer = make_fused_roberta_layer(hyclora_config)


def encoder_layer_forward(encoder_layer, hidden_states, attention_mask):
    """What the reference's encoder layer does in training mode (models/roberta/modeling_roberta.py:428-457): one call
    of the layer's `fused_roberta_layer` with the layer's own weights.  `encoder_layer` is an encoder layer with the
    stock attribute names (`attention.self.{query,key,value}`, `attention.output.{dense,LayerNorm}`,
    `intermediate.dense`, `output.{dense,LayerNorm}`) whose linears are PEFT-style LoRA wrappers
    (`base_layer`, `lora_A`, `lora_B`)."""
    att, out = encoder_layer.attention, encoder_layer.output
    heads = att.self.num_attention_heads

    def parts(linear):
        return lora_linear_parts(linear)
    return encoder_layer.fused_roberta_layer(
        hidden_states, *parts(att.self.query), *parts(att.self.key), *parts(att.self.value), *parts(att.output.dense),
        att.output.LayerNorm.weight, att.output.LayerNorm.bias,
        *parts(encoder_layer.intermediate.dense), *parts(out.dense), out.LayerNorm.weight, out.LayerNorm.bias,
        attention_mask, heads, hidden_states.shape[-1] // heads)
