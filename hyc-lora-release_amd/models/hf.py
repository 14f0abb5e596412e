"""The fused layers inside stock transformers models, without modified model files.

The reference ships its own copies of `modeling_llama.py`, `modeling_mistral.py` and `modeling_roberta.py` whose
decoder / encoder layers call a fused layer while training and fall back to the stock computation otherwise
(models/llama/modeling_llama.py:735-790, :1151-1180).  `install(model, hyclora_config)` does the same to a stock
model object: every layer gets a configured fused layer (`set_fused_*_layer`) and a `forward` that calls it through
`decoder_layer_forward` / `encoder_layer_forward` when `layer.training and fused.use_hyclora`, the layer's own
forward otherwise.  The linears of the layers must be PEFT-style LoRA wrappers (`base_layer`, `lora_A`, `lora_B`)
on all seven (six) projections, with scaling 1."""
import types

import torch

from . import llama, llama_flash_attn, mistral, roberta

_CAUSAL = {}      # (seq_len, device, dtype) -> additive causal mask [1, 1, S, S]


def _causal_mask(seq_len, device, dtype):
    key = (seq_len, device, dtype)
    mask = _CAUSAL.get(key)
    if mask is None:
        if len(_CAUSAL) > 8:
            _CAUSAL.clear()
        mask = _CAUSAL[key] = torch.full((seq_len, seq_len), float("-inf"), device=device).triu(1).to(dtype)[None, None]
    return mask


def _additive(mask, dtype):
    """A boolean attention mask (True = may attend; what transformers hands its layers with the sdpa back end) as the
    additive mask the fused layers take, with the most negative finite value where its eager back end puts it."""
    if mask is None or mask.dtype != torch.bool:
        return mask
    return torch.zeros(mask.shape, dtype=dtype, device=mask.device).masked_fill_(~mask, torch.finfo(dtype).min)


def install(model, hyclora_config, map_free=False):
    """Attach fused layers to `model` (a stock Llama, Mistral or RoBERTa model of transformers, chosen by
    `model.config.model_type`) and route its layers through them in training mode.  `map_free=True` takes the
    long-sequence Llama layers, which save no attention map (reference: models/llama_flash_attn).  Returns the model."""
    kind = getattr(model.config, "model_type", None)
    if kind == "roberta":
        roberta.set_fused_roberta_layer(model, hyclora_config)
        for layer in model.roberta.encoder.layer:
            _route_encoder_layer(layer)
        return model
    if kind == "llama":
        pkg, attr = (llama_flash_attn if map_free else llama), "fused_llama_layer"
        pkg.set_fused_llama_layer(model, hyclora_config)
    elif kind == "mistral" and not map_free:
        pkg, attr = mistral, "fused_mistral_layer"
        pkg.set_fused_mistral_layer(model, hyclora_config)
    else:
        raise ValueError(f"no fused layers for model type {kind!r}" + (" without an attention map" if map_free else ""))
    for layer in model.model.layers:
        _route_decoder_layer(layer, pkg, attr, map_free)
    return model


def _route_decoder_layer(layer, pkg, attr, map_free):
    stock_forward = layer.forward

    def forward(self, hidden_states, attention_mask=None, *args, position_embeddings=None, **kwargs):
        fused = getattr(self, attr)
        if not (self.training and fused.use_hyclora):
            return stock_forward(hidden_states, attention_mask, *args, position_embeddings=position_embeddings, **kwargs)
        if position_embeddings is None:
            raise RuntimeError("the decoder layer was called without position_embeddings=(cos, sin); "
                               "this transformers version computes the rotary tables elsewhere")
        cos, sin = position_embeddings
        if map_free:
            # the map-free layers take a key-padding mask [B, S] or nothing; a 4-D mask is passed on as it is
            mask = attention_mask
        elif attention_mask is None:              # attention back ends that build the causal mask themselves
            mask = _causal_mask(hidden_states.shape[1], hidden_states.device, hidden_states.dtype)
        else:
            mask = _additive(attention_mask, hidden_states.dtype)
        return pkg.decoder_layer_forward(self, hidden_states, mask, cos, sin)
    layer.forward = types.MethodType(forward, layer)


def _route_encoder_layer(layer):
    stock_forward = layer.forward

    def forward(self, hidden_states, attention_mask=None, *args, **kwargs):
        fused = self.fused_roberta_layer
        if not (self.training and fused.use_hyclora):
            return stock_forward(hidden_states, attention_mask, *args, **kwargs)
        return roberta.encoder_layer_forward(self, hidden_states, _additive(attention_mask, hidden_states.dtype))
    layer.forward = types.MethodType(forward, layer)
