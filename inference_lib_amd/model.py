"""The attention layer that talks to HogwildCache, and the swap that puts it into a decoder model: the host-side mirror
of `AttentionModule` / `model_surgery` of the reference (python/hogwild/attention.py:263-354).

The layer projects q/k/v, hands the new keys (un-rotated) and values to the cache, which rotates the keys and appends
them to every worker's segment in one launch, and calls the fused operator with the un-rotated queries: each fragment
gets its own query rotation inside the kernel (attention.py:313-339).  Nothing here imports the model library; the
modules are taken from the model that is operated on (`q_proj`, `k_proj`, `v_proj`, `o_proj` of its attention layers,
`model.model.rotary_emb`), so any decoder with that layout (Qwen2, Llama, Mistral ...) works.

`decode_step` runs the decoder stack on top of such a model without the model library's own mask and cache plumbing
(the reference neutralises that plumbing by overwriting `_update_causal_mask`, attention.py:352-354, a hook newer
versions of the library no longer have): visibility is entirely the cache's business.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import nn

from .attention import hogwild_fused
from .cache import CacheStructure, HogwildCache


class AttentionModule(nn.Module):
    """Attention layer adapted to HogwildCache (attention.py:263-343).  Batch rows are workers."""

    def __init__(self, config, layer_idx: int, *, q_proj: Optional[nn.Module] = None, k_proj: Optional[nn.Module] = None,
                 v_proj: Optional[nn.Module] = None, o_proj: Optional[nn.Module] = None):
        super().__init__()
        self.config = config
        self.layer_idx = layer_idx
        self.head_dim = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
        self.num_key_value_groups = config.num_attention_heads // config.num_key_value_heads
        self.scaling = self.head_dim ** -0.5
        self.is_causal = True
        # attention.py:277-288: biased q/k/v projections, unbiased output projection, unless the caller brings its own
        self.q_proj = q_proj if q_proj is not None else nn.Linear(config.hidden_size, config.num_attention_heads * self.head_dim, bias=True)
        self.k_proj = k_proj if k_proj is not None else nn.Linear(config.hidden_size, config.num_key_value_heads * self.head_dim, bias=True)
        self.v_proj = v_proj if v_proj is not None else nn.Linear(config.hidden_size, config.num_key_value_heads * self.head_dim, bias=True)
        self.o_proj = o_proj if o_proj is not None else nn.Linear(config.num_attention_heads * self.head_dim, config.hidden_size, bias=False)

    def forward(self, hidden_states: torch.Tensor, position_embeddings: Tuple[torch.Tensor, torch.Tensor],
                attention_mask: Optional[torch.Tensor] = None, past_key_values: Optional[HogwildCache] = None,
                cache_position: Optional[torch.Tensor] = None, position_ids: Optional[torch.Tensor] = None,
                past_key_value: Optional[HogwildCache] = None, **kwargs):
        cache = past_key_values if past_key_values is not None else past_key_value      # both spellings of the argument exist
        if not isinstance(cache, HogwildCache):
            raise TypeError("AttentionModule needs a HogwildCache as past_key_values")
        input_shape = hidden_states.shape[:-1]                                          # [W, S]
        hidden_shape = (*input_shape, -1, self.head_dim)
        if input_shape[0] != 1 and position_ids is None:                                 # attention.py:304-305
            raise ValueError("when processing several workers, position_ids are mandatory")
        if position_ids is not None and tuple(position_ids.shape) != tuple(input_shape):
            raise ValueError(f"position_ids {tuple(position_ids.shape)} do not match the input {tuple(input_shape)}")

        query_states = self.q_proj(hidden_states).view(hidden_shape).transpose(1, 2)     # [W, Hq, S, D]
        key_states = self.k_proj(hidden_states).view(hidden_shape).transpose(1, 2)       # [W, Hkv, S, D] (a view: no copy)
        value_states = self.v_proj(hidden_states).view(hidden_shape).transpose(1, 2)

        cos, sin = position_embeddings                                                   # [W, S, RotE] for the new tokens
        # keys: rotation (attention.py:313-315) and append (:148-158) in one launch, with the eager expression's roundings
        cs: CacheStructure = cache.update_fused(key_states, value_states, cos, sin, self.layer_idx, mask=attention_mask)
        # queries are rotated per fragment inside the operator (attention.py:326-339)
        rq = cache.get_queries_buffer(query_states, layer_idx=self.layer_idx)
        attn = hogwild_fused(query_states, cs.loc, cs.keys, cs.values, self.scaling, cs.frags, cs.cos, cs.sin,
                             rotated_queries=rq, out=cache.get_att_buffer(rq, layer_idx=self.layer_idx),
                             device_lengths=cache.device_lengths)
        attn = attn.transpose(1, 2).reshape(*input_shape, -1).contiguous()
        return self.o_proj(attn), None


def model_surgery(model) -> None:
    """Replace the attention layers of `model.model.layers` by AttentionModule, keeping their projections
    (attention.py:345-354)."""
    config = model.model.config if hasattr(model.model, "config") else model.config
    for layer in model.model.layers:
        old = layer.self_attn
        layer.self_attn = AttentionModule(config, old.layer_idx, q_proj=old.q_proj, k_proj=old.k_proj, v_proj=old.v_proj, o_proj=old.o_proj)


@torch.no_grad()
def decode_step(model, cache: HogwildCache, input_ids: torch.Tensor, attention_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One step of a model that went through model_surgery: input_ids [W, S] (row w = the new tokens of worker w, left
    padded where attention_mask [W, S] is 0) -> logits [W, S, vocab].  Position ids are those of
    HogwildCache.get_input_kwargs (positions inside the segment a worker writes to, attention.py:238-246)."""
    kw = cache.get_input_kwargs(input_ids, attention_mask)
    core = model.model
    hidden = core.embed_tokens(input_ids)
    position_ids = kw["position_ids"]
    position_embeddings = core.rotary_emb(hidden, position_ids)
    for layer in core.layers:
        out = layer(hidden, attention_mask=attention_mask, position_ids=position_ids, past_key_values=cache,
                    use_cache=True, position_embeddings=position_embeddings)
        hidden = out[0] if isinstance(out, tuple) else out
    return model.lm_head(core.norm(hidden))
