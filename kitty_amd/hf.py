"""Hook for stock transformers attention modules (Llama, Qwen3, ... on transformers >= 4.48).

The reference ships a modified copy of the Qwen3 modeling file whose attention layer calls
``past_key_values.update(...)``, ``kitty_attention_forward(...)`` and ``quantize_decode`` /
``quantize_prefill`` itself (src/kitty/models/qwen3/modeling_qwen3.py:203-255).  Stock modules
instead call ``past_key_values.update`` and hand whatever it returns to the attention function
selected by ``config._attn_implementation``.  This module provides both halves:

* ``KittyHFCache``: a ``KittyCache`` whose ``update`` does what the reference's does and returns the
  states it was given, as stock modules expect;
* the attention function ``"kitty"``: the reference's sequence for the layer that calls it — dense
  causal attention on the prompt followed by ``quantize_prefill`` (prefill), or packed decode
  attention followed by ``quantize_decode`` (one new token), or chunked-prefill attention followed by
  ``append`` (several new tokens over a non-empty cache: no counterpart in the reference).

    from kitty_amd import hf
    hf.register()
    model = AutoModelForCausalLM.from_pretrained(..., attn_implementation="kitty")
    cache = hf.KittyHFCache(model.config, batch, max_length)
    model.generate(..., past_key_values=cache)

Batches must not be padded (the reference has the same restriction: one set of counters per layer);
the attention mask of the model is ignored in decode and assumed causal in prefill.
"""
from __future__ import annotations

import threading
import types
from typing import Any, Optional

import torch

from .kvcache.kitty import KittyCache
from .kvcache.paging import PagedKittyCache
from .kvcache.kernels import kitty_attention_forward, kitty_prefill_attention

NAME = "kitty"
_current = threading.local()     # the cache whose update() ran last on this thread


class KittyHFCache(KittyCache):
    """``KittyCache`` for stock attention modules: ``update`` returns ``(key_states, value_states)``."""

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[dict[str, Any]] = None):
        layer = self.kv_cache[layer_idx]
        _current.cache = self
        if layer.Sink_Count > 0 and key_states.shape[-2] > 1:
            # a chunk over a cache that holds tokens: attention needs the cache as it was, the
            # attention function appends afterwards
            _current.phase = "chunk"
        else:
            _current.phase = "prefill" if super().update(key_states, value_states, layer_idx, cache_kwargs) else "decode"
        return key_states, value_states

    def get_mask_sizes(self, query_length, layer_idx: int = 0):
        """(kv_length, kv_offset) of the mask a stock model prepares.  Only the prompt's causal mask
        is ever looked at (and only for its shape), so the new tokens alone are reported."""
        n = query_length if isinstance(query_length, int) else int(query_length.shape[0])
        return n, 0


class PagedKittyHFCache(PagedKittyCache):
    """``PagedKittyCache`` for stock attention modules.  A prompt is admitted with a batch-1 forward
    inside ``with cache.admitting(slot):``; decode forwards take all slots as the batch, with
    ``position_ids=cache.position_ids()`` since the sequences differ in length (rows of free
    slots are computed and ignored)."""

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[dict[str, Any]] = None):
        _current.cache = self
        if self._admit_slot is None and key_states.shape[-2] != 1:
            # several new tokens for every slot over what the slots hold: attention needs the cache
            # as it was, the attention function appends afterwards
            _current.phase = "chunk"
        else:
            _current.phase = "prefill" if super().update(key_states, value_states, layer_idx, cache_kwargs) else "decode"
        return key_states, value_states

    def get_seq_length(self, layer_idx: int = 0) -> int:
        """What a stock model derives positions from: 0 while a prompt is being admitted (its
        positions start at 0), else the longest active sequence."""
        return 0 if self._admit_slot is not None else super().get_seq_length(layer_idx)

    def get_mask_sizes(self, query_length, layer_idx: int = 0):
        n = query_length if isinstance(query_length, int) else int(query_length.shape[0])
        return n, 0

    def position_ids(self, n_tokens: int = 1) -> torch.Tensor:
        """[slots, n_tokens] int64 on the cache's device: the positions of each slot's next tokens."""
        first = torch.from_numpy(self.seq_lengths().astype("int64")).view(-1, 1)
        return (first + torch.arange(n_tokens, dtype=torch.int64).view(1, -1)).to(self.seq_counts.device)


def kitty_attention(module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                    attention_mask: Optional[torch.Tensor] = None, dropout: float = 0.0,
                    scaling: Optional[float] = None, **kwargs):
    """Attention function for ``ALL_ATTENTION_FUNCTIONS``: query [B, H_Q, T_q, D], key / value
    [B, H_KV, T_q, D] as returned by ``KittyHFCache.update``; returns ([B, T_q, H_Q, D], None)."""
    cache = getattr(_current, "cache", None)
    if cache is None:
        raise RuntimeError("attn_implementation='kitty' needs a KittyHFCache as past_key_values")
    if dropout:
        raise NotImplementedError("attention dropout is not supported on the packed-KV path")
    layer_idx = module.layer_idx
    layer = cache.kv_cache[layer_idx]
    # the head counts the reference's attention module carries as attributes
    heads = types.SimpleNamespace(num_attention_heads=query.shape[1], num_key_value_heads=key.shape[1])
    scaling = query.shape[-1] ** -0.5 if scaling is None else scaling
    phase = _current.phase
    if phase == "decode":
        out, _ = kitty_attention_forward(heads, query, layer, scaling)
        cache.quantize_decode(layer_idx)
        return out, None
    if phase == "chunk":
        out, _ = kitty_prefill_attention(heads, query, key, value, layer, scaling)
        cache.append(key, value, layer_idx)
        return out, None
    # prefill on an empty cache: dense causal attention on the prompt (benchmark_kitty.py:302 runs
    # the reference the same way), then the whole prompt is packed
    g = query.shape[1] // key.shape[1]
    out = torch.nn.functional.scaled_dot_product_attention(
        query, key.repeat_interleave(g, 1), value.repeat_interleave(g, 1), is_causal=query.shape[2] > 1, scale=scaling)
    cache.quantize_prefill(layer_idx)
    return out.transpose(1, 2).contiguous(), None


def register() -> None:
    """Make ``attn_implementation="kitty"`` available to transformers models (idempotent)."""
    from transformers import AttentionInterface
    from transformers.masking_utils import AttentionMaskInterface, sdpa_mask
    AttentionInterface.register(NAME, kitty_attention)
    AttentionMaskInterface.register(NAME, sdpa_mask)
