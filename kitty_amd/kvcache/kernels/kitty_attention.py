"""Decode attention over the packed cache with the reference's signature
(src/kitty/kvcache/kernels/kitty_attention.py:403-408): ``kitty_attention_forward(module, query,
kv_cache, scaling) -> (attn_output [B, 1, H_Q, D] fp16, None)``.

The reference runs a QK kernel, a torch softmax over a ``[B, H_Q, T]`` score tensor in HBM and an
SV kernel, each on a ``(B, H_KV)`` grid (:433-523).  Here one fused split-K kernel streams the
packed pages once (QK^T, online softmax and PV per split of the sequence) and a merge kernel
combines the splits; no score tensor exists.
"""
from typing import Optional

import torch
import torch.nn as nn

from ... import _lib
from ..utils_kv_per_layer import KVCache_Layer

MAX_KV_GROUP = 16   # kitty_attention.py:418


def kitty_attention_forward(
    module: nn.Module,
    query: torch.Tensor,
    kv_cache: KVCache_Layer,
    scaling: float,
    *,
    num_splits: Optional[int] = None,
    variant: int = 0,
):
    assert query.is_contiguous(), "Query tensor must be contiguous."
    B, H_Q, t_query, D = query.size()
    assert t_query == 1, "Only decoding step with t_query=1 is supported."
    assert H_Q == module.num_attention_heads, "H_Q must match num_attention_heads."
    H_KV = module.num_key_value_heads
    KV_GROUP = H_Q // H_KV
    assert KV_GROUP <= MAX_KV_GROUP, f"KV_GROUP ({KV_GROUP}) exceeds MAX_KV_GROUP ({MAX_KV_GROUP})."
    _lib.require_hip(query, "query")
    if query.dtype != torch.float16:
        raise ValueError(f"query must be float16, got {query.dtype}")
    if H_KV != kv_cache.H_KV or B > kv_cache.MAX_BS:
        raise ValueError("query does not match the cache (H_KV or batch size)")

    lib = _lib.lib()
    if kv_cache.seq_counts is None:
        max_tiles = 1 + (kv_cache.get_total_length() - kv_cache.Sink_Count + kv_cache.PAGE_SIZE - 1) // kv_cache.PAGE_SIZE
    else:
        max_tiles = 2 + kv_cache.MAX_PAGE
    if not num_splits or num_splits <= 0:
        num_splits = lib.kitty_decode_attn_default_splits(B, H_KV, max_tiles, int(kv_cache.seq_counts is not None))
    ws_bytes = lib.kitty_decode_attn_workspace_bytes(B, H_Q, D, num_splits)
    ws = kv_cache.workspace(ws_bytes)
    # [B, T=1, H_Q, D], the layout HF attention modules expect (kitty_attention.py:475-481)
    attn_output = torch.empty((B, t_query, H_Q, D), dtype=query.dtype, device=query.device)
    desc = kv_cache.descriptor()
    rc = lib.kitty_decode_attn(desc, query.data_ptr(), B, H_Q, float(scaling), attn_output.data_ptr(),
                               ws.data_ptr(), ws.numel(), num_splits, variant,
                               _lib.current_stream_ptr(query.device))
    _lib.check(rc, "kitty_attention_forward")
    return attn_output, None


def kitty_prefill_attention(
    module: nn.Module,
    query: torch.Tensor,
    key_states: torch.Tensor,
    value_states: torch.Tensor,
    kv_cache: KVCache_Layer,
    scaling: float,
):
    """Chunked-prefill attention: ``query [B, H_Q, T_q, D]`` attends to everything ``kv_cache``
    holds and, causally, to the chunk's own ``key_states`` / ``value_states [B, H_KV, T_q, D]``
    (fp16, not yet appended).  Returns ``(attn_output [B, T_q, H_Q, D] fp16, None)``.

    An extension of the reference's interface, whose attention asserts ``t_query == 1``
    (kitty_attention.py:411) and whose prefill is dense attention on an empty cache
    (benchmark_kitty.py:302); cached tokens enter exactly as in decode.  Append the chunk afterwards
    with ``KittyCache.update`` (empty cache) or ``KittyCache.append``.
    """
    B, H_Q, T_q, D = query.size()
    assert H_Q == module.num_attention_heads, "H_Q must match num_attention_heads."
    H_KV = module.num_key_value_heads
    KV_GROUP = H_Q // H_KV
    assert KV_GROUP <= MAX_KV_GROUP, f"KV_GROUP ({KV_GROUP}) exceeds MAX_KV_GROUP ({MAX_KV_GROUP})."
    for name, t in (("query", query), ("key_states", key_states), ("value_states", value_states)):
        _lib.require_hip(t, name)
        if t.dtype != torch.float16:
            raise ValueError(f"{name} must be float16, got {t.dtype}")
    if key_states.shape != (B, H_KV, T_q, D) or value_states.shape != key_states.shape:
        raise ValueError(f"key_states / value_states must be [B, H_KV, T_q, D] = {(B, H_KV, T_q, D)}, got "
                         f"{tuple(key_states.shape)} / {tuple(value_states.shape)}")
    if H_KV != kv_cache.H_KV or B > kv_cache.MAX_BS:
        raise ValueError("query does not match the cache (H_KV or batch size)")
    if query.stride(-1) != 1:
        query = query.contiguous()
    if key_states.stride(-1) != 1:
        key_states = key_states.contiguous()
    if value_states.stride() != key_states.stride():
        value_states = value_states.contiguous()
        key_states = key_states.contiguous()

    lib = _lib.lib()
    attn_output = torch.empty((B, T_q, H_Q, D), dtype=query.dtype, device=query.device)
    desc = kv_cache.descriptor()
    qs, ks = [x * 2 for x in query.stride()], [x * 2 for x in key_states.stride()]
    rc = lib.kitty_prefill_attn(desc, query.data_ptr(), qs[0], qs[1], qs[2], key_states.data_ptr(),
                                value_states.data_ptr(), ks[0], ks[1], ks[2], B, H_Q, T_q, float(scaling),
                                attn_output.data_ptr(), _lib.current_stream_ptr(query.device))
    _lib.check(rc, "kitty_prefill_attention")
    return attn_output, None
