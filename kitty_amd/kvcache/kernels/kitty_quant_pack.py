"""Quantize-and-pack entry points with the reference's signatures
(src/kitty/kvcache/kernels/kitty_quant_pack.py:253-266 and :315-327), backed by the HIP kernels.

Unlike the reference nothing is copied on the host side: the kernels read the ``[B, H, T, D]``
source through its strides (the reference slices and ``.contiguous()``-copies first, :275, :333),
and the boost selection (``abs().mean().topk()`` + ``scatter_``, :280-288) runs fused inside the
K kernel.  Keyword-only additions:

``select="hip"``    fused selection; ties: higher score first, then lower channel index.
``select="torch"``  the reference's literal torch ops on the same device produce the slot map, the
                    kernel consumes it (tie order is then whatever ``torch.topk`` does there).
``slot_map=``       a caller-supplied uint8 ``[B, H, pages, D]`` map (the kernel boundary of the
                    reference's ``quantize_pack_k_kernel``).
``status=``         int32 ``[B, 4]`` device tensor: a page id outside the cache is never written
                    to, and row b's "bad page" word is raised instead (the reference would write
                    out of bounds).
"""
from typing import Optional

import torch

from ... import _lib


def _src_args(x: torch.Tensor, name: str):
    _lib.require_hip(x, name)
    assert x.dim() == 4
    if x.dtype != torch.float16:
        raise ValueError(f"{name} must be float16, got {x.dtype}")
    if x.stride(3) != 1 or any(s % 8 for s in x.stride()[:3]) or x.data_ptr() % 16:
        x = x.contiguous()
    B, H, T, D = x.shape
    return x, (x.data_ptr(), x.stride(0) * 2, x.stride(1) * 2, x.stride(2) * 2, B, H, T, D)


def _status_ptr(status, B: int, device):
    if status is None:
        return None
    _lib.require_hip(status, "status")
    if status.dtype != torch.int32 or status.dim() != 2 or status.shape[0] < B or status.shape[1] != _lib.STATUS_FIELDS \
            or not status.is_contiguous():
        raise ValueError(f"status must be a contiguous int32 [>= {B}, {_lib.STATUS_FIELDS}] tensor")
    return status.data_ptr()


def _check_dst(page_table, cache, cache_metadata):
    for t, n, dt in ((page_table, "page_table", torch.int64), (cache, "cache", torch.uint8),
                     (cache_metadata, "cache_metadata", torch.float16)):
        _lib.require_hip(t, n)
        if t.dtype != dt:
            raise ValueError(f"{n} must be {dt}, got {t.dtype}")
    if page_table.stride(1) != 1 or cache.stride(1) != 1 or not cache_metadata[0].is_contiguous():
        raise ValueError("page_table, cache and cache_metadata rows must be contiguous")


def select_boost_k(key_states: torch.Tensor, key_states_t_offset: int, key_states_page_count: int,
                   page_size: int, d_boost: int) -> torch.Tensor:
    """uint8 ``[B, H, pages, D]`` slot map: rank of each channel among the top ``d_boost`` by
    mean |K| over the page, or ``d_boost`` when the channel is not boosted."""
    key_states, src = _src_args(key_states, "key_states")
    B, H, T, D = src[4:]
    out = torch.empty((B, H, key_states_page_count, D), dtype=torch.uint8, device=key_states.device)
    rc = _lib.lib().kitty_select_boost_k(*src, key_states_t_offset, key_states_page_count, page_size, d_boost,
                                         out.data_ptr(), _lib.current_stream_ptr(key_states.device))
    _lib.check(rc, "select_boost_k")
    return out


def _torch_slot_map(key_states, t_offset, page_count, page_size, d_boost):
    # the reference's own sequence of torch ops (kitty_quant_pack.py:275-288)
    B, H, _, D = key_states.shape
    k = key_states[:, :, t_offset: t_offset + page_size * page_count, :].contiguous()
    k = k.view(B, H, page_count, page_size, D)
    score = k.abs().mean(dim=-2)
    _, top_idx = score.topk(d_boost, dim=-1)
    idx = torch.full((B, H, page_count, D), d_boost, dtype=torch.uint8, device=key_states.device)
    idx.scatter_(-1, top_idx, torch.arange(d_boost, device=key_states.device, dtype=torch.uint8)
                 .view(1, 1, 1, -1).expand_as(top_idx))
    return idx


def quantize_pack_k(
    key_states: torch.Tensor,           # (B, H_KV, T, D): the whole prefill or the 1-page Q-buffer
    key_states_t_offset: int,           # first token to quantize
    key_states_page_count: int,         # number of pages to quantize
    page_table_k: torch.Tensor,
    page_offset_k: int,
    cache: torch.Tensor,                # [MAX_BS * MAX_PAGE, bytes_per_page_K] uint8
    cache_metadata: torch.Tensor,       # [MAX_BS * MAX_PAGE, H_KV, D, 2] float16
    page_size: int,
    d_boost: int,
    *,
    select: str = "hip",
    slot_map: Optional[torch.Tensor] = None,
    status: Optional[torch.Tensor] = None,
) -> None:
    """Quantize and pack the key states into the paged key cache."""
    assert key_states.dim() == 4
    D = key_states.shape[-1]
    assert 0 <= d_boost <= D, f"d_boost must be in [0, {D}], got {d_boost}"
    key_states, src = _src_args(key_states, "key_states")
    _check_dst(page_table_k, cache, cache_metadata)
    if slot_map is None and select == "torch":
        slot_map = _torch_slot_map(key_states, key_states_t_offset, key_states_page_count, page_size, d_boost)
    elif slot_map is None and select != "hip":
        raise ValueError(f"select must be 'hip' or 'torch', got {select!r}")
    if slot_map is not None:
        _lib.require_hip(slot_map, "slot_map")
        B, H = key_states.shape[:2]
        if slot_map.dtype != torch.uint8 or tuple(slot_map.shape) != (B, H, key_states_page_count, D):
            raise ValueError("slot_map must be uint8 [B, H, pages, D]")
        slot_map = slot_map.contiguous()
    rc = _lib.lib().kitty_quant_pack_k(
        *src, key_states_t_offset, key_states_page_count, page_size, d_boost,
        None if slot_map is None else slot_map.data_ptr(),
        page_table_k.data_ptr(), page_table_k.stride(0), page_offset_k,
        cache.data_ptr(), cache.stride(0), cache_metadata.data_ptr(), cache_metadata.stride(0) * 2,
        cache.shape[0], _status_ptr(status, key_states.shape[0], key_states.device),
        _lib.current_stream_ptr(key_states.device))
    _lib.check(rc, "quantize_pack_k")


def quantize_pack_v(
    value_states: torch.Tensor,                 # (B, H_KV, T, D)
    value_states_t_offset: int,
    value_states_page_count: int,
    page_table_v: torch.Tensor,                 # (MAX_BS, MAX_PAGE) int64
    page_offset_v: int,
    cache: torch.Tensor,                        # (MAX_BS * MAX_PAGE, bytes_per_page_V) uint8
    cache_metadata: torch.Tensor,               # (MAX_BS * MAX_PAGE, H_KV, PAGE_SIZE, 2) float16
    page_size: int,
    *,
    status: Optional[torch.Tensor] = None,
) -> None:
    """Quantize and pack the value states into the paged value cache."""
    assert value_states.dim() == 4
    value_states, src = _src_args(value_states, "value_states")
    _check_dst(page_table_v, cache, cache_metadata)
    rc = _lib.lib().kitty_quant_pack_v(
        *src, value_states_t_offset, value_states_page_count, page_size,
        page_table_v.data_ptr(), page_table_v.stride(0), page_offset_v,
        cache.data_ptr(), cache.stride(0), cache_metadata.data_ptr(), cache_metadata.stride(0) * 2,
        cache.shape[0], _status_ptr(status, value_states.shape[0], value_states.device),
        _lib.current_stream_ptr(value_states.device))
    _lib.check(rc, "quantize_pack_v")
