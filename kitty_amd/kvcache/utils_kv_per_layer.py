"""Per-layer storage of the packed KV cache.

Mirrors the reference's ``KVCache_Layer`` (src/kitty/kvcache/utils_kv_per_layer.py:12-95): same
constructor arguments, same attribute names, same tensor shapes and dtypes, so code written
against the reference keeps working.  Differences, all additive:

* ``device=`` (default ``"cuda"``, the reference hard-codes it, :38-78);
* the identity page tables are filled with ``arange`` instead of 2*MAX_BS*MAX_PAGE scalar writes
  (:56-59);
* ``seq_counts`` - an optional int32 ``[MAX_BS, 8]`` device tensor with per-sequence occupancy for
  ragged batches (the reference keeps one set of host ints for the whole batch, :53-54,65,71-72,
  79-80).  When it is ``None`` the shared counters are used, exactly like the reference;
* ``enable_device_counters()`` - from then on decode steps advance ``seq_counts`` on the device
  (one fused append kernel, one flush launch) and the host ints only shadow the longest sequence;
* ``status`` - int32 ``[MAX_BS, 4]`` on the device: what the kernels could not do (tokens dropped,
  flushes skipped, page ids out of range); the reference asserts on the host instead
  (kitty.py:109,113,118), which kernels that take their counters from device memory cannot;
* ``n_pages=`` / ``page_tables=`` - a page pool smaller (or larger) than the reference's static
  ``MAX_BS * MAX_PAGE`` pages, with page tables handed in by the owner of the pool (entries of -1:
  no page assigned); see ``paging.PagedKittyCache``.
"""
import math
from typing import Optional

import torch

from .. import _lib


class KVCache_Layer:
    """KV cache of a single layer; pages are statically allocated."""

    def __init__(self, MAX_BS: int, MAX_LEN: int, H_KV: int, D: int, D_BOOSTED: int, LOW_BIT: int, HIGH_BIT: int,
                 PAGE_SIZE: int, S: int, device="cuda", *, n_pages: Optional[int] = None,
                 page_tables: Optional[tuple] = None):
        assert PAGE_SIZE % 128 == 0, "PAGE_SIZE must be a multiple of 128."
        self.BITS_PER_BYTE = 8
        self.HIGH_BIT = HIGH_BIT
        self.LOW_BIT = LOW_BIT
        self.MAX_BS = MAX_BS
        self.MAX_LEN = MAX_LEN
        self.H_KV = H_KV
        self.D = D
        self.D_BOOSTED = D_BOOSTED
        self.PAGE_SIZE = PAGE_SIZE
        self.S = S
        self.device = torch.device(device)
        dev = self.device
        # packed pages
        self.MAX_PAGE = math.ceil(MAX_LEN / PAGE_SIZE)
        self.bytes_per_page_K = (H_KV * D * PAGE_SIZE * LOW_BIT // 8             # low 2-bit plane
                                 + H_KV * D_BOOSTED * PAGE_SIZE * LOW_BIT // 8   # high 2-bit plane (boosted)
                                 + H_KV * D)                                     # channel -> slot map
        if n_pages is None:
            n_pages = MAX_BS * self.MAX_PAGE
        elif n_pages < 1 or page_tables is None:
            raise ValueError("a page pool needs n_pages >= 1 and the page tables of its owner")
        self.KeyCache = torch.zeros((n_pages, self.bytes_per_page_K), dtype=torch.uint8, device=dev)
        self.KeyCache_metadata = torch.zeros((n_pages, H_KV, D, 2), dtype=torch.half, device=dev)
        self.bytes_per_page_V = H_KV * PAGE_SIZE * D * LOW_BIT // 8
        self.ValueCache = torch.zeros((n_pages, self.bytes_per_page_V), dtype=torch.uint8, device=dev)
        self.ValueCache_metadata = torch.zeros((n_pages, H_KV, PAGE_SIZE, 2), dtype=torch.half, device=dev)
        if page_tables is None:
            ident = (torch.arange(self.MAX_PAGE, dtype=torch.int64).view(1, -1)
                     + torch.arange(MAX_BS, dtype=torch.int64).view(-1, 1) * self.MAX_PAGE)
            self.PageTable_K = ident.to(dev)
            self.PageTable_V = ident.clone().to(dev)
        else:
            self.PageTable_K, self.PageTable_V = page_tables
            for t in page_tables:
                if t.dtype != torch.int64 or tuple(t.shape) != (MAX_BS, self.MAX_PAGE) or not t.is_contiguous() \
                        or t.device.type != dev.type:
                    raise ValueError(f"page tables must be contiguous int64 [{MAX_BS}, {self.MAX_PAGE}] on {dev}")
        self.PageCount_K = 0
        self.PageCount_V = 0
        # fp16 windows
        self.Sink_Buffer_K = torch.zeros((MAX_BS, H_KV, S, D), dtype=torch.float16, device=dev)
        self.Sink_Buffer_V = torch.zeros((MAX_BS, H_KV, S, D), dtype=torch.float16, device=dev)
        self.Sink_Count = 0
        self.Q_Buffer_K = torch.zeros((MAX_BS, H_KV, PAGE_SIZE, D), dtype=torch.float16, device=dev)
        self.Q_Buffer_V = torch.zeros((MAX_BS, H_KV, PAGE_SIZE, D), dtype=torch.float16, device=dev)
        self.Q_Buffer_Count_K = 0
        self.Q_Buffer_Count_V = 0
        self.Local_Buffer_V = torch.zeros((MAX_BS, H_KV, PAGE_SIZE, D), dtype=torch.float16, device=dev)
        self.Local_Count_V = 0
        self.Write_Offset_Local_V = 0
        # prefill stash
        self.key_states: Optional[torch.Tensor] = None
        self.value_states: Optional[torch.Tensor] = None
        # extensions
        self.seq_counts: Optional[torch.Tensor] = None
        self.status = torch.zeros((MAX_BS, _lib.STATUS_FIELDS), dtype=torch.int32, device=dev)
        self.device_counters = False
        self.active_batch = MAX_BS
        self._workspace: Optional[torch.Tensor] = None
        self._desc: Optional[_lib.KittyKVLayer] = None

    def get_total_length(self) -> int:
        """Total number of cached tokens (the reference's :85-95, including its K == V check)."""
        total_length = self.PageCount_K * self.PAGE_SIZE + self.Sink_Count + self.Q_Buffer_Count_K
        seqlen_V = (self.PageCount_V * self.PAGE_SIZE + self.Sink_Count + self.Q_Buffer_Count_V
                    + self.Local_Count_V)
        assert total_length == seqlen_V, f"seqlen_K: {total_length}, seqlen_V: {seqlen_V}"
        return total_length

    COUNT_FIELDS = ("Sink_Count", "PageCount_K", "Q_Buffer_Count_K", "PageCount_V", "Q_Buffer_Count_V",
                    "Local_Count_V", "Write_Offset_Local_V")

    def enable_device_counters(self, seq_counts: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Keep the occupancy counters on the device, one int32 row of 8 per sequence, and let
        ``KittyCache.update`` / ``quantize_decode`` advance them there.

        ``seq_counts`` (``[MAX_BS, 8]``, field order of ``counts()``) gives every sequence its own
        state; without it every row starts from the host counters.  The host ints stay in use as
        a shadow of the longest sequence: they advance by the same rules on every step, without
        reading the device, and answer ``get_total_length()`` and the capacity checks.
        """
        if self.D != 128:
            raise ValueError(f"device-side counters (fused append, flush and chunk kernels) are built for head_dim 128; "
                             f"a cache with head_dim {self.D} keeps the reference's host counters")
        if seq_counts is None:
            seq_counts = torch.tensor([self.counts()] * self.MAX_BS, dtype=torch.int32)
        if tuple(seq_counts.shape) != (self.MAX_BS, _lib.SEQ_COUNT_FIELDS):
            raise ValueError(f"seq_counts must be [{self.MAX_BS}, {_lib.SEQ_COUNT_FIELDS}], got {tuple(seq_counts.shape)}")
        host = seq_counts.detach().to("cpu", torch.int64)
        P = self.PAGE_SIZE
        if bool((host < 0).any()) or bool((host[:, [0]] > self.S).any()) or bool((host[:, [2, 4, 5]] > P).any()) \
                or bool((host[:, 6] >= P).any()) or bool((host[:, [1, 3]] > self.MAX_PAGE).any()):
            raise ValueError("seq_counts holds a counter outside its range")
        len_k = host[:, 0] + host[:, 1] * P + host[:, 2]
        len_v = host[:, 0] + host[:, 3] * P + host[:, 4] + host[:, 5]
        if not bool((len_k == len_v).all()):
            raise ValueError("seq_counts: a sequence holds different numbers of keys and values")
        longest = host[int(torch.argmax(len_k))].tolist()
        for f, v in zip(self.COUNT_FIELDS, longest):
            setattr(self, f, int(v))
        self.seq_counts = seq_counts.detach().to(self.device, torch.int32).contiguous().clone()
        self.device_counters = True
        return self.seq_counts

    def step_host_counters(self) -> None:
        """One decode token in the host counters (the reference's rules, kitty.py:104-123)."""
        if self.Sink_Count < self.S:
            self.Sink_Count += 1
            return
        assert self.Q_Buffer_Count_K < self.PAGE_SIZE
        self.Q_Buffer_Count_K += 1
        if self.Local_Count_V < self.PAGE_SIZE:
            self.Local_Count_V += 1
        else:
            assert self.Q_Buffer_Count_V < self.PAGE_SIZE
            self.Q_Buffer_Count_V += 1
            self.Write_Offset_Local_V = (self.Write_Offset_Local_V + 1) % self.PAGE_SIZE

    # ---- C-ABI view -------------------------------------------------------------------------
    def counts(self):
        return [self.Sink_Count, self.PageCount_K, self.Q_Buffer_Count_K, self.PageCount_V,
                self.Q_Buffer_Count_V, self.Local_Count_V, self.Write_Offset_Local_V, 0]

    def descriptor(self) -> "_lib.KittyKVLayer":
        """struct kitty_kv_layer for this layer; pointers are cached, counters refreshed."""
        d = self._desc
        if d is None:
            d = _lib.KittyKVLayer()
            d.H_KV, d.D, d.D_BOOSTED, d.PAGE_SIZE, d.S, d.MAX_PAGE = (
                self.H_KV, self.D, self.D_BOOSTED, self.PAGE_SIZE, self.S, self.MAX_PAGE)
            d.key_cache, d.key_cache_stride_page = self.KeyCache.data_ptr(), self.KeyCache.stride(0)
            d.key_meta, d.key_meta_stride_page = self.KeyCache_metadata.data_ptr(), self.KeyCache_metadata.stride(0) * 2
            d.value_cache, d.value_cache_stride_page = self.ValueCache.data_ptr(), self.ValueCache.stride(0)
            d.value_meta = self.ValueCache_metadata.data_ptr()
            d.value_meta_stride_page = self.ValueCache_metadata.stride(0) * 2
            d.page_table_k, d.page_table_k_stride_b = self.PageTable_K.data_ptr(), self.PageTable_K.stride(0)
            d.page_table_v, d.page_table_v_stride_b = self.PageTable_V.data_ptr(), self.PageTable_V.stride(0)
            d.sink_k, d.sink_v = self.Sink_Buffer_K.data_ptr(), self.Sink_Buffer_V.data_ptr()
            d.sink_stride_b, d.sink_stride_h = self.Sink_Buffer_K.stride(0) * 2, self.Sink_Buffer_K.stride(1) * 2
            d.qbuf_k, d.qbuf_v = self.Q_Buffer_K.data_ptr(), self.Q_Buffer_V.data_ptr()
            d.local_v = self.Local_Buffer_V.data_ptr()
            d.win_stride_b, d.win_stride_h = self.Q_Buffer_K.stride(0) * 2, self.Q_Buffer_K.stride(1) * 2
            d.cache_pages_k, d.cache_pages_v = self.KeyCache.shape[0], self.ValueCache.shape[0]
            d.status = self.status.data_ptr()
            self._desc = d
        for i, v in enumerate(self.counts()):
            d.counts[i] = int(v)
        d.seq_counts = None if self.seq_counts is None else self.seq_counts.data_ptr()
        return d

    def workspace(self, nbytes: int) -> torch.Tensor:
        """Split-K scratch, grown on demand and kept with the layer (the reference allocates its
        score tensor on every call, kitty_attention.py:425-430)."""
        if self._workspace is None or self._workspace.numel() < nbytes:
            self._workspace = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=self.device)
        return self._workspace
