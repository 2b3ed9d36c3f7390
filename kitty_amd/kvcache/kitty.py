"""``KittyCache``: the HF-Transformers cache plugin of the packed 2-bit KV cache.

Same class name, constructor, methods and return conventions as the reference
(src/kitty/kvcache/kitty.py:24-258): ``update()`` returns ``True`` in prefill and ``False`` in
decode, the caller runs attention and then calls ``quantize_prefill`` / ``quantize_decode``
(call order fixed by src/kitty/models/qwen3/modeling_qwen3.py:225-251).
"""
from typing import Any, Optional

import torch

try:  # the plugin subclasses HF's Cache when transformers is importable
    from transformers.cache_utils import Cache as _HFCache
except Exception:  # pragma: no cover - transformers is optional for the kernels themselves
    _HFCache = object

from .. import _lib
from .kernels.kitty_quant_pack import quantize_pack_k, quantize_pack_v
from .utils_kv_per_layer import KVCache_Layer


def prefill_split(len_prefill: int, S: int, P: int) -> dict:
    """Where the tokens of a prefill go (kitty.py:126-192): the first ``sink`` stay fp16 for good;
    of the keys, the newest ``(T - S) % P`` wait in the Q-buffer and whole pages in between are
    packed; of the values, the newest ``min(P, T - S)`` fill the local ring, the ``% P`` remainder
    before them waits in the Q-buffer, the rest is packed."""
    sink = min(S, len_prefill)
    qbuf_k = max(0, len_prefill - sink) % P
    pages_k = (len_prefill - sink - qbuf_k) // P
    local_v = max(0, min(P, len_prefill - sink))
    qbuf_v = max(0, len_prefill - sink - local_v) % P
    pages_v = (len_prefill - sink - local_v - qbuf_v) // P
    return dict(sink=sink, qbuf_k=qbuf_k, pages_k=pages_k, local_v=local_v, qbuf_v=qbuf_v, pages_v=pages_v)


class KittyCache(_HFCache):
    """Kitty KV cache: fp16 sink + packed 2-bit pages (25 % of key channels at 4 bit) + fp16
    residual windows that are flushed into packed pages when full."""
    is_compileable = False

    def __init__(self, config, max_batch_size: int, max_length: int, *, device="cuda",
                 select: str = "hip", layer_kwargs: Optional[dict] = None) -> None:
        if _HFCache is not object:
            try:
                super().__init__(layers=[])          # transformers >= 4.54
            except TypeError:
                super().__init__()                   # transformers 4.53 (the reference's pin)
        self.kv_cache: list[KVCache_Layer] = []
        self.num_hidden_layers = config.num_hidden_layers
        self.head_dim = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
        self.num_key_value_heads = config.num_key_value_heads
        # Kitty constants (kitty.py:43-47)
        self.page_size = 128
        self.d_boosted = self.head_dim // 4
        self.sink_length = 32
        self.low_bit = 2
        self.high_bit = 4
        self.select = select
        for _ in range(self.num_hidden_layers):
            self.kv_cache.append(KVCache_Layer(
                MAX_BS=max_batch_size, MAX_LEN=max_length, H_KV=self.num_key_value_heads, D=self.head_dim,
                D_BOOSTED=self.d_boosted, LOW_BIT=self.low_bit, HIGH_BIT=self.high_bit,
                PAGE_SIZE=self.page_size, S=self.sink_length, device=device, **(layer_kwargs or {})))

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[dict[str, Any]] = None) -> bool:
        """Append to layer ``layer_idx``.  Returns True in prefill (the states are stashed for
        ``quantize_prefill``), False in decode (one token written to the fp16 windows)."""
        kvcache = self.kv_cache[layer_idx]
        if kvcache.Sink_Count == 0:
            kvcache.key_states = key_states
            kvcache.value_states = value_states
            return True
        assert key_states.shape[-2] == 1 and value_states.shape[-2] == 1, \
            "Decode: key_states and value_states should have sequence length of 1."
        B = key_states.shape[0]
        if kvcache.device_counters:
            self._append_token_device(kvcache, key_states, value_states)
            return False
        with torch.no_grad():
            if kvcache.Sink_Count < kvcache.S:
                idx = kvcache.Sink_Count
                kvcache.Sink_Buffer_K[:B, :, idx, :] = key_states[:, :, 0, :]
                kvcache.Sink_Buffer_V[:B, :, idx, :] = value_states[:, :, 0, :]
                kvcache.Sink_Count += 1
            else:
                assert kvcache.Q_Buffer_Count_K < kvcache.Q_Buffer_K.size(2)
                kvcache.Q_Buffer_K[:B, :, kvcache.Q_Buffer_Count_K, :] = key_states[:, :, 0, :]
                kvcache.Q_Buffer_Count_K += 1
                assert kvcache.Local_Count_V <= kvcache.PAGE_SIZE
                if kvcache.Local_Count_V < kvcache.PAGE_SIZE:
                    kvcache.Local_Buffer_V[:B, :, kvcache.Local_Count_V, :] = value_states[:, :, 0, :]
                    kvcache.Local_Count_V += 1
                else:   # ring full: the oldest row moves to the V Q-buffer, the new one takes its place
                    assert kvcache.Q_Buffer_Count_V < kvcache.Q_Buffer_V.size(2)
                    w = kvcache.Write_Offset_Local_V
                    kvcache.Q_Buffer_V[:B, :, kvcache.Q_Buffer_Count_V, :] = kvcache.Local_Buffer_V[:B, :, w, :]
                    kvcache.Q_Buffer_Count_V += 1
                    kvcache.Local_Buffer_V[:B, :, w, :] = value_states[:, :, 0, :]
                    kvcache.Write_Offset_Local_V = (w + 1) % kvcache.PAGE_SIZE
        return False

    def quantize_prefill(self, layer_idx: int = 0) -> None:
        """Split the stashed prefill into sink / packed pages / fp16 residuals (kitty.py:126-192)."""
        kvcache = self.kv_cache[layer_idx]
        if kvcache.key_states is None or kvcache.value_states is None:
            raise ValueError("No key_states or value_states to quantize. Please call update() first.")
        n = self._store_prefill(kvcache, kvcache.key_states, kvcache.value_states, 0)
        kvcache.Sink_Count = n["sink"]
        kvcache.Q_Buffer_Count_K = n["qbuf_k"]
        kvcache.PageCount_K += n["pages_k"]
        kvcache.Local_Count_V = n["local_v"]
        kvcache.Q_Buffer_Count_V = n["qbuf_v"]
        kvcache.PageCount_V += n["pages_v"]
        kvcache.key_states = None
        kvcache.value_states = None

    def _store_prefill(self, kvcache: KVCache_Layer, K: torch.Tensor, V: torch.Tensor, first_row: int) -> dict:
        """Write a prefill ``[B, H_KV, T, D]`` into rows ``first_row .. first_row + B`` of an empty
        layer: sink, packed pages (through those rows of the page tables, from entry 0) and fp16
        residuals.  Returns ``prefill_split``'s counts; the caller owns the counters."""
        B, P = K.shape[0], kvcache.PAGE_SIZE
        rows = slice(first_row, first_row + B)
        len_prefill = K.shape[-2]
        n = prefill_split(len_prefill, kvcache.S, P)
        len_sink, len_qbuf_k, pages_k = n["sink"], n["qbuf_k"], n["pages_k"]
        len_local_v, len_qbuf_v, pages_v = n["local_v"], n["qbuf_v"], n["pages_v"]
        if pages_k > kvcache.MAX_PAGE:
            raise ValueError(f"prefill of {len_prefill} tokens exceeds max_length={kvcache.MAX_LEN}")
        kvcache.Sink_Buffer_K[rows, :, :len_sink, :].copy_(K[:, :, :len_sink, :])
        if len_qbuf_k > 0:
            kvcache.Q_Buffer_K[rows, :, :len_qbuf_k, :].copy_(K[:, :, len_prefill - len_qbuf_k:, :])
        if pages_k > 0:
            quantize_pack_k(K, len_sink, pages_k, kvcache.PageTable_K[rows], 0, kvcache.KeyCache,
                            kvcache.KeyCache_metadata, P, kvcache.D_BOOSTED, select=self.select,
                            status=kvcache.status[rows])
        kvcache.Sink_Buffer_V[rows, :, :len_sink, :].copy_(V[:, :, :len_sink, :])
        if len_local_v > 0:
            kvcache.Local_Buffer_V[rows, :, :len_local_v, :].copy_(V[:, :, len_prefill - len_local_v:, :])
        if len_qbuf_v > 0:
            assert len_local_v > 0, "Local buffer must be filled before using Q-buffer."
            lo = len_prefill - len_local_v - len_qbuf_v
            kvcache.Q_Buffer_V[rows, :, :len_qbuf_v, :].copy_(V[:, :, lo: lo + len_qbuf_v, :])
        if pages_v > 0:
            assert len_prefill - len_sink - len_local_v - len_qbuf_v == pages_v * P
            quantize_pack_v(V, len_sink, pages_v, kvcache.PageTable_V[rows], 0, kvcache.ValueCache,
                            kvcache.ValueCache_metadata, P, status=kvcache.status[rows])
        return n

    def quantize_decode(self, layer_idx: int = 0) -> None:
        """Flush a full Q-buffer into the next packed page; K and V fill up independently
        (kitty.py:194-236)."""
        kvcache = self.kv_cache[layer_idx]
        if kvcache.device_counters:
            self._flush_full_device(kvcache)
            return
        if kvcache.Q_Buffer_Count_K == kvcache.PAGE_SIZE:
            if kvcache.PageCount_K >= kvcache.MAX_PAGE:
                raise ValueError(f"key cache is full (max_length={kvcache.MAX_LEN})")
            quantize_pack_k(kvcache.Q_Buffer_K, 0, 1, kvcache.PageTable_K, kvcache.PageCount_K, kvcache.KeyCache,
                            kvcache.KeyCache_metadata, kvcache.PAGE_SIZE, kvcache.D_BOOSTED, select=self.select,
                            status=kvcache.status)
            kvcache.PageCount_K += 1
            kvcache.Q_Buffer_Count_K = 0
        if kvcache.Q_Buffer_Count_V == kvcache.PAGE_SIZE:
            if kvcache.PageCount_V >= kvcache.MAX_PAGE:
                raise ValueError(f"value cache is full (max_length={kvcache.MAX_LEN})")
            quantize_pack_v(kvcache.Q_Buffer_V, 0, 1, kvcache.PageTable_V, kvcache.PageCount_V, kvcache.ValueCache,
                            kvcache.ValueCache_metadata, kvcache.PAGE_SIZE, status=kvcache.status)
            kvcache.PageCount_V += 1
            kvcache.Q_Buffer_Count_V = 0

    # ---- what the device could not do --------------------------------------------------------------
    def check_status(self, raise_on_error: bool = True, clear: bool = False) -> dict:
        """Read the layers' device-side status words (one synchronising copy per call).

        The reference stops with an assert before a buffer overflows (kitty.py:109,113,118).  With
        per-sequence counters on the device the host cannot know, so the kernels skip such work,
        exit normally and leave a record per sequence: tokens dropped because a Q-buffer was still
        full, flushes skipped for want of a page, page ids outside the cache met by a writer or by
        attention.  Returns ``{name: int32 array [layers, MAX_BS]}`` and raises ``RuntimeError``
        when anything is set (unless ``raise_on_error=False``); ``clear=True`` zeroes the words."""
        import numpy as np
        st = torch.stack([L.status for L in self.kv_cache]).cpu().numpy()
        out = {name: st[:, :, i].copy() for i, name in enumerate(_lib.STATUS_NAMES)}
        if clear:
            for L in self.kv_cache:
                L.status.zero_()
        if raise_on_error and st.any():
            parts = []
            for name, a in out.items():
                if a.any():
                    layers, seqs = np.nonzero(a)
                    parts.append(f"{name}: layer {int(layers[0])} sequence {int(seqs[0])} = {int(a[layers[0], seqs[0]])}"
                                 f" ({len(seqs)} (layer, sequence) pairs)")
            raise RuntimeError("the device skipped work it could not do: " + "; ".join(parts))
        return out

    # ---- per-sequence counters on the device ---------------------------------------------------
    def enable_device_counters(self, seq_counts: Optional[torch.Tensor] = None) -> None:
        """Switch every layer to device-side per-sequence counters (after the prefill): decode
        steps then cost one append launch and one flush launch per layer, never read the device,
        and serve sequences of different lengths.  ``seq_counts [MAX_BS, 8]`` sets a ragged
        starting state for all layers; default: every sequence at the layer's current state."""
        if self.select != "hip":
            raise ValueError("device counters use the fused channel selection (select='hip')")
        for L in self.kv_cache:
            L.enable_device_counters(seq_counts)

    def step_host_counters(self) -> None:
        """Advance every layer's host shadow by one decode step (append + flush) without launching
        anything.  For callers that replay a captured HIP graph of the decode step: the replay
        advances the device counters, this keeps ``get_seq_length`` and the capacity checks in
        step.  Capturing runs the Python of one step without executing its kernels: save
        ``host_counters()`` before a capture and ``restore_host_counters`` after it."""
        for L in self.kv_cache:
            if not L.device_counters:
                raise ValueError("step_host_counters is for layers with device counters")
            P = L.PAGE_SIZE
            if L.Sink_Count >= L.S and L.Q_Buffer_Count_K >= P:
                raise ValueError("Q-buffer is full")
            L.step_host_counters()
            if (L.Q_Buffer_Count_K == P and L.PageCount_K >= L.MAX_PAGE) or \
                    (L.Q_Buffer_Count_V == P and L.PageCount_V >= L.MAX_PAGE):
                raise ValueError(f"cache is full (max_length={L.MAX_LEN})")
            if L.Q_Buffer_Count_K == P:
                L.PageCount_K += 1
                L.Q_Buffer_Count_K = 0
            if L.Q_Buffer_Count_V == P:
                L.PageCount_V += 1
                L.Q_Buffer_Count_V = 0

    def host_counters(self) -> list:
        return [L.counts() for L in self.kv_cache]

    def restore_host_counters(self, saved: list) -> None:
        for L, row in zip(self.kv_cache, saved):
            for f, v in zip(L.COUNT_FIELDS, row):
                setattr(L, f, int(v))

    def _append_token_device(self, L: KVCache_Layer, key_states: torch.Tensor, value_states: torch.Tensor,
                             rope=None) -> None:
        if L.Sink_Count >= L.S and L.Q_Buffer_Count_K >= L.PAGE_SIZE:
            raise ValueError("Q-buffer is full: call quantize_decode() after every decode step")
        self._launch_append(L, key_states, value_states, rope)
        L.step_host_counters()

    def update_with_rope(self, key_states: torch.Tensor, value_states: torch.Tensor, cos: torch.Tensor,
                         sin: torch.Tensor, layer_idx: int) -> bool:
        """Decode-step ``update`` that also applies the rotary embedding to the new key:
        ``key_states`` are the keys BEFORE the rotation, ``cos`` / ``sin`` fp16 ``[B, 1, D]`` (or
        ``[B, D]``, or one row for all) as the model's rotary module returns them.  The append kernel
        stores ``k * cos + rotate_half(k) * sin`` with fp16 tensor arithmetic's roundings, i.e. the
        bits the caller's own ``apply_rotary_pos_emb`` would have produced
        (modeling_qwen3.py:215-220), without materialising the rotated key.  Needs device counters."""
        L = self.kv_cache[layer_idx]
        if not L.device_counters:
            raise ValueError("the fused rotary append is part of the device-counter path: call enable_device_counters()")
        assert key_states.shape[-2] == 1 and value_states.shape[-2] == 1, \
            "Decode: key_states and value_states should have sequence length of 1."
        B, D = key_states.shape[0], L.D
        rope = []
        for name, t in (("cos", cos), ("sin", sin)):
            _lib.require_hip(t, name)
            if t.dtype != torch.float16 or t.shape[-1] != D or t.numel() not in (D, B * D):
                raise ValueError(f"{name} must be float16 with {D} or {B} x {D} elements, got {tuple(t.shape)} {t.dtype}")
            rope.append(t.reshape(-1, D).contiguous())
        self._append_token_device(L, key_states, value_states, rope)
        return False

    def _launch_append(self, L: KVCache_Layer, key_states: torch.Tensor, value_states: torch.Tensor, rope=None) -> None:
        B = key_states.shape[0]
        for name, t in (("key_states", key_states), ("value_states", value_states)):
            _lib.require_hip(t, name)
            if t.dtype != torch.float16:
                raise ValueError(f"{name} must be float16, got {t.dtype}")
        if key_states.shape != (B, L.H_KV, 1, L.D) or value_states.shape != key_states.shape or B > L.MAX_BS:
            raise ValueError(f"key_states / value_states must be [B <= {L.MAX_BS}, {L.H_KV}, 1, {L.D}]")
        if key_states.stride(-1) != 1:
            key_states = key_states.contiguous()
        if value_states.stride() != key_states.stride():
            key_states, value_states = key_states.contiguous(), value_states.contiguous()
        cos_p = sin_p = None
        rope_stride = 0
        if rope is not None:
            cos, sin = rope
            cos_p, sin_p = cos.data_ptr(), sin.data_ptr()
            rope_stride = 0 if cos.shape[0] == 1 else cos.stride(0) * 2
        rc = _lib.lib().kitty_append_token(L.descriptor(), key_states.data_ptr(), value_states.data_ptr(),
                                           key_states.stride(0) * 2, key_states.stride(1) * 2, cos_p, sin_p, rope_stride,
                                           B, _lib.current_stream_ptr(key_states.device))
        _lib.check(rc, "KittyCache.update")
        L.active_batch = B

    def _flush_full_device(self, L: KVCache_Layer) -> None:
        P = L.PAGE_SIZE
        if (L.Q_Buffer_Count_K == P and L.PageCount_K >= L.MAX_PAGE) or \
                (L.Q_Buffer_Count_V == P and L.PageCount_V >= L.MAX_PAGE):
            raise ValueError(f"cache is full (max_length={L.MAX_LEN})")
        self._launch_flush(L)
        if L.Q_Buffer_Count_K == P:
            L.PageCount_K += 1
            L.Q_Buffer_Count_K = 0
        if L.Q_Buffer_Count_V == P:
            L.PageCount_V += 1
            L.Q_Buffer_Count_V = 0

    def _launch_flush(self, L: KVCache_Layer) -> None:
        rc = _lib.lib().kitty_flush_full(L.descriptor(), L.active_batch, _lib.current_stream_ptr(L.device))
        _lib.check(rc, "KittyCache.quantize_decode")

    def append(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int = 0) -> None:
        """Append a chunk of T >= 1 tokens ``[B, H_KV, T, D]`` to a layer in one go.

        An extension (the reference's ``update`` takes one token at a time once the cache holds
        anything, kitty.py:97-98).  The resulting state is the one T calls of ``update`` +
        ``quantize_decode`` would leave: same counters, same packed pages bit for bit, same fp16
        rows in the same slots of the sink, the Q-buffers and the local ring.  Pages that lie
        entirely inside the chunk are quantized straight from it; only pages that start with
        rows already buffered go through the Q-buffer.  On an empty layer this is
        ``update`` + ``quantize_prefill``.

        With device counters the kernels decide per sequence whether the chunk fits: a sequence it
        does not fit (it would pass ``MAX_PAGE``, or a page-table entry it needs is not a valid page
        id) keeps its state and has its T tokens counted in the ``tokens_dropped`` status word,
        while the host ints - a shadow of the longest sequence, advanced in closed form without
        reading the device - move on regardless.  Call ``check_status()`` after chunk appends on such
        caches when the tables or counters were written by anyone but this class.
        """
        L = self.kv_cache[layer_idx]
        if key_states.shape != value_states.shape or key_states.dim() != 4:
            raise ValueError("key_states and value_states must both be [B, H_KV, T, D]")
        if L.device_counters:
            self._append_chunk_device(L, key_states, value_states)
            return
        if L.get_total_length() == 0:
            self.update(key_states, value_states, layer_idx)
            self.quantize_prefill(layer_idx)
            return
        B, T, P = key_states.shape[0], key_states.shape[-2], L.PAGE_SIZE
        a = min(L.S - L.Sink_Count, T)                  # tokens that still go to the sink
        n = T - a
        # capacity first, so that a rejected chunk leaves the layer untouched
        new_pk = (L.Q_Buffer_Count_K + n) // P
        lv_after = min(P, L.Local_Count_V + n)
        evicted = L.Local_Count_V + n - lv_after        # rows leaving the ring for the V Q-buffer
        new_pv = (L.Q_Buffer_Count_V + evicted) // P
        if L.PageCount_K + new_pk > L.MAX_PAGE or L.PageCount_V + new_pv > L.MAX_PAGE:
            raise ValueError(f"appending {T} tokens exceeds max_length={L.MAX_LEN}")
        with torch.no_grad():
            if a > 0:
                L.Sink_Buffer_K[:B, :, L.Sink_Count:L.Sink_Count + a, :].copy_(key_states[:, :, :a, :])
                L.Sink_Buffer_V[:B, :, L.Sink_Count:L.Sink_Count + a, :].copy_(value_states[:, :, :a, :])
                L.Sink_Count += a
            if n == 0:
                return
            # K: every new row enters the quantize stream
            self._push_k(L, key_states, a, T, B)
            # V: the ring keeps the newest P rows; what it evicts, oldest first, enters the stream:
            # first rows of the old ring (age order = slots from Write_Offset_Local_V), then the head
            # of the chunk
            from_ring = min(evicted, L.Local_Count_V)
            off = L.Write_Offset_Local_V
            first = min(from_ring, P - off)
            self._push_v(L, L.Local_Buffer_V, off, off + first, B)
            self._push_v(L, L.Local_Buffer_V, 0, from_ring - first, B)
            from_chunk = evicted - from_ring
            self._push_v(L, value_states, a, a + from_chunk, B)
            # the newest rows take the slots single steps would have given them
            base = L.Local_Count_V if L.Local_Count_V < P else off
            j = from_chunk
            while j < n:
                slot = (base + j) % P
                run = min(n - j, P - slot)
                L.Local_Buffer_V[:B, :, slot:slot + run, :].copy_(value_states[:, :, a + j:a + j + run, :])
                j += run
            L.Local_Count_V = lv_after
            L.Write_Offset_Local_V = (off + evicted) % P

    @staticmethod
    def chunk_counts(c: dict, T: int, S: int, P: int) -> dict:
        """The counters after a chunk of ``T`` tokens (what T single steps leave; the device's
        chunk kernels use the same closed form).  ``c``: sink, pk, rk, pv, rv, lv, off."""
        a = min(S - c["sink"], T)
        n = T - a
        lv2 = min(P, c["lv"] + n)
        e = c["lv"] + n - lv2
        return dict(sink=c["sink"] + a, pk=c["pk"] + (c["rk"] + n) // P, rk=(c["rk"] + n) % P,
                    pv=c["pv"] + (c["rv"] + e) // P, rv=(c["rv"] + e) % P, lv=lv2, off=(c["off"] + e) % P)

    def _append_chunk_device(self, L: KVCache_Layer, key_states: torch.Tensor, value_states: torch.Tensor) -> None:
        """``append`` with per-sequence counters on the device: three launches (new pages straight
        from their sources, fp16 rows, counters), every sequence from its own state.  The host ints
        follow the longest sequence by the same closed form."""
        B, H, T, D = key_states.shape
        for name, t in (("key_states", key_states), ("value_states", value_states)):
            _lib.require_hip(t, name)
            if t.dtype != torch.float16:
                raise ValueError(f"{name} must be float16, got {t.dtype}")
        if (H, D) != (L.H_KV, L.D) or B > L.MAX_BS or T < 1:
            raise ValueError(f"key_states / value_states must be [B <= {L.MAX_BS}, {L.H_KV}, T >= 1, {L.D}]")
        if key_states.stride(-1) != 1 or any(s % 8 for s in key_states.stride()[:3]) or key_states.data_ptr() % 16:
            key_states = key_states.contiguous()
        if value_states.stride() != key_states.stride() or value_states.data_ptr() % 16:
            key_states, value_states = key_states.contiguous(), value_states.contiguous()
        names = ("sink", "pk", "rk", "pv", "rv", "lv", "off")
        before = dict(zip(names, L.counts()[:7]))
        after = self.chunk_counts(before, T, L.S, L.PAGE_SIZE)
        if after["pk"] > L.MAX_PAGE or after["pv"] > L.MAX_PAGE:
            raise ValueError(f"appending {T} tokens exceeds max_length={L.MAX_LEN}")
        ks = [x * 2 for x in key_states.stride()]
        rc = _lib.lib().kitty_append_chunk(L.descriptor(), key_states.data_ptr(), value_states.data_ptr(),
                                           ks[0], ks[1], ks[2], B, T, _lib.current_stream_ptr(key_states.device))
        _lib.check(rc, "KittyCache.append")
        L.active_batch = B
        for f, name in zip(L.COUNT_FIELDS, names):
            setattr(L, f, int(after[name]))

    def _push_k(self, L: KVCache_Layer, src: torch.Tensor, lo: int, hi: int, B: int) -> None:
        """Rows ``src[:, :, lo:hi]`` enter the K quantize stream: whole pages straight from ``src``
        when the Q-buffer is empty, otherwise through the Q-buffer, flushing it when full."""
        P = L.PAGE_SIZE
        while lo < hi:
            if L.Q_Buffer_Count_K == 0 and hi - lo >= P:
                pages = (hi - lo) // P
                quantize_pack_k(src, lo, pages, L.PageTable_K, L.PageCount_K, L.KeyCache, L.KeyCache_metadata, P,
                                L.D_BOOSTED, select=self.select)
                L.PageCount_K += pages
                lo += pages * P
                continue
            m = min(P - L.Q_Buffer_Count_K, hi - lo)
            L.Q_Buffer_K[:B, :, L.Q_Buffer_Count_K:L.Q_Buffer_Count_K + m, :].copy_(src[:, :, lo:lo + m, :])
            L.Q_Buffer_Count_K += m
            lo += m
            if L.Q_Buffer_Count_K == P:
                quantize_pack_k(L.Q_Buffer_K, 0, 1, L.PageTable_K, L.PageCount_K, L.KeyCache, L.KeyCache_metadata,
                                P, L.D_BOOSTED, select=self.select)
                L.PageCount_K += 1
                L.Q_Buffer_Count_K = 0

    def _push_v(self, L: KVCache_Layer, src: torch.Tensor, lo: int, hi: int, B: int) -> None:
        """The V side of ``_push_k``."""
        P = L.PAGE_SIZE
        while lo < hi:
            if L.Q_Buffer_Count_V == 0 and hi - lo >= P:
                pages = (hi - lo) // P
                quantize_pack_v(src, lo, pages, L.PageTable_V, L.PageCount_V, L.ValueCache, L.ValueCache_metadata, P)
                L.PageCount_V += pages
                lo += pages * P
                continue
            m = min(P - L.Q_Buffer_Count_V, hi - lo)
            L.Q_Buffer_V[:B, :, L.Q_Buffer_Count_V:L.Q_Buffer_Count_V + m, :].copy_(src[:, :, lo:lo + m, :])
            L.Q_Buffer_Count_V += m
            lo += m
            if L.Q_Buffer_Count_V == P:
                quantize_pack_v(L.Q_Buffer_V, 0, 1, L.PageTable_V, L.PageCount_V, L.ValueCache,
                                L.ValueCache_metadata, P)
                L.PageCount_V += 1
                L.Q_Buffer_Count_V = 0

    def get_seq_length(self, layer_idx: int = 0) -> int:
        """Number of cached tokens of a layer."""
        return self.kv_cache[layer_idx].get_total_length()


def get_kvcache_kitty(config, max_batch_size: int, max_length: int, **kwargs) -> KittyCache:
    """Factory with the reference's signature (kitty.py:244-258)."""
    return KittyCache(config=config, max_batch_size=max_batch_size, max_length=max_length, **kwargs)
