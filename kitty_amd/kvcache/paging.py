"""Dynamic paging for the packed KV cache: a pool of pages shared by all sequence slots.

The reference allocates ``MAX_BS * MAX_PAGE`` pages per layer up front and fills its page tables
with the identity (src/kitty/kvcache/utils_kv_per_layer.py:33-59): every slot owns the pages of
its worst case for good.  Here a layer holds ``pool_pages`` pages, a sequence is given pages as it
grows and returns them when it ends, and sequences are admitted to and released from slots while
the others keep decoding.  Nothing changes in the wire format or in the kernels' arithmetic: they
always went through the page tables.

Division of labour: the *host* owns the free lists and decides which page a sequence gets (it has
to know anyway whether a request fits before admitting it); the *device* owns the per-sequence
counters and runs the append / flush state machine (``kitty_append_token`` / ``kitty_flush_full``).
The host never reads the device: the counters of a sequence are a function of its prompt length
and the number of decode steps, so a numpy shadow steps along.  Every active sequence always has
the page of its *next* flush assigned, so a decode step (or the replay of a captured graph of it)
finds its page in the table; the entry for the flush after that is written right after the step
in which a flush happened, 128 steps ahead of its use.

One pair of page tables serves all layers (a sequence uses the same page ids in every layer, each
layer has its own page arrays), so admitting, growing and releasing a sequence costs one small
table write, not one per layer.
"""
from __future__ import annotations

import contextlib
from typing import Any, Optional

import numpy as np
import torch

from .kitty import KittyCache, prefill_split

INACTIVE = 1      # KITTY_SEQ_INACTIVE
_F_SINK, _F_PK, _F_RK, _F_PV, _F_RV, _F_LV, _F_OFF, _F_FLAGS = range(8)


class OutOfPages(RuntimeError):
    """The pool cannot supply the pages asked for; nothing was taken."""


class PagePool:
    """Free list of the page ids ``0 .. n_pages - 1`` (host side, last freed = first reused)."""

    def __init__(self, n_pages: int):
        if n_pages < 1:
            raise ValueError("a pool needs at least one page")
        self.n_pages = int(n_pages)
        self._free = list(range(self.n_pages - 1, -1, -1))
        self._is_free = bytearray(b"\x01" * self.n_pages)

    @property
    def free(self) -> int:
        return len(self._free)

    def take(self, n: int) -> list[int]:
        if n < 0:
            raise ValueError("cannot take a negative number of pages")
        if n > len(self._free):
            raise OutOfPages(f"{n} pages wanted, {len(self._free)} of {self.n_pages} free")
        ids = [self._free.pop() for _ in range(n)]
        for i in ids:
            self._is_free[i] = 0
        return ids

    def give(self, ids) -> None:
        ids = [int(i) for i in ids]
        for i in ids:
            if not 0 <= i < self.n_pages:
                raise ValueError(f"page id {i} is not in the pool")
        if len(set(ids)) != len(ids) or any(self._is_free[i] for i in ids):
            raise ValueError("a page is given back twice")
        for i in ids:
            self._is_free[i] = 1
        self._free.extend(ids)


def step_counters(c: np.ndarray, active: np.ndarray, table_k: np.ndarray, table_v: np.ndarray, S: int, P: int,
                  max_page: int):
    """One decode step (append, then flush) on the host shadow ``c [slots, 8]`` of the device
    counters, by the rules of ``kitty_append_token`` / ``kitty_flush_full`` (the reference's
    kitty.py:97-123 and :194-236 per sequence).  Returns the masks of the sequences whose K / V
    Q-buffer was flushed in this step."""
    to_sink = active & (c[:, _F_SINK] < S)
    rest = active & ~to_sink
    # a full Q-buffer (its flush found no page) drops the token, as the device does
    rest &= (c[:, _F_RK] < P) & ((c[:, _F_LV] < P) | (c[:, _F_RV] < P))
    ring_free = rest & (c[:, _F_LV] < P)
    evict = rest & ~ring_free
    c[to_sink, _F_SINK] += 1
    c[rest, _F_RK] += 1
    c[ring_free, _F_LV] += 1
    c[evict, _F_RV] += 1
    c[evict, _F_OFF] = (c[evict, _F_OFF] + 1) % P
    rows = np.arange(c.shape[0])
    flushed = []
    for f_pages, f_rows, table in ((_F_PK, _F_RK, table_k), (_F_PV, _F_RV, table_v)):
        full = active & (c[:, f_rows] == P) & (c[:, f_pages] < max_page)
        full &= table[rows, np.minimum(c[:, f_pages], max_page - 1)] >= 0
        c[full, f_pages] += 1
        c[full, f_rows] = 0
        flushed.append(full)
    return flushed[0], flushed[1]


class PagedKittyCache(KittyCache):
    """``KittyCache`` over a page pool, with slots that are admitted and released one by one.

        cache = PagedKittyCache(config, max_batch_size=64, max_length=32768, pool_pages=4096)
        with cache.admitting(slot):                 # prefill of one sequence, batch size 1
            model(prompt_ids, past_key_values=cache)    # update(..) -> True, then quantize_prefill(..)
        ...
        model(next_ids[max_batch_size, 1], past_key_values=cache)   # decode: all slots, inactive ones idle
        ...
        cache.release(slot)

    Decode batches are the slots ``0 .. B-1`` themselves (row b of the batch is slot b, as in the
    reference): rows of inactive slots are computed and ignored - their attention output is zero -
    which keeps the launch sequence of a step fixed, so a captured graph of it stays valid while
    sequences come and go.  The counters live on the device from the start.
    """

    def __init__(self, config, max_batch_size: int, max_length: int, pool_pages: int, *, device="cuda") -> None:
        dev = torch.device(device)
        head_dim = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
        if head_dim != 128:
            raise ValueError(f"a page pool keeps its counters on the device, which is built for head_dim 128 "
                             f"(got {head_dim}); use KittyCache for other head dimensions")
        max_page = -(-max_length // 128)          # the layers' MAX_PAGE (page size 128, kitty.py:43)
        self.PageTable_K = torch.full((max_batch_size, max_page), -1, dtype=torch.int64, device=dev)
        self.PageTable_V = torch.full((max_batch_size, max_page), -1, dtype=torch.int64, device=dev)
        super().__init__(config, max_batch_size, max_length, device=device, select="hip",
                         layer_kwargs=dict(n_pages=pool_pages, page_tables=(self.PageTable_K, self.PageTable_V)))
        L0 = self.kv_cache[0]
        assert L0.MAX_PAGE == max_page
        self.n_slots, self.max_page = max_batch_size, max_page
        self.pool_k, self.pool_v = PagePool(pool_pages), PagePool(pool_pages)
        self._table_k = np.full((max_batch_size, max_page), -1, dtype=np.int64)   # host copies of the tables
        self._table_v = np.full((max_batch_size, max_page), -1, dtype=np.int64)
        self._shadow = np.zeros((max_batch_size, 8), dtype=np.int64)
        self._shadow[:, _F_FLAGS] = INACTIVE
        self._active = np.zeros(max_batch_size, dtype=bool)
        self._starved: set[tuple[str, int]] = set()          # ("k" | "v", slot) waiting for a page
        # one tensor of counters for all layers: a slot is (de)activated everywhere with one write
        self.seq_counts = torch.zeros((len(self.kv_cache), max_batch_size, 8), dtype=torch.int32, device=dev)
        self.seq_counts[:, :, _F_FLAGS] = INACTIVE
        for i, L in enumerate(self.kv_cache):
            L.seq_counts = self.seq_counts[i]
            L.device_counters = True
        self._admit_slot: Optional[int] = None
        self._admit_len: Optional[int] = None
        self._capturing = False

    # ---- bookkeeping ---------------------------------------------------------------------------
    def active_slots(self) -> list[int]:
        return [int(b) for b in np.flatnonzero(self._active)]

    def seq_lengths(self) -> np.ndarray:
        """Tokens held per slot (0 for a free slot), from the host shadow."""
        c = self._shadow
        return np.where(self._active, c[:, _F_SINK] + c[:, _F_PK] * self.page_size + c[:, _F_RK], 0)

    def pages_in_use(self) -> tuple[int, int]:
        return self.pool_k.n_pages - self.pool_k.free, self.pool_v.n_pages - self.pool_v.free

    def pages_for(self, n_tokens: int) -> tuple[int, int]:
        """Pages (K, V) a prompt of ``n_tokens`` takes on admission, the page of its next flush
        included: what ``admitting`` needs to find free."""
        L = self.kv_cache[0]
        n = prefill_split(n_tokens, L.S, L.PAGE_SIZE)
        return min(n["pages_k"] + 1, self.max_page), min(n["pages_v"] + 1, self.max_page)

    def _sync_longest(self) -> None:
        """The layers' host ints shadow the longest active sequence (capacity checks, lengths)."""
        lens = self.seq_lengths()
        row = self._shadow[int(np.argmax(lens))] if self._active.any() else np.zeros(8, dtype=np.int64)
        for L in self.kv_cache:
            for f, v in zip(L.COUNT_FIELDS, row[:7]):
                setattr(L, f, int(v))

    def _write_tables(self, kind: str, slots, entries, ids) -> None:
        host, dev = (self._table_k, self.PageTable_K) if kind == "k" else (self._table_v, self.PageTable_V)
        host[slots, entries] = ids
        dev[torch.as_tensor(slots, device=dev.device), torch.as_tensor(entries, device=dev.device)] = \
            torch.as_tensor(ids, dtype=torch.int64, device=dev.device)

    def ensure_pages(self) -> list[tuple[str, int]]:
        """Give every active sequence the page of its next flush where it has none (after pages
        came back to a pool that had run dry).  Returns the (kind, slot) pairs still waiting."""
        for kind, pool, host, f in (("k", self.pool_k, self._table_k, _F_PK), ("v", self.pool_v, self._table_v, _F_PV)):
            slots, entries = [], []
            for k, slot in sorted(self._starved):
                if k != kind:
                    continue
                entry = int(self._shadow[slot, f])
                if not self._active[slot] or entry >= self.max_page or host[slot, entry] >= 0:
                    self._starved.discard((kind, slot))
                elif len(slots) < pool.free:
                    slots.append(slot)
                    entries.append(entry)
                    self._starved.discard((kind, slot))
            if slots:
                self._write_tables(kind, slots, entries, pool.take(len(slots)))
        return sorted(self._starved)

    # ---- admission and release -----------------------------------------------------------------
    @contextlib.contextmanager
    def admitting(self, slot: int):
        """Route ``update`` / ``quantize_prefill`` (every layer, batch size 1) to the free slot
        ``slot``.  The slot turns active when the block ends; if it raises, or a layer was left
        out, the slot stays free and its pages go back."""
        if not 0 <= slot < self.n_slots:
            raise ValueError(f"slot {slot} outside [0, {self.n_slots})")
        if self._active[slot]:
            raise ValueError(f"slot {slot} holds a sequence: release it first")
        if self._admit_slot is not None:
            raise RuntimeError("one admission at a time")
        self._admit_slot, self._admit_len = slot, None
        self._admit_layers: set[int] = set()
        # the status words are sticky and per slot: what the previous tenant of the slot left (a dry
        # pool is an ordinary event here) must not be read as the new sequence's
        for L in self.kv_cache:
            L.status[slot].zero_()
        try:
            yield self
            if self._admit_len is None or len(self._admit_layers) != len(self.kv_cache):
                raise RuntimeError("admission needs update() + quantize_prefill() on every layer")
        except BaseException:
            self._return_pages(slot)
            for L in self.kv_cache:
                L.key_states = L.value_states = None
            raise
        finally:
            self._admit_slot = None
        L = self.kv_cache[0]
        n = prefill_split(self._admit_len, L.S, L.PAGE_SIZE)
        row = [n["sink"], n["pages_k"], n["qbuf_k"], n["pages_v"], n["qbuf_v"], n["local_v"], 0, 0]
        self._shadow[slot] = row
        self._active[slot] = True
        self.seq_counts[:, slot] = torch.tensor(row, dtype=torch.int32, device=self.seq_counts.device)
        self._sync_longest()

    def _take_for_admission(self, slot: int, n_tokens: int) -> None:
        L = self.kv_cache[0]
        n = prefill_split(n_tokens, L.S, L.PAGE_SIZE)
        if n["pages_k"] > self.max_page:
            raise ValueError(f"prompt of {n_tokens} tokens exceeds max_length={L.MAX_LEN}")
        need_k, need_v = self.pages_for(n_tokens)
        if need_k > self.pool_k.free or need_v > self.pool_v.free:
            raise OutOfPages(f"prompt of {n_tokens} tokens needs {need_k} K and {need_v} V pages; "
                             f"{self.pool_k.free} and {self.pool_v.free} are free")
        self._write_tables("k", [slot] * need_k, list(range(need_k)), self.pool_k.take(need_k))
        self._write_tables("v", [slot] * need_v, list(range(need_v)), self.pool_v.take(need_v))

    def _return_pages(self, slot: int) -> None:
        for kind, pool, host, dev in (("k", self.pool_k, self._table_k, self.PageTable_K),
                                      ("v", self.pool_v, self._table_v, self.PageTable_V)):
            ids = host[slot][host[slot] >= 0]
            if ids.size:
                pool.give(ids.tolist())
            host[slot] = -1
            dev[slot] = -1
            self._starved.discard((kind, slot))

    def release(self, slot: int) -> None:
        """End the sequence in ``slot``: its pages return to the pools (kernels already enqueued on
        the stream still read them; the next writer is ordered behind them on the same stream)."""
        if not 0 <= slot < self.n_slots or not self._active[slot]:
            raise ValueError(f"slot {slot} holds no sequence")
        self._return_pages(slot)
        self._active[slot] = False
        self._shadow[slot] = 0
        self._shadow[slot, _F_FLAGS] = INACTIVE
        row = torch.zeros(8, dtype=torch.int32, device=self.seq_counts.device)
        row[_F_FLAGS] = INACTIVE
        self.seq_counts[:, slot] = row
        self._sync_longest()
        self.ensure_pages()

    # ---- the reference's cache interface ---------------------------------------------------------
    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[dict[str, Any]] = None) -> bool:
        L = self.kv_cache[layer_idx]
        if self._admit_slot is not None:
            if key_states.shape[0] != 1 or key_states.shape != value_states.shape:
                raise ValueError("admission takes one sequence: key_states / value_states [1, H_KV, T, D]")
            L.key_states, L.value_states = key_states, value_states
            return True
        assert key_states.shape[-2] == 1 and value_states.shape[-2] == 1, \
            "Decode: key_states and value_states should have sequence length of 1."
        if key_states.shape[0] != self.n_slots:
            # the host shadow steps every active slot; a smaller batch would leave the slots past it behind
            raise ValueError(f"a decode batch of a paged cache is all {self.n_slots} slots, got {key_states.shape[0]} rows")
        self._launch_append(L, key_states, value_states)     # the host ints follow at the end of the step
        return False

    def quantize_prefill(self, layer_idx: int = 0) -> None:
        slot = self._admit_slot
        if slot is None:
            raise ValueError("prefill goes through `with cache.admitting(slot):`")
        L = self.kv_cache[layer_idx]
        if L.key_states is None or L.value_states is None:
            raise ValueError("No key_states or value_states to quantize. Please call update() first.")
        T = L.key_states.shape[-2]
        if self._admit_len is None:
            self._take_for_admission(slot, T)
            self._admit_len = T
        elif T != self._admit_len:
            raise ValueError("the layers of one admission must see the same number of tokens")
        self._store_prefill(L, L.key_states, L.value_states, slot)
        L.key_states = L.value_states = None
        self._admit_layers.add(layer_idx)

    def quantize_decode(self, layer_idx: int = 0) -> None:
        self._launch_flush(self.kv_cache[layer_idx])
        if layer_idx == len(self.kv_cache) - 1 and not self._capturing:
            self._end_of_step()

    @contextlib.contextmanager
    def capturing(self):
        """Run one decode step under HIP graph capture: its Python runs, its kernels do not, so the
        host side stays as it is and no page is assigned (that write must not be recorded).  After
        each replay call ``step_host_counters()``."""
        self._capturing = True
        try:
            yield self
        finally:
            self._capturing = False

    def step_host_counters(self) -> None:
        """After the replay of a captured decode step (all layers): advance the host side."""
        self._end_of_step()

    def append(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int = 0) -> None:
        """``T`` new tokens for every slot at once, ``[n_slots, H_KV, T, D]`` (rows of free slots are
        ignored): the state afterwards is the one ``T`` decode steps leave.  Call it for every layer,
        layer 0 first, the last layer last, like the decode step's calls.  The pages the chunk fills
        (and the page of the flush after it) are taken from the pools before the first layer's
        launch; if they cannot be had, ``OutOfPages`` is raised and nothing has changed."""
        if self._admit_slot is not None:
            raise ValueError("a prompt under admission goes through update() + quantize_prefill()")
        if key_states.dim() != 4 or key_states.shape != value_states.shape or key_states.shape[0] != self.n_slots:
            raise ValueError(f"key_states / value_states must both be [{self.n_slots}, H_KV, T, D]")
        T = key_states.shape[-2]
        if layer_idx == 0 and not self._capturing:
            self._reserve_for_chunk(T)
        L = self.kv_cache[layer_idx]
        saved = L.counts()
        self._append_chunk_device(L, key_states, value_states)
        for f, v in zip(L.COUNT_FIELDS, saved):          # the host ints are set for all layers at the end
            setattr(L, f, int(v))
        if layer_idx == len(self.kv_cache) - 1 and not self._capturing:
            self._end_of_chunk(T)

    def _chunk_after(self, T: int) -> np.ndarray:
        """The shadow counters of every slot after a chunk of T tokens (active slots only change)."""
        L = self.kv_cache[0]
        c = self._shadow.copy()
        for slot in np.flatnonzero(self._active):
            r = c[slot]
            after = self.chunk_counts(dict(sink=r[_F_SINK], pk=r[_F_PK], rk=r[_F_RK], pv=r[_F_PV], rv=r[_F_RV],
                                           lv=r[_F_LV], off=r[_F_OFF]), T, L.S, L.PAGE_SIZE)
            c[slot, :7] = [after[k] for k in ("sink", "pk", "rk", "pv", "rv", "lv", "off")]
        return c

    def _reserve_for_chunk(self, T: int) -> None:
        L = self.kv_cache[0]
        c = self._shadow
        if (self._active & (c[:, _F_SINK] >= L.S) & ((c[:, _F_RK] >= L.PAGE_SIZE) | (c[:, _F_RV] >= L.PAGE_SIZE))).any():
            raise OutOfPages("a sequence still waits for the page of a flush: release pages (ensure_pages) first")
        after = self._chunk_after(T)
        if (after[:, _F_PK] > self.max_page).any() or (after[:, _F_PV] > self.max_page).any():
            raise ValueError(f"appending {T} tokens exceeds max_length={L.MAX_LEN}")
        plan = []
        for kind, pool, host, f in (("k", self.pool_k, self._table_k, _F_PK), ("v", self.pool_v, self._table_v, _F_PV)):
            slots, entries = [], []
            for slot in np.flatnonzero(self._active):
                have = int((host[slot] >= 0).sum())                       # assigned entries are a prefix of the row
                want = min(int(after[slot, f]) + 1, self.max_page)       # the pages filled, and the next flush's
                slots += [int(slot)] * max(0, want - have)
                entries += list(range(have, want))
            if len(slots) > pool.free:
                raise OutOfPages(f"a chunk of {T} tokens needs {len(slots)} more {kind.upper()} pages, {pool.free} are free")
            plan.append((kind, pool, slots, entries))
        for kind, pool, slots, entries in plan:
            if slots:
                self._write_tables(kind, slots, entries, pool.take(len(slots)))
            self._starved = {(k, s) for k, s in self._starved if k != kind}

    def _end_of_chunk(self, T: int) -> None:
        self._shadow = self._chunk_after(T)
        self._sync_longest()

    def enable_device_counters(self, seq_counts=None) -> None:
        raise ValueError("a paged cache keeps its counters on the device from the start")

    def _end_of_step(self) -> None:
        """All layers have appended and flushed: step the shadow and assign the page of the next
        flush to every sequence that flushed.  Raises OutOfPages, once and with the bookkeeping
        complete, when a pool cannot supply one: release a sequence within the next 128 steps, or
        the starved sequence keeps its full Q-buffer and stops taking tokens until a page comes."""
        L = self.kv_cache[0]
        fk, fv = step_counters(self._shadow, self._active, self._table_k, self._table_v, L.S, L.PAGE_SIZE,
                               self.max_page)
        new = set()
        for kind, mask, f in (("k", fk, _F_PK), ("v", fv, _F_PV)):
            for slot in np.flatnonzero(mask):
                if self._shadow[slot, f] < self.max_page:
                    new.add((kind, int(slot)))
        self._starved |= new
        self._sync_longest()
        c = self._shadow
        if (self._active & (c[:, _F_PK] >= self.max_page) & (c[:, _F_RK] == L.PAGE_SIZE)).any():
            raise ValueError(f"cache is full (max_length={L.MAX_LEN})")
        if self._starved:
            short = new & set(self.ensure_pages())
            if short:
                raise OutOfPages(f"no page for the next flush of {sorted(short)}")

    def check_tables(self) -> None:
        """Invariants of the allocator (for tests and debugging; reads the device tables)."""
        for kind, pool, host, dev, f in (("k", self.pool_k, self._table_k, self.PageTable_K, _F_PK),
                                         ("v", self.pool_v, self._table_v, self.PageTable_V, _F_PV)):
            assert np.array_equal(dev.cpu().numpy(), host), f"{kind}: device table differs from the host copy"
            used = host[host >= 0]
            assert used.size == np.unique(used).size, f"{kind}: a page is assigned twice"
            assert used.size == pool.n_pages - pool.free, f"{kind}: pool count"
            assert used.size == 0 or (used.max() < pool.n_pages and not any(pool._is_free[i] for i in used))
            for slot in range(self.n_slots):
                n = int(self._shadow[slot, f]) if self._active[slot] else 0
                want = min(n + 1, self.max_page) if self._active[slot] and (kind, slot) not in self._starved else n
                assert (host[slot, :want] >= 0).all() and (host[slot, want:] < 0).all(), (kind, slot, n)
