"""Host side of dynamic paging (kitty_amd/kvcache/paging.py), no GPU: the free list, the numpy
shadow of the per-sequence device counters against the oracle's state machine (the reference's
src/kitty/kvcache/kitty.py:97-123, 194-236 per sequence), and the cache's bookkeeping that runs
before any kernel is launched."""
import types

import numpy as np
import pytest

from oracle import kitty_oracle as O
from tests.helpers import make_kv
from kitty_amd.kvcache.paging import OutOfPages, PagedKittyCache, PagePool, step_counters

FIELDS = ("Sink_Count", "PageCount_K", "Q_Buffer_Count_K", "PageCount_V", "Q_Buffer_Count_V", "Local_Count_V",
          "Write_Offset_Local_V")


def _cfg(layers=2):
    return types.SimpleNamespace(num_hidden_layers=layers, head_dim=128, num_key_value_heads=2,
                                 num_attention_heads=8, hidden_size=1024)


def test_page_pool_takes_gives_and_refuses():
    pool = PagePool(5)
    assert pool.free == 5 and pool.take(0) == []
    a = pool.take(3)
    assert a == [0, 1, 2] and pool.free == 2
    with pytest.raises(OutOfPages):
        pool.take(3)
    assert pool.free == 2                                  # nothing was taken
    pool.give([1])
    assert pool.take(2) == [1, 3]                          # last freed, first reused
    for bad in ([1, 1], [4], [5], [-1]):                   # twice in one call, still free, outside
        with pytest.raises(ValueError):
            pool.give(bad)
    pool.give([0, 2, 3, 1])
    assert pool.free == 5 and sorted(pool.take(5)) == [0, 1, 2, 3, 4]
    with pytest.raises(ValueError):
        PagePool(0)


def test_shadow_counters_step_like_the_oracle_per_sequence():
    """Sequences in every phase (sink filling, ring filling, ring evicting, K and V flushing on
    different steps), one of them inactive: 400 steps against one oracle layer per sequence."""
    starts = [3, 32, 100, 32 + 128 + 5, 32 + 3 * 128, 32 + 127, 50]
    max_page = 16
    n = len(starts)
    c = np.zeros((n, 8), dtype=np.int64)
    active = np.ones(n, dtype=bool)
    active[-1] = False
    ols, toks = [], []
    for b, T0 in enumerate(starts):
        k, v = make_kv(1, 1, T0 + 1, seed=T0)
        ol = O.OracleLayer(1, max_page * 128, 1)
        ol.update(k[:, :, :T0], v[:, :, :T0])
        ol.quantize_prefill()
        c[b, :7] = [getattr(ol, f) for f in FIELDS]
        ols.append(ol)
        toks.append((k[:, :, T0:], v[:, :, T0:]))
    frozen = c[-1].copy()
    table = np.zeros((n, max_page), dtype=np.int64)        # every page assigned
    flushes = 0
    for step in range(400):
        before = c[:, [1, 3]].copy()
        fk, fv = step_counters(c, active, table, table, 32, 128, max_page)
        for b in range(n - 1):
            ols[b].update(*toks[b])
            ols[b].quantize_decode()
            assert list(c[b, :7]) == [getattr(ols[b], f) for f in FIELDS], (step, b)
        assert np.array_equal(c[:, 1] - before[:, 0], fk) and np.array_equal(c[:, 3] - before[:, 1], fv)
        flushes += int(fk.sum() + fv.sum())
    assert np.array_equal(c[-1], frozen) and flushes > 30


def test_shadow_counters_without_a_page_hold_the_full_buffer_and_drop_tokens():
    c = np.array([[32, 1, 127, 0, 127, 128, 5, 0]], dtype=np.int64)
    active = np.ones(1, dtype=bool)
    tk = np.array([[7, -1, -1]])
    tv = np.array([[-1, -1, -1]])
    fk, fv = step_counters(c, active, tk, tv, 32, 128, 3)
    assert not fk[0] and not fv[0] and list(c[0]) == [32, 1, 128, 0, 128, 128, 6, 0]
    step_counters(c, active, tk, tv, 32, 128, 3)           # both Q-buffers full: the token is dropped
    assert list(c[0]) == [32, 1, 128, 0, 128, 128, 6, 0]
    tk[0, 1] = 4                                            # K gets its page, V still waits
    fk, fv = step_counters(c, active, tk, tv, 32, 128, 3)
    assert fk[0] and not fv[0] and list(c[0]) == [32, 2, 0, 0, 128, 128, 6, 0]
    c[0, 1] = 3                                             # at MAX_PAGE nothing is flushed
    c[0, 2] = 128
    fk, _ = step_counters(c, active, tk, tv, 32, 128, 3)
    assert not fk[0] and c[0, 1] == 3 and c[0, 2] == 128


def test_paged_cache_bookkeeping_before_any_launch():
    cache = PagedKittyCache(_cfg(), 4, 32 + 128 * 6, pool_pages=5, device="cpu")
    L = cache.kv_cache[0]
    assert L.KeyCache.shape[0] == 5 and L.ValueCache.shape[0] == 5 and cache.max_page == 7
    assert L.PageTable_K is cache.PageTable_K and cache.kv_cache[1].PageTable_V is cache.PageTable_V
    assert int(cache.PageTable_K.max()) == -1 and L.device_counters
    assert cache.seq_counts.shape == (2, 4, 8) and bool((cache.seq_counts[:, :, 7] == 1).all())
    assert L.seq_counts.data_ptr() == cache.seq_counts[0].data_ptr()
    assert cache.pages_for(20) == (1, 1) and cache.pages_for(32 + 128) == (2, 1)
    assert cache.pages_for(32 + 128 * 2 + 50) == (3, 2) and cache.pages_for(32 + 128 * 7) == (7, 7)
    assert cache.active_slots() == [] and cache.pages_in_use() == (0, 0) and cache.get_seq_length() == 0
    cache.check_tables()
    import torch
    k = torch.zeros(1, 2, 32 + 128 * 5 + 3, 128, dtype=torch.float16)
    with pytest.raises(OutOfPages):                        # 6 K pages wanted, 5 in the pool
        with cache.admitting(1):
            assert cache.update(k, k, 0) is True
            cache.quantize_prefill(0)
    assert cache.pages_in_use() == (0, 0) and cache.active_slots() == [] and L.key_states is None
    with pytest.raises(RuntimeError):                      # a block that prefills nothing admits nothing
        with cache.admitting(1):
            pass
    with pytest.raises(ValueError):
        with cache.admitting(4):
            pass
    with pytest.raises(ValueError):
        cache.release(1)
    with pytest.raises(ValueError):
        cache.quantize_prefill(0)                          # outside an admission
    with pytest.raises(ValueError):
        cache.enable_device_counters()
    cache.check_tables()
    with pytest.raises(ValueError):                        # a pool needs its owner's page tables
        from kitty_amd.kvcache.utils_kv_per_layer import KVCache_Layer
        KVCache_Layer(2, 1024, 1, 128, 32, 2, 4, 128, 32, device="cpu", n_pages=4)


def test_chunk_counts_closed_form_equals_single_steps():
    """KittyCache.chunk_counts (the host's copy of what the device's chunk kernels compute) against
    the oracle stepping token by token, from every phase of the state machine."""
    from kitty_amd.kvcache.kitty import KittyCache
    names = ("sink", "pk", "rk", "pv", "rv", "lv", "off")
    for T0 in (1, 31, 32, 33, 32 + 127, 32 + 128, 32 + 129, 32 + 128 * 2 + 5):
        for warm in (0, 140):
            for T in (1, 2, 31, 96, 127, 128, 129, 300):
                k, v = make_kv(1, 1, T0 + warm + T, seed=T0 + T)
                ol = O.OracleLayer(1, 2048, 1)
                ol.update(k[:, :, :T0], v[:, :, :T0])
                ol.quantize_prefill()
                for s in range(warm + T):
                    if s == warm:
                        before = dict(zip(names, [getattr(ol, f) for f in FIELDS]))
                    ol.update(k[:, :, T0 + s:T0 + s + 1], v[:, :, T0 + s:T0 + s + 1])
                    ol.quantize_decode()
                after = KittyCache.chunk_counts(before, T, 32, 128)
                assert [after[n] for n in names] == [getattr(ol, f) for f in FIELDS], (T0, warm, T)


def test_paged_decode_batch_must_be_all_slots():
    import torch
    cache = PagedKittyCache(_cfg(), 4, 1024, pool_pages=8, device="cpu")
    k = torch.zeros(2, 2, 1, 128, dtype=torch.float16)
    with pytest.raises(ValueError, match="all 4 slots"):   # before anything is launched
        cache.update(k, k, 0)


def test_paged_chunk_reserves_its_pages_before_the_first_launch():
    cache = PagedKittyCache(_cfg(), 3, 32 + 128 * 6, pool_pages=9, device="cpu")
    # two sequences as an admission leaves them: counters in the shadow, pages up to the next flush's
    for slot, T0 in ((0, 32 + 128 + 100), (2, 10)):
        cache._take_for_admission(slot, T0)
        n = __import__("kitty_amd.kvcache.kitty", fromlist=["prefill_split"]).prefill_split(T0, 32, 128)
        cache._shadow[slot] = [n["sink"], n["pages_k"], n["qbuf_k"], n["pages_v"], n["qbuf_v"], n["local_v"], 0, 0]
        cache._active[slot] = True
    cache.check_tables()
    assert cache.pages_in_use() == (3, 2)                  # slot 0: 1 + 1 and 0 + 1; slot 2: 0 + 1 each
    cache._reserve_for_chunk(200)                          # slot 0: rk 100 + 200 -> 2 more K pages; V 100 + 200 -> 2
    after = cache._chunk_after(200)
    assert after[0, :7].tolist() == [32, 3, 44, 2, 44, 128, 200 % 128] and after[2, :7].tolist() == [32, 1, 50, 0, 50, 128, 50]
    assert after[1].tolist() == cache._shadow[1].tolist()  # the free slot
    # pages up to and including the one of the flush after the chunk
    assert (cache._table_k[0] >= 0).sum() == 4 and (cache._table_v[0] >= 0).sum() == 3
    assert (cache._table_k[2] >= 0).sum() == 2 and (cache._table_v[2] >= 0).sum() == 1
    cache._end_of_chunk(200)
    cache.check_tables()
    assert cache.seq_lengths().tolist() == [32 + 128 + 100 + 200, 0, 210]
    assert cache.kv_cache[1].get_total_length() == 460
    used = cache.pages_in_use()
    with pytest.raises(OutOfPages):                        # 4 more K pages for slot 0 alone, 3 are free
        cache._reserve_for_chunk(128 * 4)
    assert cache.pages_in_use() == used
    cache.check_tables()
    with pytest.raises(ValueError):                        # beyond max_length
        cache._reserve_for_chunk(128 * 7)
