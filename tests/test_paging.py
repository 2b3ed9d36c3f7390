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
