"""Append / flush state machine (reference: src/kitty/kvcache/kitty.py:63-236): the oracle's
restatement against closed forms and invariants, and the product's host logic (KittyCache on CPU
tensors with the two kernel entry points replaced by recorders) against the oracle step by step."""
import types

import numpy as np
import pytest
import torch

from oracle import kitty_oracle as O
from tests.helpers import make_kv

P, S = 128, 32


def closed_form(T):
    """Occupancy after a prefill of T tokens (kitty.py:131-188)."""
    ls = min(S, T)
    n = T - ls
    rk = n % P
    pk = (n - rk) // P
    lv = min(P, n)
    rv = (n - lv) % P
    pv = (n - lv - rv) // P
    return ls, pk, rk, pv, rv, lv


@pytest.mark.parametrize("T", [1, 31, 32, 33, 159, 160, 161, 287, 288, 289, 415, 416, 417, 1000])
def test_prefill_occupancy_closed_form(T):
    k, v = make_kv(1, 1, T, seed=T)
    ol = O.OracleLayer(1, 2048, 1)
    assert ol.update(k, v) is True
    ol.quantize_prefill()
    assert (ol.Sink_Count, ol.PageCount_K, ol.Q_Buffer_Count_K, ol.PageCount_V, ol.Q_Buffer_Count_V,
            ol.Local_Count_V) == closed_form(T)
    assert ol.get_total_length() == T and ol.Write_Offset_Local_V == 0
    assert ol.key_states is None and ol.value_states is None


def _chronological_fp16(ol, b=0, h=0):
    """fp16 tokens still held verbatim, as (token index, K row or None, V row or None)."""
    sink = ol.Sink_Count
    k_rows = {i: ol.Sink_Buffer_K[b, h, i] for i in range(sink)}
    v_rows = {i: ol.Sink_Buffer_V[b, h, i] for i in range(sink)}
    base_k = sink + P * ol.PageCount_K
    for i in range(ol.Q_Buffer_Count_K):
        k_rows[base_k + i] = ol.Q_Buffer_K[b, h, i]
    base_v = sink + P * ol.PageCount_V
    for i in range(ol.Q_Buffer_Count_V):
        v_rows[base_v + i] = ol.Q_Buffer_V[b, h, i]
    for i in range(ol.Local_Count_V):
        v_rows[base_v + ol.Q_Buffer_Count_V + i] = ol.Local_Buffer_V[b, h, (ol.Write_Offset_Local_V + i) % P]
    return k_rows, v_rows


def test_every_token_lives_in_exactly_one_place_and_fp16_rows_are_verbatim():
    T0, steps = 50, 420
    k, v = make_kv(1, 1, T0 + steps, seed=3)
    ol = O.OracleLayer(1, 2048, 1)
    ol.update(k[:, :, :T0], v[:, :, :T0])
    ol.quantize_prefill()
    for s in range(steps):
        t = T0 + s
        assert ol.update(k[:, :, t:t + 1], v[:, :, t:t + 1]) is False
        assert ol.get_total_length() == t + 1                     # K side == V side, nothing lost
        assert 1 <= ol.Q_Buffer_Count_K <= P                      # attention runs before the flush
        k_rows, v_rows = _chronological_fp16(ol)
        for i, row in k_rows.items():
            assert np.array_equal(row, k[0, 0, i])
        for i, row in v_rows.items():
            assert np.array_equal(row, v[0, 0, i])
        ol.quantize_decode()
        assert ol.Q_Buffer_Count_K < P and ol.Q_Buffer_Count_V < P
    assert ol.PageCount_K == (T0 + steps - S) // P and ol.Local_Count_V == P


def test_pages_do_not_depend_on_how_tokens_arrived():
    """Groups are anchored at token 32 + 128 p: one long prefill, or a short prefill followed by
    single-token appends, must produce identical packed pages."""
    T = S + P * 3 + 40
    k, v = make_kv(2, 2, T, seed=17)
    a = O.OracleLayer(2, 1024, 2)
    a.update(k, v)
    a.quantize_prefill()
    b = O.OracleLayer(2, 1024, 2)
    T0 = 45
    b.update(k[:, :, :T0], v[:, :, :T0])
    b.quantize_prefill()
    for t in range(T0, T):
        b.update(k[:, :, t:t + 1], v[:, :, t:t + 1])
        b.quantize_decode()
    assert a.PageCount_K == b.PageCount_K == 3
    assert np.array_equal(a.KeyCache, b.KeyCache)
    assert np.array_equal(a.KeyCache_metadata.view(np.uint16), b.KeyCache_metadata.view(np.uint16))
    pv = min(a.PageCount_V, b.PageCount_V)          # V pages lag by the local window
    assert pv >= 2
    rows = np.concatenate([np.arange(pv) + bb * a.MAX_PAGE for bb in range(2)])
    assert np.array_equal(a.ValueCache[rows], b.ValueCache[rows])
    assert np.array_equal(a.ValueCache_metadata[rows].view(np.uint16), b.ValueCache_metadata[rows].view(np.uint16))


def test_error_paths_of_the_oracle():
    ol = O.OracleLayer(1, 512, 1)
    with pytest.raises(ValueError):
        ol.quantize_prefill()                                  # update() first (kitty.py:129-130)
    k, v = make_kv(1, 1, 40, seed=1)
    ol.update(k, v)
    ol.quantize_prefill()
    with pytest.raises(AssertionError):
        ol.update(k[:, :, :2], v[:, :, :2])                    # decode appends one token (kitty.py:97-98)


# ---------------------------------------------------------------------------------------------
# the product's host logic on CPU tensors, kernels replaced by recorders
# ---------------------------------------------------------------------------------------------
@pytest.fixture()
def cpu_cache(monkeypatch):
    import kitty_amd
    from kitty_amd.kvcache import kitty as kmod
    calls = []

    def rec_k(key_states, t_offset, pages, page_table, page_offset, cache, meta, page_size, d_boost, **kw):
        calls.append(("k", tuple(key_states.shape), t_offset, pages, page_offset, page_size, d_boost))

    def rec_v(value_states, t_offset, pages, page_table, page_offset, cache, meta, page_size, **kw):
        calls.append(("v", tuple(value_states.shape), t_offset, pages, page_offset, page_size))

    monkeypatch.setattr(kmod, "quantize_pack_k", rec_k)
    monkeypatch.setattr(kmod, "quantize_pack_v", rec_v)
    cfg = types.SimpleNamespace(num_hidden_layers=2, head_dim=128, num_key_value_heads=2, num_attention_heads=8,
                                hidden_size=1024)
    return kitty_amd.KittyCache(cfg, 2, 1024, device="cpu"), calls


def test_plugin_constants_and_layout(cpu_cache):
    cache, _ = cpu_cache
    L = cache.kv_cache[1]
    assert (cache.page_size, cache.d_boosted, cache.sink_length, cache.low_bit, cache.high_bit) == (128, 32, 32, 2, 4)
    assert cache.is_compileable is False and len(cache.kv_cache) == 2
    assert L.MAX_PAGE == 8 and L.bytes_per_page_K == 2 * 5248 and L.bytes_per_page_V == 2 * 4096
    assert tuple(L.KeyCache.shape) == (16, 10496) and L.KeyCache.dtype == torch.uint8
    assert tuple(L.KeyCache_metadata.shape) == (16, 2, 128, 2) and L.KeyCache_metadata.dtype == torch.float16
    assert tuple(L.ValueCache_metadata.shape) == (16, 2, 128, 2)
    assert tuple(L.Sink_Buffer_K.shape) == (2, 2, 32, 128) and tuple(L.Local_Buffer_V.shape) == (2, 2, 128, 128)
    ident = torch.arange(8).view(1, -1) + torch.arange(2).view(-1, 1) * 8
    assert torch.equal(L.PageTable_K, ident) and torch.equal(L.PageTable_V, ident)
    d = L.descriptor()
    assert (d.H_KV, d.D, d.D_BOOSTED, d.PAGE_SIZE, d.S, d.MAX_PAGE) == (2, 128, 32, 128, 32, 8)
    assert d.key_cache_stride_page == 10496 and d.key_meta_stride_page == 2 * 128 * 2 * 2
    assert d.sink_stride_h == 32 * 128 * 2 and d.win_stride_b == 2 * 128 * 128 * 2


def test_plugin_state_machine_follows_the_oracle(cpu_cache):
    cache, calls = cpu_cache
    T0, steps = 300, 300
    k, v = make_kv(2, 2, T0 + steps, seed=5)
    kt, vt = torch.from_numpy(k), torch.from_numpy(v)
    ol = O.OracleLayer(2, 1024, 2)
    assert cache.update(kt[:, :, :T0], vt[:, :, :T0], 1) is True and ol.update(k[:, :, :T0], v[:, :, :T0]) is True
    cache.quantize_prefill(1)
    ol.quantize_prefill()
    assert calls == [("k", (2, 2, T0, 128), 32, 2, 0, 128, 32), ("v", (2, 2, T0, 128), 32, 1, 0, 128)]
    calls.clear()
    L = cache.kv_cache[1]
    fields = ("Sink_Count", "PageCount_K", "PageCount_V", "Q_Buffer_Count_K", "Q_Buffer_Count_V", "Local_Count_V",
              "Write_Offset_Local_V")
    for s in range(steps):
        t = T0 + s
        assert cache.update(kt[:, :, t:t + 1], vt[:, :, t:t + 1], 1) is False
        ol.update(k[:, :, t:t + 1], v[:, :, t:t + 1])
        cache.quantize_decode(1)
        ol.quantize_decode()
        assert [getattr(L, f) for f in fields] == [getattr(ol, f) for f in fields], f"step {s}"
        assert cache.get_seq_length(1) == t + 1
    for name in ("Sink_Buffer_K", "Sink_Buffer_V", "Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V"):
        assert np.array_equal(getattr(L, name).numpy().view(np.uint16), getattr(ol, name).view(np.uint16)), name
    # every flush quantizes exactly one page of the Q-buffer into the next page slot
    ks = [c for c in calls if c[0] == "k"]
    vs = [c for c in calls if c[0] == "v"]
    assert [c[4] for c in ks] == list(range(2, 2 + len(ks))) and all(c[1:4] == ((2, 2, 128, 128), 0, 1) for c in ks)
    assert [c[4] for c in vs] == list(range(1, 1 + len(vs))) and len(ks) == ol.PageCount_K - 2
    assert cache.get_seq_length(0) == 0                          # the other layer is untouched


def test_plugin_error_paths(cpu_cache):
    cache, _ = cpu_cache
    with pytest.raises(ValueError):
        cache.quantize_prefill(0)
    k = torch.zeros(2, 2, 40, 128, dtype=torch.float16)
    cache.update(k, k, 0)
    cache.quantize_prefill(0)
    with pytest.raises(AssertionError):
        cache.update(k[:, :, :2], k[:, :, :2], 0)
    big = torch.zeros(2, 2, 32 + 128 * 9, 128, dtype=torch.float16)
    cache.update(big, big, 1)
    with pytest.raises(ValueError):
        cache.quantize_prefill(1)                                # exceeds max_length


def test_no_cpu_fallback():
    from kitty_amd.kvcache.kernels import kitty_attention_forward, quantize_pack_k, quantize_pack_v
    x = torch.zeros(1, 1, 128, 128, dtype=torch.float16)
    pt = torch.zeros(1, 1, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="no CPU path"):
        quantize_pack_k(x, 0, 1, pt, 0, torch.zeros(1, 5248, dtype=torch.uint8), torch.zeros(1, 1, 128, 2, dtype=torch.float16), 128, 32)
    with pytest.raises(RuntimeError, match="no CPU path"):
        quantize_pack_v(x, 0, 1, pt, 0, torch.zeros(1, 4096, dtype=torch.uint8), torch.zeros(1, 1, 128, 2, dtype=torch.float16), 128)
    import kitty_amd
    cfg = types.SimpleNamespace(num_hidden_layers=1, head_dim=128, num_key_value_heads=1, num_attention_heads=4, hidden_size=512)
    cache = kitty_amd.KittyCache(cfg, 1, 256, device="cpu")
    mod = types.SimpleNamespace(num_attention_heads=4, num_key_value_heads=1)
    with pytest.raises(RuntimeError, match="no CPU path"):
        kitty_attention_forward(mod, torch.zeros(1, 4, 1, 128, dtype=torch.float16), cache.kv_cache[0], 0.1)


# ---------------------------------------------------------------------------------------------
# multi-token append: the host logic against T single steps, quantizers played by the oracle
# ---------------------------------------------------------------------------------------------
@pytest.fixture()
def cpu_cache_oracle_quant(monkeypatch):
    import kitty_amd
    from kitty_amd.kvcache import kitty as kmod

    def qk(key_states, t_offset, pages, page_table, page_offset, cache, meta, page_size, d_boost, **kw):
        O.quantize_pack_k(key_states.numpy(), t_offset, pages, page_table.numpy(), page_offset, cache.numpy(),
                          meta.numpy(), page_size, d_boost)

    def qv(value_states, t_offset, pages, page_table, page_offset, cache, meta, page_size, **kw):
        O.quantize_pack_v(value_states.numpy(), t_offset, pages, page_table.numpy(), page_offset, cache.numpy(),
                          meta.numpy(), page_size)

    monkeypatch.setattr(kmod, "quantize_pack_k", qk)
    monkeypatch.setattr(kmod, "quantize_pack_v", qv)
    cfg = types.SimpleNamespace(num_hidden_layers=1, head_dim=128, num_key_value_heads=1, num_attention_heads=4,
                                hidden_size=512)
    return lambda max_len: kitty_amd.KittyCache(cfg, 1, max_len, device="cpu")


def _same_state(L, ol):
    fields = ("Sink_Count", "PageCount_K", "PageCount_V", "Q_Buffer_Count_K", "Q_Buffer_Count_V", "Local_Count_V",
              "Write_Offset_Local_V")
    assert [getattr(L, f) for f in fields] == [getattr(ol, f) for f in fields]
    u16 = lambda a: a.view(np.uint16)
    for name in ("KeyCache", "ValueCache"):
        assert np.array_equal(getattr(L, name).numpy(), getattr(ol, name)), name
    for name in ("KeyCache_metadata", "ValueCache_metadata", "Sink_Buffer_K", "Sink_Buffer_V", "Local_Buffer_V"):
        assert np.array_equal(u16(getattr(L, name).numpy()), u16(getattr(ol, name))), name
    # rows past the fill count of a Q-buffer are stale and may differ
    for name, cnt in (("Q_Buffer_K", ol.Q_Buffer_Count_K), ("Q_Buffer_V", ol.Q_Buffer_Count_V)):
        assert np.array_equal(u16(getattr(L, name).numpy()[:, :, :cnt]), u16(getattr(ol, name)[:, :, :cnt])), name


@pytest.mark.parametrize("T0,chunks", [
    (5, [1, 3, 30, 200]),                 # sink still filling, chunk straddles sink / ring / Q-buffers
    (32, [128, 1, 127, 129]),             # exactly the sink
    (100, [60, 60, 300]),                 # ring fills, then evicts
    (300, [7, 512, 5]),                   # pages straight from the chunk
    (32 + 128 * 2 + 96, [32, 256]),       # a flush exactly at the end of a chunk
    (0, [50, 500]),                       # empty layer: the first chunk is a prefill
    (417, [1] * 5 + [250]),
])
def test_append_equals_single_steps(cpu_cache_oracle_quant, T0, chunks):
    max_len = 2048
    cache = cpu_cache_oracle_quant(max_len)
    ol = O.OracleLayer(1, max_len, 1)
    k, v = make_kv(1, 1, T0 + sum(chunks), seed=T0 + len(chunks))
    kt, vt = torch.from_numpy(k), torch.from_numpy(v)
    if T0:
        cache.update(kt[:, :, :T0], vt[:, :, :T0], 0)
        cache.quantize_prefill(0)
        ol.update(k[:, :, :T0], v[:, :, :T0])
        ol.quantize_prefill()
    t = T0
    for c in chunks:
        cache.append(kt[:, :, t:t + c], vt[:, :, t:t + c], 0)
        ol.append(k[:, :, t:t + c], v[:, :, t:t + c])
        t += c
        assert cache.get_seq_length(0) == t
        _same_state(cache.kv_cache[0], ol)


def test_append_rejects_overflow_without_side_effects(cpu_cache_oracle_quant):
    cache = cpu_cache_oracle_quant(512)
    k, v = make_kv(1, 1, 1000, seed=2)
    kt, vt = torch.from_numpy(k), torch.from_numpy(v)
    cache.append(kt[:, :, :300], vt[:, :, :300], 0)
    before = cache.get_seq_length(0)
    with pytest.raises(ValueError):
        cache.append(kt[:, :, 300:], vt[:, :, 300:], 0)
    assert cache.get_seq_length(0) == before
    with pytest.raises(ValueError):
        cache.append(kt[:, :, :3], vt[:, :, :4], 0)


# ---------------------------------------------------------------------------------------------
# device-counter mode: the host shadow of the longest sequence
# ---------------------------------------------------------------------------------------------
def test_host_shadow_counters_follow_the_oracle():
    """KVCache_Layer.step_host_counters + the flush bookkeeping advance the host ints exactly as
    the oracle's update / quantize_decode do, from every phase of the state machine."""
    from kitty_amd.kvcache.utils_kv_per_layer import KVCache_Layer
    for T0 in (3, 32, 100, 32 + 128 + 5, 32 + 3 * 128):
        k, v = make_kv(1, 1, T0 + 1, seed=T0)
        ol = O.OracleLayer(1, 4096, 1)
        ol.update(k[:, :, :T0], v[:, :, :T0])
        ol.quantize_prefill()
        L = KVCache_Layer(1, 4096, 1, 128, 32, 2, 4, 128, 32, device="cpu")
        for f in KVCache_Layer.COUNT_FIELDS:
            setattr(L, f, getattr(ol, f))
        tok = (k[:, :, T0:T0 + 1], v[:, :, T0:T0 + 1])
        for _ in range(700):
            ol.update(*tok)
            L.step_host_counters()
            assert L.counts()[:7] == [getattr(ol, f) for f in KVCache_Layer.COUNT_FIELDS]
            ol.quantize_decode()
            for cnt, pages in (("Q_Buffer_Count_K", "PageCount_K"), ("Q_Buffer_Count_V", "PageCount_V")):
                if getattr(L, cnt) == 128:          # what KittyCache._flush_full_device does on the host
                    setattr(L, pages, getattr(L, pages) + 1)
                    setattr(L, cnt, 0)
            assert L.counts()[:7] == [getattr(ol, f) for f in KVCache_Layer.COUNT_FIELDS]
        assert L.get_total_length() == T0 + 700


def test_enable_device_counters_validates_and_shadows_the_longest():
    from kitty_amd.kvcache.utils_kv_per_layer import KVCache_Layer
    L = KVCache_Layer(3, 1024, 1, 128, 32, 2, 4, 128, 32, device="cpu")
    rows = [[32, 1, 7, 0, 7, 128, 7, 0], [20, 0, 0, 0, 0, 0, 0, 0], [32, 2, 100, 1, 100, 128, 3, 0]]
    sc = L.enable_device_counters(torch.tensor(rows, dtype=torch.int32))
    assert L.device_counters and sc.dtype == torch.int32 and sc.tolist() == rows
    assert L.counts() == rows[2] and L.get_total_length() == 32 + 2 * 128 + 100
    for bad in ([[33, 0, 0, 0, 0, 0, 0, 0]] * 3, [[32, 0, 129, 0, 1, 128, 0, 0]] * 3, [[32, 0, 5, 0, 0, 4, 0, 0]] * 3,
                [[32, 9, 0, 9, 0, 0, 0, 0]] * 3, [[32, 0, 1, 0, 0, 1, 128, 0]] * 3, [[-1, 0, 0, 0, 0, 0, 0, 0]] * 3):
        with pytest.raises(ValueError):
            L.enable_device_counters(torch.tensor(bad, dtype=torch.int32))
    with pytest.raises(ValueError):
        L.enable_device_counters(torch.zeros(2, 8, dtype=torch.int32))
    M = KVCache_Layer(2, 1024, 1, 128, 32, 2, 4, 128, 32, device="cpu")
    M.Sink_Count, M.Q_Buffer_Count_K, M.Local_Count_V = 32, 9, 9
    assert M.enable_device_counters().tolist() == [[32, 0, 9, 0, 0, 9, 0, 0]] * 2
