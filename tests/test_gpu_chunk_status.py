"""GPU parity of the multi-token append with per-sequence counters on the device
(kitty_append_chunk through KittyCache.append / PagedKittyCache.append), of the rotary embedding
fused into the decode-step append, and of the device-side status words, against the CPU oracle
stepping every sequence on its own.  Everything here is bit-exact."""
import numpy as np
import pytest
import torch

from oracle import kitty_oracle as O
from tests.helpers import make_kv, make_q

pytestmark = pytest.mark.gpu
ATOL = 2e-3
FIELDS = ("Sink_Count", "PageCount_K", "Q_Buffer_Count_K", "PageCount_V", "Q_Buffer_Count_V", "Local_Count_V",
          "Write_Offset_Local_V")


@pytest.fixture(scope="module")
def K():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import kitty_amd
    from kitty_amd import _lib
    _lib.lib()                                   # raises if the HIP library is not built
    from kitty_amd.kvcache.kernels import kitty_attention_forward, kitty_prefill_attention
    from tests import gpu_util
    return type("NS", (), dict(KittyCache=kitty_amd.KittyCache, Paged=kitty_amd.PagedKittyCache,
                               OutOfPages=kitty_amd.OutOfPages, attn=kitty_attention_forward,
                               chunk_attn=kitty_prefill_attention, u=gpu_util, lib=_lib))


def _counts(ol):
    return [getattr(ol, f) for f in FIELDS] + [0]


def _load_row(K, L, b, ol):
    """Copy a batch-1 oracle layer into row b of a device layer with the identity page table."""
    for name in ("Sink_Buffer_K", "Sink_Buffer_V", "Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V"):
        getattr(L, name)[b].copy_(K.u.to_dev(getattr(ol, name)[0]))
    for name in ("KeyCache", "KeyCache_metadata", "ValueCache", "ValueCache_metadata"):
        getattr(L, name)[b * L.MAX_PAGE:(b + 1) * L.MAX_PAGE].copy_(K.u.to_dev(getattr(ol, name)))


def _bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint16) if a.dtype == np.float16 else a


def _state_mismatches(L, b, ol, counts_row, pages_k=None, pages_v=None):
    """Row b of a device layer against a batch-1 oracle layer: counters, sink, ring, the live rows
    of the Q-buffers (rows past the fill count are not state) and the packed pages.  ``pages_k`` /
    ``pages_v``: the device page ids of the sequence's pages in order (default: the identity table)."""
    bad = []

    def cmp(name, t, a):
        got = _bits(t.detach().cpu().numpy())
        if not np.array_equal(got, _bits(a)):
            bad.append((name, int((got != _bits(a)).sum())))

    if list(counts_row[:7]) != _counts(ol)[:7]:
        return [("seq_counts", list(counts_row), _counts(ol))]
    cmp("Sink_Buffer_K", L.Sink_Buffer_K[b], ol.Sink_Buffer_K[0])
    cmp("Sink_Buffer_V", L.Sink_Buffer_V[b], ol.Sink_Buffer_V[0])
    cmp("Local_Buffer_V", L.Local_Buffer_V[b], ol.Local_Buffer_V[0])
    cmp("Q_Buffer_K", L.Q_Buffer_K[b, :, :ol.Q_Buffer_Count_K], ol.Q_Buffer_K[0, :, :ol.Q_Buffer_Count_K])
    cmp("Q_Buffer_V", L.Q_Buffer_V[b, :, :ol.Q_Buffer_Count_V], ol.Q_Buffer_V[0, :, :ol.Q_Buffer_Count_V])
    if pages_k is None:
        pages_k = list(range(b * L.MAX_PAGE, b * L.MAX_PAGE + ol.PageCount_K))
        pages_v = list(range(b * L.MAX_PAGE, b * L.MAX_PAGE + ol.PageCount_V))
    pk, pv = torch.as_tensor(pages_k, dtype=torch.long), torch.as_tensor(pages_v, dtype=torch.long)
    cmp("KeyCache", L.KeyCache[pk.to(L.device)], ol.KeyCache[:ol.PageCount_K])
    cmp("KeyCache_metadata", L.KeyCache_metadata[pk.to(L.device)], ol.KeyCache_metadata[:ol.PageCount_K])
    cmp("ValueCache", L.ValueCache[pv.to(L.device)], ol.ValueCache[:ol.PageCount_V])
    cmp("ValueCache_metadata", L.ValueCache_metadata[pv.to(L.device)], ol.ValueCache_metadata[:ol.PageCount_V])
    return bad


# starting lengths that put a sequence in every phase: sink filling, ring filling, ring full, and
# (through the decode steps that follow the prefill) a ring whose head has moved
STARTS = [5, 31, 32, 40, 32 + 127, 32 + 128, 32 + 255, 32 + 128 * 3 + 77]


def _ragged(K, H_KV, H_Q, max_len, extra, seed, warm_steps=0):
    """A device cache and per-sequence oracles in the states of STARTS, ``warm_steps`` single decode
    steps later (so that rings have wrapped), plus ``extra`` more tokens per sequence to append."""
    B = len(STARTS)
    cache = K.KittyCache(K.u.cfg(H_KV, H_Q), B, max_len)
    L = cache.kv_cache[0]
    ols, kvs = [], []
    for b, T in enumerate(STARTS):
        k, v = make_kv(1, H_KV, T + warm_steps + extra, seed=seed + b)
        ol = O.OracleLayer(1, max_len, H_KV)
        ol.update(k[:, :, :T], v[:, :, :T])
        ol.quantize_prefill()
        for s in range(warm_steps):
            ol.update(k[:, :, T + s:T + s + 1], v[:, :, T + s:T + s + 1])
            ol.quantize_decode()
        _load_row(K, L, b, ol)
        ols.append(ol)
        kvs.append((k, v, T + warm_steps))
    cache.enable_device_counters(torch.tensor([_counts(ol) for ol in ols], dtype=torch.int32))
    return cache, L, ols, kvs


def _chunk(kvs, lo, hi):
    kn = np.concatenate([k[:, :, T + lo:T + hi] for k, v, T in kvs], axis=0)
    vn = np.concatenate([v[:, :, T + lo:T + hi] for k, v, T in kvs], axis=0)
    return kn, vn


@pytest.mark.parametrize("chunks", [(1,), (7, 1), (96, 33), (128,), (129, 127), (300,), (13, 700)])
@pytest.mark.parametrize("warm", [0, 150])
def test_chunk_append_with_device_counters_equals_single_steps(K, chunks, warm):
    H_KV, H_Q = 2, 8
    max_len = 32 + 128 * 14
    cache, L, ols, kvs = _ragged(K, H_KV, H_Q, max_len, sum(chunks) + 1, seed=300 + 7 * len(chunks), warm_steps=warm)
    done = 0
    for T in chunks:
        kn, vn = _chunk(kvs, done, done + T)
        cache.append(K.u.to_dev(kn), K.u.to_dev(vn), 0)
        for b, ol in enumerate(ols):
            ol.append(kn[b:b + 1], vn[b:b + 1])
        done += T
        got = L.seq_counts.cpu().numpy()
        for b, ol in enumerate(ols):
            assert _state_mismatches(L, b, ol, got[b]) == [], f"chunk {T}, row {b} (start {STARTS[b]} + {warm})"
        assert L.get_total_length() == max(STARTS) + warm + done
    assert not L.status.any()
    # the state is good for what follows: one more decode step, attention against the oracle
    kn, vn = _chunk(kvs, done, done + 1)
    assert cache.update(K.u.to_dev(kn), K.u.to_dev(vn), 0) is False
    q = make_q(len(STARTS), H_Q, seed=done)
    out, _ = K.attn(K.u.module(H_KV, H_Q), K.u.to_dev(q), L, 128 ** -0.5, variant=1)
    gotq = out.detach().cpu().numpy().astype(np.float64)
    for b, ol in enumerate(ols):
        ol.update(kn[b:b + 1], vn[b:b + 1])
        want = O.decode_attention(ol, q[b:b + 1], 128 ** -0.5, reference_rounding=False)
        assert np.abs(gotq[b:b + 1] - want).max() <= ATOL, b
    cache.check_status()


def test_chunk_append_through_a_strided_view(K):
    """The chunk is read through its strides: a slice of a longer tensor is not copied first."""
    H_KV, H_Q, T = 2, 8, 200
    cache, L, ols, kvs = _ragged(K, H_KV, H_Q, 32 + 128 * 8, T, seed=41)
    kn, vn = _chunk(kvs, 0, T)
    pad_k = torch.full((len(STARTS), H_KV, T + 64, 128), 9.0, dtype=torch.float16, device="cuda")
    pad_v = pad_k.clone()
    pad_k[:, :, 40:40 + T] = K.u.to_dev(kn)
    pad_v[:, :, 40:40 + T] = K.u.to_dev(vn)
    cache.append(pad_k[:, :, 40:40 + T], pad_v[:, :, 40:40 + T], 0)
    got = L.seq_counts.cpu().numpy()
    for b, ol in enumerate(ols):
        ol.append(kn[b:b + 1], vn[b:b + 1])
        assert _state_mismatches(L, b, ol, got[b]) == [], b


def test_chunk_that_does_not_fit_leaves_the_sequence_alone_and_says_so(K):
    """Row 0 has room, row 1 would pass MAX_PAGE, row 2 lacks a page (-1 in its table), row 3 is
    inactive: only row 0 changes; the others keep every byte and the status rows say why."""
    H_KV, H_Q, T = 1, 4, 300
    max_len = 32 + 128 * 4                      # MAX_PAGE = 5 (ceil of 544 / 128)
    c = K.KittyCache(K.u.cfg(H_KV, H_Q), 4, max_len)
    L = c.kv_cache[0]
    rows = [[32, 1, 10, 0, 10, 128, 0, 0], [32, 4, 100, 3, 100, 128, 0, 0], [32, 1, 10, 0, 10, 128, 0, 0],
            [32, 1, 10, 0, 10, 128, 0, 1]]
    L.enable_device_counters(torch.tensor(rows, dtype=torch.int32))
    L.PageTable_K[2, 2] = -1
    k = torch.randn(4, H_KV, T, 128, device="cuda").half()
    names = ("KeyCache", "ValueCache", "KeyCache_metadata", "ValueCache_metadata", "Q_Buffer_K", "Q_Buffer_V",
             "Local_Buffer_V", "Sink_Buffer_K")
    before = {n: getattr(L, n).clone() for n in names}
    rc = K.lib.lib().kitty_append_chunk(L.descriptor(), k.data_ptr(), k.data_ptr(), k.stride(0) * 2, k.stride(1) * 2,
                                        k.stride(2) * 2, 4, T, K.lib.current_stream_ptr(k.device))
    assert rc == 0
    torch.cuda.synchronize()
    got = L.seq_counts.cpu().tolist()
    assert got[1:] == rows[1:]
    assert got[0] == [32, 1 + (10 + T) // 128, (10 + T) % 128, (10 + T) // 128, (10 + T) % 128, 128, T % 128, 0]
    MP = L.MAX_PAGE
    for n in ("KeyCache", "ValueCache", "KeyCache_metadata", "ValueCache_metadata"):
        assert torch.equal(getattr(L, n)[MP:], before[n][MP:]), n          # the pages of rows 1..3
    for n in ("Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V", "Sink_Buffer_K"):
        assert torch.equal(getattr(L, n)[1:], before[n][1:]), n
    assert L.status.cpu().tolist() == [[0, 0, 0, 0], [T, 0, 0, 0], [T, 0, 0, 0], [0, 0, 0, 0]]
    with pytest.raises(RuntimeError, match="tokens_dropped"):
        c.check_status()
    st = c.check_status(raise_on_error=False, clear=True)
    assert st["tokens_dropped"].tolist() == [[0, T, T, 0]] and not L.status.any()


def test_status_words_of_the_decode_step(K):
    """A flush that finds no page is skipped and counted, the tokens that follow are dropped and
    counted, a page id outside the cache is never written to, and nothing else changes."""
    H_KV, H_Q = 1, 4
    c = K.KittyCache(K.u.cfg(H_KV, H_Q), 3, 32 + 128 * 4)
    L = c.kv_cache[0]
    L.enable_device_counters(torch.tensor([[32, 1, 127, 0, 127, 128, 0, 0]] * 3, dtype=torch.int32))
    L.PageTable_K[1, 1] = -1                     # sequence 1: no page for its K flush
    L.PageTable_V[2, 0] = 10 ** 9                # sequence 2: a page id far outside the cache
    k = torch.randn(3, H_KV, 1, 128, device="cuda").half()
    kc, vc = L.KeyCache.clone(), L.ValueCache.clone()
    for step in range(3):
        c._launch_append(L, k, k)
        c._launch_flush(L)
    torch.cuda.synchronize()
    MP = L.MAX_PAGE
    assert L.seq_counts.cpu().tolist() == [[32, 2, 2, 1, 2, 128, 3, 0], [32, 1, 128, 1, 0, 128, 1, 0],
                                           [32, 2, 0, 0, 128, 128, 1, 0]]
    assert torch.equal(L.KeyCache[MP:2 * MP], kc[MP:2 * MP]) and not torch.equal(L.KeyCache[1], kc[1])
    assert torch.equal(L.ValueCache[2 * MP:], vc[2 * MP:]) and torch.equal(L.ValueCache[MP + 1:2 * MP], vc[MP + 1:2 * MP])
    # sequence 1: K flush skipped on each of the three steps, the two later tokens dropped;
    # sequence 2: the same on the V side, and the bad id recorded
    assert L.status.cpu().tolist() == [[0, 0, 0, 0], [2, 3, 0, 0], [2, 3, 1, 0]]
    st = c.check_status(raise_on_error=False)
    assert st["flush_skipped"].tolist() == [[0, 3, 3]] and st["bad_page_write"].tolist() == [[0, 0, 1]]
    # the page arrives: the next flush goes through and the sequence takes tokens again
    L.PageTable_K[1, 1] = MP + 1
    c._launch_flush(L)
    c._launch_append(L, k, k)
    torch.cuda.synchronize()
    assert L.seq_counts[1].cpu().tolist() == [32, 2, 1, 1, 1, 128, 2, 0]
    assert not torch.equal(L.KeyCache[MP + 1], kc[MP + 1])


def test_quantizer_records_a_page_id_outside_the_cache(K):
    from kitty_amd.kvcache.kernels import quantize_pack_k, quantize_pack_v
    x = torch.randn(2, 1, 256, 128, device="cuda").half()
    pt = torch.tensor([[0, 1], [2, 77]], dtype=torch.int64, device="cuda")
    lay = O.Layout(H_KV=1)
    kc = torch.zeros(4, lay.bytes_per_page_K, dtype=torch.uint8, device="cuda")
    km = torch.zeros(4, 1, 128, 2, dtype=torch.float16, device="cuda")
    vc = torch.zeros(4, lay.bytes_per_page_V, dtype=torch.uint8, device="cuda")
    vm = torch.zeros(4, 1, 128, 2, dtype=torch.float16, device="cuda")
    st = torch.zeros(2, 4, dtype=torch.int32, device="cuda")
    quantize_pack_k(x, 0, 2, pt, 0, kc, km, 128, 32, status=st)
    quantize_pack_v(x, 0, 2, pt, 0, vc, vm, 128, status=st)
    torch.cuda.synchronize()
    assert st.cpu().tolist() == [[0, 0, 0, 0], [0, 0, 1, 0]]
    assert kc[:3].any(1).all() and not kc[3].any() and vc[:3].any(1).all() and not vc[3].any()


@pytest.mark.parametrize("variant", [0, 1])
def test_attention_reads_page_zero_for_a_page_id_outside_the_cache(K, variant):
    """A page table entry that is not a page id (-1: nothing assigned, or garbage) under counters
    that claim the page: the kernels read page 0 in its place, finish normally and raise the status
    word of that sequence; the other sequence's output is untouched by it."""
    B, H_KV, H_Q, T = 2, 2, 8, 32 + 128 * 3 + 50
    k, v = make_kv(B, H_KV, T, seed=5)
    c = K.KittyCache(K.u.cfg(H_KV, H_Q), B, 1024)
    c.update(K.u.to_dev(k), K.u.to_dev(v), 0)
    c.quantize_prefill(0)
    L = c.kv_cache[0]
    mod = K.u.module(H_KV, H_Q)
    q = K.u.to_dev(make_q(B, H_Q, seed=1))
    good, _ = K.attn(mod, q, L, 128 ** -0.5, variant=variant)
    L.PageTable_K[1, 1] = -1
    L.PageTable_V[1, 0] = L.KeyCache.shape[0] + 5
    bad, _ = K.attn(mod, q, L, 128 ** -0.5, variant=variant)
    chunk_q = torch.randn(B, H_Q, 4, 128, device="cuda").half()
    chunk_k = torch.randn(B, H_KV, 4, 128, device="cuda").half()
    K.chunk_attn(mod, chunk_q, chunk_k, chunk_k, L, 128 ** -0.5)
    torch.cuda.synchronize()
    assert torch.equal(good[0], bad[0])
    assert torch.isfinite(bad.float()).all()
    assert L.status.cpu().tolist() == [[0, 0, 0, 0], [0, 0, 0, 1]]
    # page 0 in the place of both: the same output as a table that names page 0 there
    L.PageTable_K[1, 1] = 0
    L.PageTable_V[1, 0] = 0
    L.status.zero_()
    same, _ = K.attn(mod, q, L, 128 ** -0.5, variant=variant)
    torch.cuda.synchronize()
    assert torch.equal(same, bad) and not L.status.any()


def test_rotary_embedding_fused_into_the_append(K):
    """update_with_rope on un-rotated keys leaves the bytes that rotating with fp16 tensor
    arithmetic (the oracle's rope_fp16, and torch's operators on the device) followed by update
    leaves, for sequences whose token goes to the sink, to the Q-buffer with the ring full and with
    room in the ring, and for a free slot."""
    B, H_KV, H_Q, D = 4, 2, 8, 128
    rng = np.random.default_rng(11)
    k = (rng.standard_normal((B, H_KV, 1, D)) * 3).astype(np.float16)
    v = rng.standard_normal((B, H_KV, 1, D)).astype(np.float16)
    pos = np.array([7, 5000, 31999, 100], dtype=np.float64)
    inv = 1.0 / (500000.0 ** (np.arange(0, D, 2) / D))
    ang = pos[:, None] * inv[None, :]
    cos = np.concatenate([np.cos(ang), np.cos(ang)], -1).astype(np.float16)[:, None, :]      # [B, 1, D]
    sin = np.concatenate([np.sin(ang), np.sin(ang)], -1).astype(np.float16)[:, None, :]
    want = O.rope_fp16(k, cos, sin)
    kd, cd, sd = K.u.to_dev(k), K.u.to_dev(cos), K.u.to_dev(sin)
    x1, x2 = kd[..., :D // 2], kd[..., D // 2:]
    on_device = kd * cd.unsqueeze(1) + torch.cat((-x2, x1), dim=-1) * sd.unsqueeze(1)
    assert np.array_equal(on_device.cpu().numpy().view(np.uint16), want.view(np.uint16))
    rows = [[10, 0, 0, 0, 0, 0, 0, 0], [32, 1, 5, 0, 5, 128, 0, 0], [32, 0, 100, 0, 0, 100, 0, 0], [32, 1, 5, 0, 5, 128, 0, 1]]
    caches = []
    for fused in (True, False):
        c = K.KittyCache(K.u.cfg(H_KV, H_Q), B, 1024)
        c.enable_device_counters(torch.tensor(rows, dtype=torch.int32))
        if fused:
            assert c.update_with_rope(kd, K.u.to_dev(v), cd, sd, 0) is False
        else:
            c.update(K.u.to_dev(want), K.u.to_dev(v), 0)
        caches.append(c.kv_cache[0])
    a, b = caches
    torch.cuda.synchronize()
    for n in ("Sink_Buffer_K", "Sink_Buffer_V", "Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V"):
        assert torch.equal(getattr(a, n).view(torch.int16), getattr(b, n).view(torch.int16)), n
    assert torch.equal(a.seq_counts, b.seq_counts) and torch.equal(a.status, b.status)
    assert np.array_equal(a.Sink_Buffer_K[0, :, 10].cpu().numpy().view(np.uint16), want[0, :, 0].view(np.uint16))
    assert np.array_equal(a.Q_Buffer_K[1, :, 5].cpu().numpy().view(np.uint16), want[1, :, 0].view(np.uint16))
    assert np.array_equal(a.Q_Buffer_K[2, :, 100].cpu().numpy().view(np.uint16), want[2, :, 0].view(np.uint16))
    assert a.seq_counts.cpu().tolist() == [[11, 0, 0, 0, 0, 0, 0, 0], [32, 1, 6, 0, 6, 128, 1, 0],
                                           [32, 0, 101, 0, 0, 101, 0, 0], rows[3]]
    assert not a.status.any()
    # a full Q-buffer drops the rotated token like any other
    c = K.KittyCache(K.u.cfg(H_KV, H_Q), B, 1024)
    L = c.kv_cache[0]
    L.enable_device_counters(torch.tensor([[32, 0, 128, 0, 0, 128, 0, 0]] * B, dtype=torch.int32))
    c._launch_append(L, kd, K.u.to_dev(v), [cd.reshape(-1, D), sd.reshape(-1, D)])
    torch.cuda.synchronize()
    assert L.status.cpu().tolist() == [[1, 0, 0, 0]] * B and not L.Q_Buffer_K.any()
    with pytest.raises(ValueError):
        K.KittyCache(K.u.cfg(H_KV, H_Q), B, 1024).update_with_rope(kd, kd, cd, sd, 0)     # host counters


def test_paged_chunk_append_and_chunk_attention_per_sequence(K):
    """Slots of a page pool holding sequences of different lengths (one slot free) take a chunk
    each: chunk attention over the packed cache, then the append; every sequence ends up, page for
    page, where the oracle's single steps put it, and the pool's books balance."""
    H_KV, H_Q, slots, Tq = 2, 8, 4, 150
    max_len, pool_pages = 32 + 128 * 10, 40
    cache = K.Paged(K.u.cfg(H_KV, H_Q, layers=2), slots, max_len, pool_pages)
    lens = {0: 32 + 128 * 2 + 60, 1: 20, 3: 32 + 128 + 127}
    ols, kvs = {}, {}
    for slot, T in lens.items():
        k, v = make_kv(1, H_KV, T + Tq, seed=700 + slot)
        with cache.admitting(slot):
            for li in range(2):
                assert cache.update(K.u.to_dev(k[:, :, :T]), K.u.to_dev(v[:, :, :T]), li) is True
                cache.quantize_prefill(li)
        ol = O.OracleLayer(1, max_len, H_KV)
        ol.update(k[:, :, :T], v[:, :, :T])
        ol.quantize_prefill()
        ols[slot], kvs[slot] = ol, (k, v, T)
    kn = np.zeros((slots, H_KV, Tq, 128), np.float16)
    vn = np.zeros_like(kn)
    for slot, (k, v, T) in kvs.items():
        kn[slot], vn[slot] = k[0, :, T:], v[0, :, T:]
    q = np.random.default_rng(3).standard_normal((slots, H_Q, Tq, 128)).astype(np.float16)
    mod = K.u.module(H_KV, H_Q)
    kd, vd = K.u.to_dev(kn), K.u.to_dev(vn)
    free_before = (cache.pool_k.free, cache.pool_v.free)
    for li in range(2):
        out, _ = K.chunk_attn(mod, K.u.to_dev(q), kd, vd, cache.kv_cache[li], 128 ** -0.5)
        cache.append(kd, vd, li)
        got = out.detach().cpu().numpy().astype(np.float64)
        for slot, ol in ols.items():
            want = O.chunk_attention(ol, q[slot:slot + 1], kn[slot:slot + 1], vn[slot:slot + 1], 128 ** -0.5)
            assert np.abs(got[slot:slot + 1] - want).max() <= ATOL, (li, slot)
        assert not got[2].any()                  # the free slot holds nothing, and its chunk is all zeros
    torch.cuda.synchronize()
    cache.check_tables()
    cache.check_status()
    for slot, ol in ols.items():
        ol.append(kn[slot:slot + 1], vn[slot:slot + 1])
    tk, tv = cache.PageTable_K.cpu().numpy(), cache.PageTable_V.cpu().numpy()
    for li in range(2):
        L = cache.kv_cache[li]
        counts = L.seq_counts.cpu().numpy()
        for slot, ol in ols.items():
            assert _state_mismatches(L, slot, ol, counts[slot], tk[slot, :ol.PageCount_K], tv[slot, :ol.PageCount_V]) == [], \
                (li, slot)
        assert counts[2].tolist() == [0, 0, 0, 0, 0, 0, 0, 1]
    assert cache.seq_lengths().tolist() == [lens[0] + Tq, lens[1] + Tq, 0, lens[3] + Tq]
    assert cache.pool_k.free < free_before[0] and cache.pool_v.free < free_before[1]
    # a chunk the pool cannot hold is refused before anything changes
    big = torch.zeros(slots, H_KV, 128 * 9, 128, dtype=torch.float16, device="cuda")
    state = (cache.pool_k.free, cache.pool_v.free, cache.seq_counts.clone(), cache.PageTable_K.clone())
    with pytest.raises((K.OutOfPages, ValueError)):
        cache.append(big, big, 0)
    assert (cache.pool_k.free, cache.pool_v.free) == state[:2]
    assert torch.equal(cache.seq_counts, state[2]) and torch.equal(cache.PageTable_K, state[3])
    # and decoding goes on from the appended state
    step_k = torch.randn(slots, H_KV, 1, 128, device="cuda").half()
    for li in range(2):
        assert cache.update(step_k, step_k, li) is False
        cache.quantize_decode(li)
    assert cache.seq_lengths().tolist() == [lens[0] + Tq + 1, lens[1] + Tq + 1, 0, lens[3] + Tq + 1]
    with pytest.raises(ValueError, match="all 4 slots"):
        cache.update(step_k[:2], step_k[:2], 0)
