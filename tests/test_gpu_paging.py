"""GPU parity of the paged cache (kitty_amd/kvcache/paging.py): sequences are admitted to and
released from slots of a page pool while the others decode.  Every sequence is checked against a
CPU oracle layer of its own that was fed the same tokens (the reference's state machine and
quantizers, src/kitty/kvcache/kitty.py:63-236, kernels/kitty_quant_pack.py): packed pages bit for
bit through the page table, fp16 windows, counters; attention within max-abs 2e-3."""
import numpy as np
import pytest
import torch

from oracle import kitty_oracle as O
from tests.helpers import make_kv, make_q

pytestmark = pytest.mark.gpu
ATOL = 2e-3
FIELDS = ("Sink_Count", "PageCount_K", "Q_Buffer_Count_K", "PageCount_V", "Q_Buffer_Count_V", "Local_Count_V",
          "Write_Offset_Local_V")
H_KV, H_Q, LAYERS = 2, 8, 2


@pytest.fixture(scope="module")
def K():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import kitty_amd
    from kitty_amd import _lib
    _lib.lib()                                   # raises if the HIP library is not built
    from kitty_amd.kvcache.kernels import kitty_attention_forward
    from tests import gpu_util
    return type("NS", (), dict(Paged=kitty_amd.PagedKittyCache, OutOfPages=kitty_amd.OutOfPages,
                               attn=kitty_attention_forward, u=gpu_util))


class Seq:
    """One sequence: its tokens per layer and one oracle layer per model layer."""

    def __init__(self, seed, T0, total, max_len):
        self.kv = [make_kv(1, H_KV, total, seed=seed * 10 + l) for l in range(LAYERS)]
        self.T0, self.pos = T0, T0
        self.ols = [O.OracleLayer(1, max_len, H_KV) for _ in range(LAYERS)]

    def admit(self, K, cache, slot):
        with cache.admitting(slot):
            for l, (k, v) in enumerate(self.kv):
                assert cache.update(K.u.to_dev(k[:, :, :self.T0]), K.u.to_dev(v[:, :, :self.T0]), l) is True
                cache.quantize_prefill(l)
                self.ols[l].update(k[:, :, :self.T0], v[:, :, :self.T0])
                self.ols[l].quantize_prefill()

    def token(self, l):
        k, v = self.kv[l]
        return k[:, :, self.pos:self.pos + 1], v[:, :, self.pos:self.pos + 1]


def _step(K, cache, seqs, n_slots, check=None, seed=0):
    """One decode step over all slots; free slots are fed zeros.  ``check``: attention of every
    layer against the oracles, between append and flush as the model runs it."""
    mod = K.u.module(H_KV, H_Q)
    for l in range(LAYERS):
        kn = np.zeros((n_slots, H_KV, 1, 128), dtype=np.float16)
        vn = np.zeros_like(kn)
        for slot, s in seqs.items():
            kn[slot], vn[slot] = (x[0] for x in s.token(l))
        assert cache.update(K.u.to_dev(kn), K.u.to_dev(vn), l) is False
        for slot, s in seqs.items():
            s.ols[l].update(kn[slot:slot + 1], vn[slot:slot + 1])
        if check:
            q = make_q(n_slots, H_Q, seed=seed + l)
            out, _ = K.attn(mod, K.u.to_dev(q), cache.kv_cache[l], 128 ** -0.5)
            got = out.detach().cpu().numpy().astype(np.float64)
            for slot in range(n_slots):
                if slot in seqs:
                    # the matrix-core kernel evaluates code * scale + zero without the reference's
                    # intermediate fp16 rounding: it is held to the tolerance against that value
                    want = O.decode_attention(seqs[slot].ols[l], q[slot:slot + 1], 128 ** -0.5, dequant="affine",
                                              reference_rounding=False)
                    assert np.abs(got[slot:slot + 1] - want).max() <= ATOL, (check, l, slot)
                else:
                    assert not got[slot].any(), (check, l, slot)      # a free slot attends to nothing
        cache.quantize_decode(l)
        for s in seqs.values():
            s.ols[l].quantize_decode()
    for s in seqs.values():
        s.pos += 1


def _state_mismatches(cache, seqs):
    """Every active sequence, every layer: bytes and counters equal the oracle's, pages looked up
    through the (non-identity) page tables."""
    bad = []
    tk, tv = cache.PageTable_K.cpu().numpy(), cache.PageTable_V.cpu().numpy()
    counts = cache.seq_counts.cpu().numpy()

    def cmp(what, got, want):
        got = got.detach().cpu().numpy()
        if got.dtype == np.float16:
            got, want = got.view(np.uint16), np.ascontiguousarray(want).view(np.uint16)
        if not np.array_equal(got, want):
            bad.append(what)

    for slot, s in seqs.items():
        for l, ol in enumerate(s.ols):
            L = cache.kv_cache[l]
            if list(counts[l, slot]) != [getattr(ol, f) for f in FIELDS] + [0]:
                bad.append((slot, l, "counts", list(counts[l, slot])))
            for name in ("Sink_Buffer_K", "Sink_Buffer_V", "Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V"):
                cmp((slot, l, name), getattr(L, name)[slot], getattr(ol, name)[0])
            for p in range(ol.PageCount_K):
                cmp((slot, l, "KeyCache", p), L.KeyCache[tk[slot, p]], ol.KeyCache[p])
                cmp((slot, l, "KeyCache_metadata", p), L.KeyCache_metadata[tk[slot, p]], ol.KeyCache_metadata[p])
            for p in range(ol.PageCount_V):
                cmp((slot, l, "ValueCache", p), L.ValueCache[tv[slot, p]], ol.ValueCache[p])
                cmp((slot, l, "ValueCache_metadata", p), L.ValueCache_metadata[tv[slot, p]], ol.ValueCache_metadata[p])
    for slot in range(cache.n_slots):
        if slot not in seqs:
            assert list(counts[:, slot].reshape(-1)) == [0, 0, 0, 0, 0, 0, 0, 1] * LAYERS, slot
    return bad


def _expected_pages(seqs):
    pk = sum(min(s.ols[0].PageCount_K + 1, 7) for s in seqs.values())
    pv = sum(min(s.ols[0].PageCount_V + 1, 7) for s in seqs.values())
    return pk, pv


def test_sequences_come_and_go_in_a_shared_pool(K):
    """Four slots over a pool of 14 pages (the static layout would hold 28): three sequences of
    different lengths are admitted in scrambled slot order, decode across K and V flushes, one is
    released, a fourth takes over its pages, the batch decodes on."""
    n_slots, max_len, pool = 4, 32 + 128 * 6, 14
    cache = K.Paged(K.u.cfg(H_KV, H_Q, layers=LAYERS), n_slots, max_len, pool_pages=pool)
    assert cache.kv_cache[0].KeyCache.shape[0] == pool
    seqs = {}
    for slot, seed, T0 in ((2, 1, 32 + 128 * 2 + 50), (0, 2, 20), (3, 3, 32 + 128 + 127)):
        seqs[slot] = Seq(seed, T0, T0 + 300, max_len)
        seqs[slot].admit(K, cache, slot)
    cache.check_tables()
    assert cache.active_slots() == [0, 2, 3] and cache.pages_in_use() == _expected_pages(seqs)
    assert list(cache.seq_lengths()) == [20, 0, 32 + 128 * 2 + 50, 32 + 128 + 127]
    assert _state_mismatches(cache, seqs) == []
    assert cache.get_seq_length() == 32 + 128 * 2 + 50
    for step in range(140):
        _step(K, cache, seqs, n_slots, check=f"step {step}" if step in (0, 1, 77, 78, 139) else None, seed=step)
    cache.check_tables()
    assert _state_mismatches(cache, seqs) == []
    assert cache.pages_in_use() == _expected_pages(seqs)
    assert sum(s.ols[0].PageCount_K for s in seqs.values()) == 3 + 1 + 3      # every sequence flushed along the way

    before = cache.pages_in_use()
    freed = cache._table_k[2][cache._table_k[2] >= 0].tolist()
    cache.release(2)
    gone = seqs.pop(2)
    assert cache.pages_in_use() == (before[0] - gone.ols[0].PageCount_K - 1, before[1] - gone.ols[0].PageCount_V - 1)
    seqs[1] = Seq(4, 32 + 128 * 3 + 5, 32 + 128 * 3 + 5 + 200, max_len)
    seqs[1].admit(K, cache, 1)
    assert set(freed) <= set(cache._table_k[1].tolist())        # the newcomer sits in the pages just freed
    assert sorted(cache._table_k[1][:4].tolist()) != cache._table_k[1][:4].tolist()   # ... in scrambled order
    cache.check_tables()
    assert cache.get_seq_length() == max(s.pos for s in seqs.values())
    for step in range(130):
        _step(K, cache, seqs, n_slots, check=f"second phase, step {step}" if step in (0, 129) else None, seed=500 + step)
    cache.check_tables()
    assert _state_mismatches(cache, seqs) == []
    assert cache.pages_in_use() == _expected_pages(seqs)
    with pytest.raises(ValueError):
        seqs[1].admit(K, cache, 1)                               # the slot is taken
    for slot in list(seqs):
        cache.release(slot)
    cache.check_tables()
    assert cache.pages_in_use() == (0, 0) and cache.active_slots() == [] and cache.get_seq_length() == 0


def test_a_dry_pool_stalls_the_sequence_until_pages_return(K):
    """The pool runs dry when a flush needs the page after next: the step raises OutOfPages with
    the bookkeeping complete; 128 steps later the starved sequence holds its full Q-buffers and
    drops tokens, on the device exactly as in the host shadow; after another sequence is released
    it flushes and carries on."""
    n_slots, max_len = 2, 32 + 128 * 6
    cache = K.Paged(K.u.cfg(H_KV, H_Q, layers=LAYERS), n_slots, max_len, pool_pages=4)
    a, b = Seq(7, 32 + 128 + 120, 1000, max_len), Seq(8, 32 + 100, 1000, max_len)
    a.admit(K, cache, 0)            # K pages 0 + next = 2, V 1
    b.admit(K, cache, 1)            # 1 and 1
    assert cache.pages_in_use() == (3, 2)
    seqs = {0: a, 1: b}

    def step():
        for l in range(LAYERS):
            kn = np.concatenate([seqs[s].token(l)[0] if s in seqs else np.zeros((1, H_KV, 1, 128), np.float16)
                                 for s in range(n_slots)])
            vn = np.concatenate([seqs[s].token(l)[1] if s in seqs else np.zeros((1, H_KV, 1, 128), np.float16)
                                 for s in range(n_slots)])
            cache.update(K.u.to_dev(kn), K.u.to_dev(vn), l)
            cache.quantize_decode(l)
        for s in seqs.values():
            s.pos += 1

    for _ in range(7):
        step()                       # a: 127 rows in the K Q-buffer
    step()                           # a flushes K (page 2 of 4 K pages in use -> takes the 4th)
    assert cache.pages_in_use()[0] == 4
    raised = 0
    for _ in range(28 + 128 + 20):   # b flushes K after 28 steps: no page left for its next flush
        try:
            step()
        except K.OutOfPages:
            raised += 1
    assert raised >= 1 and ("k", 1) in cache._starved
    dev = cache.seq_counts.cpu().numpy()
    for l in range(LAYERS):
        assert np.array_equal(dev[l], cache._shadow), l
    assert cache._shadow[1, 2] == 128 and cache._shadow[1, 1] == 1       # b: full K Q-buffer, still one page
    held = cache._shadow[1].copy()
    cache.release(0)
    del seqs[0]
    assert ("k", 1) not in cache._starved
    step()
    assert cache._shadow[1, 1] == 2 and cache._shadow[1, 2] == 0          # flushed at once
    assert cache._shadow[1, 3] == held[3] + (held[4] == 128)
    for _ in range(5):
        step()
    dev = cache.seq_counts.cpu().numpy()
    for l in range(LAYERS):
        assert np.array_equal(dev[l], cache._shadow), l
    cache.check_tables()
    # the stall left its record in slot 1's sticky status words, in every layer; the slot's next tenant
    # starts with clean ones
    st = cache.check_status(raise_on_error=False)
    assert st["tokens_dropped"][:, 1].all() and st["flush_skipped"][:, 1].all() and not st["tokens_dropped"][:, 0].any()
    with pytest.raises(RuntimeError, match="skipped work"):
        cache.check_status()
    cache.release(1)
    Seq(9, 32 + 50, 1000, max_len).admit(K, cache, 1)
    cache.check_status()


def test_decode_step_graph_survives_admission_and_release(K):
    """One captured graph of a decode step (both layers) is replayed while sequences are released
    and admitted between replays; outputs and final bytes equal those of an eager twin."""
    n_slots, max_len, pool = 3, 32 + 128 * 6, 12
    mod = K.u.module(H_KV, H_Q)

    def make():
        c = K.Paged(K.u.cfg(H_KV, H_Q, layers=LAYERS), n_slots, max_len, pool_pages=pool)
        Seq(11, 32 + 128 + 100, 600, max_len).admit(K, c, 0)
        Seq(12, 32 + 60, 600, max_len).admit(K, c, 2)
        return c

    kin = [torch.zeros(n_slots, H_KV, 1, 128, dtype=torch.float16, device="cuda") for _ in range(LAYERS)]
    vin = [torch.zeros_like(k) for k in kin]
    qin = torch.zeros(n_slots, H_Q, 1, 128, dtype=torch.float16, device="cuda")

    def step(c):
        outs = []
        for l in range(LAYERS):
            c.update(kin[l], vin[l], l)
            outs.append(K.attn(mod, qin, c.kv_cache[l], 128 ** -0.5, num_splits=3)[0])
            c.quantize_decode(l)
        return outs

    def feed(s):
        g = torch.Generator().manual_seed(9000 + s)
        for t in kin + vin + [qin]:
            t.copy_(torch.randn(t.shape, generator=g).half())

    cg, ce = make(), make()
    side = torch.cuda.Stream()
    for s in range(2):                      # eager steps first: the workspace exists before the capture
        feed(s)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step(cg)
        torch.cuda.current_stream().wait_stream(side)
        step(ce)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with cg.capturing():
        with torch.cuda.graph(graph):
            out_g = step(cg)
    for s in range(2, 2 + 170):
        if s == 60:                          # between replays: one leaves, a longer one arrives
            for c in (cg, ce):
                c.release(0)
                Seq(13, 32 + 128 * 2 + 127, 600, max_len).admit(K, c, 1)
        feed(s)
        graph.replay()
        cg.step_host_counters()
        out_e = step(ce)
        torch.cuda.synchronize()
        for l in range(LAYERS):
            assert torch.equal(out_g[l], out_e[l]), (s, l)
    assert np.array_equal(cg._shadow, ce._shadow) and np.array_equal(cg._table_k, ce._table_k)
    assert torch.equal(cg.seq_counts, ce.seq_counts) and np.array_equal(cg.seq_counts[0].cpu().numpy(), cg._shadow)
    for a, d in zip(ce.kv_cache, cg.kv_cache):
        for name in ("KeyCache", "KeyCache_metadata", "ValueCache", "ValueCache_metadata", "Sink_Buffer_K",
                     "Sink_Buffer_V", "Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V"):
            assert torch.equal(getattr(a, name).view(torch.uint8), getattr(d, name).view(torch.uint8)), name
        assert a.counts() == d.counts()
    cg.check_tables()
    assert cg._shadow[1, 1] >= 3 and cg._shadow[2, 1] >= 1          # flushes happened inside replays
