"""GPU parity of the decode-time state machine with per-sequence counters on the device
(kitty_append_token / kitty_flush_full through KittyCache.update / quantize_decode) against the CPU
oracle stepping every sequence on its own.  Everything is bit-exact: fp16 rows in the same slots,
packed pages, scales/zeros, counters.  Attention along the way within max-abs 2e-3."""
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
    from kitty_amd.kvcache.kernels import kitty_attention_forward
    from tests import gpu_util
    return type("NS", (), dict(KittyCache=kitty_amd.KittyCache, attn=kitty_attention_forward, u=gpu_util, lib=_lib))


def _oracle_counts(ol):
    return [getattr(ol, f) for f in FIELDS] + [0]


def _load_row(K, L, b, ol):
    """Copy a batch-1 oracle layer into row b of a device layer (identity page table)."""
    for name in ("Sink_Buffer_K", "Sink_Buffer_V", "Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V"):
        getattr(L, name)[b].copy_(K.u.to_dev(getattr(ol, name)[0]))
    for name in ("KeyCache", "KeyCache_metadata", "ValueCache", "ValueCache_metadata"):
        getattr(L, name)[b * L.MAX_PAGE:(b + 1) * L.MAX_PAGE].copy_(K.u.to_dev(getattr(ol, name)))


def _row_mismatches(L, b, ol, counts_row):
    bad = []

    def cmp(name, t, a):
        got = t.detach().cpu().numpy()
        if got.dtype == np.float16:
            got, a = got.view(np.uint16), np.ascontiguousarray(a).view(np.uint16)
        if not np.array_equal(got, a):
            bad.append((name, int((got != a).sum())))

    for name in ("Sink_Buffer_K", "Sink_Buffer_V", "Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V"):
        cmp(name, getattr(L, name)[b], getattr(ol, name)[0])
    for name in ("KeyCache", "KeyCache_metadata", "ValueCache", "ValueCache_metadata"):
        cmp(name, getattr(L, name)[b * L.MAX_PAGE:(b + 1) * L.MAX_PAGE], getattr(ol, name))
    if list(counts_row) != _oracle_counts(ol):
        bad.append(("seq_counts", list(counts_row), _oracle_counts(ol)))
    return bad


def test_ragged_batch_steps_like_the_oracle_per_sequence(K):
    """Sequences in every phase of the state machine (sink still filling, ring filling, ring
    evicting, K and V flushing on different steps) decode 300 steps in one batch."""
    H_KV, H_Q, steps = 2, 8, 300
    starts = [5, 31, 32, 40, 32 + 127, 32 + 128, 32 + 255, 32 + 128 * 3 + 77]
    B = len(starts)
    max_len = 32 + 128 * 8
    cache = K.KittyCache(K.u.cfg(H_KV, H_Q), B, max_len)
    L = cache.kv_cache[0]
    ols, kvs = [], []
    for b, T in enumerate(starts):
        k, v = make_kv(1, H_KV, T + steps, seed=900 + b)
        ol = O.OracleLayer(1, max_len, H_KV)
        ol.update(k[:, :, :T], v[:, :, :T])
        ol.quantize_prefill()
        _load_row(K, L, b, ol)
        ols.append(ol)
        kvs.append((k, v, T))
    counts = torch.tensor([_oracle_counts(ol) for ol in ols], dtype=torch.int32)
    cache.enable_device_counters(counts)
    assert L.get_total_length() == max(starts)
    mod = K.u.module(H_KV, H_Q)
    check_at = {0, 95, 96, 97, 223, 224, 299}
    for s in range(steps):
        kn = np.concatenate([k[:, :, T + s:T + s + 1] for k, v, T in kvs], axis=0)
        vn = np.concatenate([v[:, :, T + s:T + s + 1] for k, v, T in kvs], axis=0)
        assert cache.update(K.u.to_dev(kn), K.u.to_dev(vn), 0) is False
        for b, ol in enumerate(ols):
            ol.update(kn[b:b + 1], vn[b:b + 1])
        if s in check_at:
            q = make_q(B, H_Q, seed=s)
            out, _ = K.attn(mod, K.u.to_dev(q), L, 128 ** -0.5, variant=1)
            got = out.detach().cpu().numpy().astype(np.float64)
            for b, ol in enumerate(ols):
                want = O.decode_attention(ol, q[b:b + 1], 128 ** -0.5, reference_rounding=False)
                assert np.abs(got[b:b + 1] - want).max() <= ATOL, (s, b)
            got_counts = L.seq_counts.cpu().numpy()
            for b, ol in enumerate(ols):       # state between update and quantize_decode
                assert list(got_counts[b]) == _oracle_counts(ol), (s, b)
        cache.quantize_decode(0)
        for ol in ols:
            ol.quantize_decode()
    got_counts = L.seq_counts.cpu().numpy()
    for b, ol in enumerate(ols):
        assert _row_mismatches(L, b, ol, got_counts[b]) == [], f"row {b} (start {starts[b]})"
    assert L.get_total_length() == max(starts) + steps
    assert sum(ol.PageCount_K for ol in ols) > sum((T - 32) // 128 for T in starts if T > 32) + 8   # flushes happened


def test_uniform_batch_matches_host_counter_mode(K):
    """The same prefill and decode steps with host counters (the reference's mode) and with device
    counters leave the same bytes everywhere, and the host shadow agrees with the device."""
    B, H_KV, H_Q, T, steps = 3, 2, 8, 32 + 128 + 100, 200
    k, v = make_kv(B, H_KV, T + steps, seed=77)
    caches = []
    for mode in ("host", "device"):
        c = K.KittyCache(K.u.cfg(H_KV, H_Q), B, 1024)
        assert c.update(K.u.to_dev(k[:, :, :T]), K.u.to_dev(v[:, :, :T]), 0) is True
        c.quantize_prefill(0)
        if mode == "device":
            c.enable_device_counters()
        for s in range(steps):
            c.update(K.u.to_dev(k[:, :, T + s:T + s + 1]), K.u.to_dev(v[:, :, T + s:T + s + 1]), 0)
            c.quantize_decode(0)
        caches.append(c.kv_cache[0])
    a, d = caches
    for name in ("KeyCache", "KeyCache_metadata", "ValueCache", "ValueCache_metadata", "Sink_Buffer_K",
                 "Sink_Buffer_V", "Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V"):
        assert torch.equal(getattr(a, name).view(torch.uint8), getattr(d, name).view(torch.uint8)), name
    assert a.counts() == d.counts()
    assert d.seq_counts.cpu().tolist() == [a.counts()] * B
    q = K.u.to_dev(make_q(B, H_Q, seed=5))
    mod = K.u.module(H_KV, H_Q)
    for variant in (0, 1):
        oa, _ = K.attn(mod, q, a, 128 ** -0.5, variant=variant, num_splits=3)
        od, _ = K.attn(mod, q, d, 128 ** -0.5, variant=variant, num_splits=3)
        assert torch.equal(oa, od), variant


def test_smaller_active_batch_leaves_other_rows_alone(K):
    B, H_KV, H_Q, T = 4, 1, 4, 32 + 128
    k, v = make_kv(B, H_KV, T + 130, seed=12)
    c = K.KittyCache(K.u.cfg(H_KV, H_Q), B, 1024)
    c.update(K.u.to_dev(k[:, :, :T]), K.u.to_dev(v[:, :, :T]), 0)
    c.quantize_prefill(0)
    c.enable_device_counters()
    L = c.kv_cache[0]
    before = L.seq_counts.cpu().clone()
    qk_before = L.Q_Buffer_K[2:].clone()
    for s in range(130):
        c.update(K.u.to_dev(k[:2, :, T + s:T + s + 1]), K.u.to_dev(v[:2, :, T + s:T + s + 1]), 0)
        c.quantize_decode(0)
    after = L.seq_counts.cpu()
    assert torch.equal(after[2:], before[2:]) and torch.equal(L.Q_Buffer_K[2:], qk_before)
    assert after[0].tolist() == after[1].tolist() == L.counts()
    assert after[0, 1].item() == 2 and after[0, 2].item() == 2       # prefill page + one flushed page, two rows after it


def test_skipped_flush_drops_the_token_instead_of_overrunning(K):
    """Through the C ABI directly: a sequence whose K Q-buffer is full is left untouched."""
    B, H_KV, H_Q = 2, 1, 4
    c = K.KittyCache(K.u.cfg(H_KV, H_Q), B, 1024)
    L = c.kv_cache[0]
    L.enable_device_counters(torch.tensor([[32, 0, 128, 0, 0, 128, 0, 0], [32, 0, 127, 0, 0, 127, 0, 0]], dtype=torch.int32))
    k = torch.ones(B, H_KV, 1, 128, dtype=torch.float16, device="cuda")
    snapshot = [t.clone() for t in (L.Q_Buffer_K, L.Q_Buffer_V, L.Local_Buffer_V, L.Sink_Buffer_K)]
    rc = K.lib.lib().kitty_append_token(L.descriptor(), k.data_ptr(), k.data_ptr(), k.stride(0) * 2, k.stride(1) * 2,
                                        None, None, 0, B, K.lib.current_stream_ptr(k.device))
    assert rc == 0
    torch.cuda.synchronize()
    assert L.seq_counts.cpu().tolist() == [[32, 0, 128, 0, 0, 128, 0, 0], [32, 0, 128, 0, 0, 128, 0, 0]]
    assert torch.equal(L.Q_Buffer_K[0], snapshot[0][0]) and torch.equal(L.Local_Buffer_V[0], snapshot[2][0])
    assert bool((L.Q_Buffer_K[1, :, 127] == 1).all()) and bool((L.Local_Buffer_V[1, :, 127] == 1).all())


def test_device_counter_calls_reject_bad_arguments(K):
    c = K.KittyCache(K.u.cfg(1, 4), 2, 512)
    L = c.kv_cache[0]
    k = torch.zeros(2, 1, 1, 128, dtype=torch.float16, device="cuda")
    lib = K.lib.lib()
    st = K.lib.current_stream_ptr(k.device)
    assert lib.kitty_append_token(L.descriptor(), k.data_ptr(), k.data_ptr(), 256, 256, None, None, 0, 2, st) == -1   # no seq_counts
    assert b"seq_counts" in lib.kitty_last_error()
    assert lib.kitty_flush_full(L.descriptor(), 2, st) == -1
    with pytest.raises(ValueError):
        L.enable_device_counters(torch.zeros(3, 8, dtype=torch.int32))
    with pytest.raises(ValueError):
        L.enable_device_counters(torch.tensor([[32, 0, 5, 0, 0, 4, 0, 0]] * 2, dtype=torch.int32))   # K != V length
    L.enable_device_counters()
    assert lib.kitty_append_token(L.descriptor(), None, k.data_ptr(), 256, 256, None, None, 0, 2, st) == -1
    assert lib.kitty_append_token(L.descriptor(), k.data_ptr() + 2, k.data_ptr(), 256, 256, None, None, 0, 2, st) == -4
    assert lib.kitty_append_chunk(L.descriptor(), k.data_ptr() + 2, k.data_ptr(), 256, 256, 256, 2, 1, st) == -4


def test_decode_step_replays_from_one_captured_graph(K):
    """update -> attend -> quantize_decode captured once and replayed 150 times (across a K flush,
    a V flush and the ring wrap), with eager work and a synchronisation between replays; every
    replay's output and the final state equal those of an eager twin."""
    B, H_KV, H_Q, T, steps = 3, 2, 8, 32 + 128 + 120, 150
    k, v = make_kv(B, H_KV, T + steps + 2, seed=41)
    mod = K.u.module(H_KV, H_Q)

    def make():
        c = K.KittyCache(K.u.cfg(H_KV, H_Q), B, 1024)
        c.update(K.u.to_dev(k[:, :, :T]), K.u.to_dev(v[:, :, :T]), 0)
        c.quantize_prefill(0)
        c.enable_device_counters()
        return c

    def step(c, kk, vv, qq):
        c.update(kk, vv, 0)
        out, _ = K.attn(mod, qq, c.kv_cache[0], 128 ** -0.5, num_splits=3)
        c.quantize_decode(0)
        return out

    cg, ce = make(), make()
    kin = torch.zeros(B, H_KV, 1, 128, dtype=torch.float16, device="cuda")
    vin, qin = torch.zeros_like(kin), torch.zeros(B, H_Q, 1, 128, dtype=torch.float16, device="cuda")

    def feed(s):
        kin.copy_(K.u.to_dev(k[:, :, T + s:T + s + 1]))
        vin.copy_(K.u.to_dev(v[:, :, T + s:T + s + 1]))
        qin.copy_(K.u.to_dev(make_q(B, H_Q, seed=1000 + s)))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    for s in range(2):                      # eager steps first: the workspace exists before the capture
        feed(s)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step(cg, kin, vin, qin)
        torch.cuda.current_stream().wait_stream(side)
        step(ce, kin, vin, qin)
    torch.cuda.synchronize()
    saved = cg.host_counters()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g = step(cg, kin, vin, qin)
    cg.restore_host_counters(saved)
    for s in range(2, 2 + steps):
        feed(s)
        graph.replay()
        cg.step_host_counters()
        out_e = step(ce, kin, vin, qin)
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e), f"replay {s - 2}"
    a, d = ce.kv_cache[0], cg.kv_cache[0]
    for name in ("KeyCache", "KeyCache_metadata", "ValueCache", "ValueCache_metadata", "Sink_Buffer_K",
                 "Sink_Buffer_V", "Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V", "seq_counts"):
        assert torch.equal(getattr(a, name).view(torch.uint8), getattr(d, name).view(torch.uint8)), name
    assert a.counts() == d.counts() and d.get_total_length() == T + 2 + steps
    assert d.PageCount_K == 3 and d.PageCount_V == 2      # both flushes happened inside replays
