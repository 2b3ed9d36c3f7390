"""kitty_decode_attn_static (decode attention whose split-K partials live in the library's own
device array, for callers that cannot allocate) against kitty_decode_attn with a caller-owned
workspace: same kernels, so the outputs must be bit-identical.  Two calls in a row, the second on a
smaller input, then the first again: whatever a call leaves in the shared array must not leak into
the next."""
import numpy as np
import pytest
import torch

from tests.helpers import make_kv, make_q

pytestmark = pytest.mark.gpu
SC = 128 ** -0.5
STATIC_BYTES = 16 << 20


@pytest.fixture(scope="module")
def K():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import kitty_amd
    from kitty_amd import _lib
    _lib.lib()
    from tests import gpu_util
    return type("NS", (), dict(KittyCache=kitty_amd.KittyCache, u=gpu_util, lib=_lib))


def _cache(K, B, H_KV, H_Q, T, seed):
    k, v = make_kv(B, H_KV, T, seed=seed)
    c = K.KittyCache(K.u.cfg(H_KV, H_Q), B, T + 256)
    c.update(K.u.to_dev(k), K.u.to_dev(v), 0)
    c.quantize_prefill(0)
    return c


def _both(K, cache, q, splits, variant=0):
    """(output through the caller-owned workspace, output through the library's array, return code)"""
    lib = K.lib.lib()
    L = cache.kv_cache[0]
    B, H_Q = q.shape[0], q.shape[1]
    st = K.lib.current_stream_ptr(q.device)
    n = splits if splits > 0 else lib.kitty_decode_attn_default_splits(
        B, L.H_KV, 1 + (L.get_total_length() - L.Sink_Count + 127) // 128, int(L.seq_counts is not None))
    ws = torch.empty(lib.kitty_decode_attn_workspace_bytes(B, H_Q, 128, n), dtype=torch.uint8, device=q.device)
    want = torch.full((B, 1, H_Q, 128), 7.0, dtype=torch.float16, device=q.device)
    got = torch.full_like(want, -7.0)
    K.lib.check(lib.kitty_decode_attn(L.descriptor(), q.data_ptr(), B, H_Q, SC, want.data_ptr(), ws.data_ptr(),
                                      ws.numel(), n, variant, st), "kitty_decode_attn")
    rc = lib.kitty_decode_attn_static(L.descriptor(), q.data_ptr(), B, H_Q, SC, got.data_ptr(), splits, variant, st)
    torch.cuda.synchronize()
    return want, got, rc


def test_static_entry_point_matches_the_workspace_one_on_calls_in_a_row(K):
    big = _cache(K, 4, 2, 8, 32 + 128 * 9 + 70, seed=61)
    small = _cache(K, 2, 2, 8, 32 + 128 * 2 + 5, seed=62)
    qb = K.u.to_dev(make_q(4, 8, seed=61))
    qs = K.u.to_dev(make_q(2, 8, seed=62))
    for cache, q, splits in ((big, qb, 5), (small, qs, 2), (big, qb, 0), (small, qs, 0), (big, qb, 5)):
        for variant in (0, 1):
            want, got, rc = _both(K, cache, q, splits, variant)
            assert rc == 0, K.lib.lib().kitty_last_error()
            assert torch.equal(want, got), (splits, variant)
            assert torch.isfinite(got.float()).all()


def test_static_entry_point_allocates_nothing(K):
    """Device memory in use by the process does not move across calls (the first call on a device
    only asks the runtime where the array lies)."""
    cache = _cache(K, 2, 2, 8, 32 + 128 * 3, seed=63)
    q = K.u.to_dev(make_q(2, 8, seed=63))
    lib = K.lib.lib()
    L = cache.kv_cache[0]
    out = torch.empty((2, 1, 8, 128), dtype=torch.float16, device="cuda")
    st = K.lib.current_stream_ptr(q.device)
    desc = L.descriptor()
    assert lib.kitty_decode_attn_static(desc, q.data_ptr(), 2, 8, SC, out.data_ptr(), 3, 0, st) == 0
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(20):
        assert lib.kitty_decode_attn_static(desc, q.data_ptr(), 2, 8, SC, out.data_ptr(), 3, 0, st) == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0


def test_static_entry_point_rejects_what_does_not_fit(K):
    cache = _cache(K, 2, 2, 8, 32 + 128 * 3, seed=64)
    q = K.u.to_dev(make_q(2, 8, seed=64))
    lib = K.lib.lib()
    L = cache.kv_cache[0]
    out = torch.zeros((2, 1, 8, 128), dtype=torch.float16, device="cuda")
    st = K.lib.current_stream_ptr(q.device)
    per_split = 2 * 8 * (2 + 128) * 4
    too_many = STATIC_BYTES // per_split + 1
    assert lib.kitty_decode_attn_static(L.descriptor(), q.data_ptr(), 2, 8, SC, out.data_ptr(), too_many, 0, st) == -5
    assert b"array holds" in lib.kitty_last_error()
    assert lib.kitty_decode_attn_static(L.descriptor(), None, 2, 8, SC, out.data_ptr(), 2, 0, st) == -1
    assert lib.kitty_decode_attn_static(L.descriptor(), q.data_ptr(), 2, 7, SC, out.data_ptr(), 2, 0, st) == -2
    torch.cuda.synchronize()
    assert not out.any()


def test_decode_step_replayed_from_a_graph(K):
    """What the entry point is for: one decode step of a layer - append the new token, attend, flush
    the full Q-buffers - captured once in a HIP graph (per-sequence counters on the device, so the
    kernels' arguments never change) and replayed step after step, with eager copies into the
    graph's input buffers and synchronisations in between.  Every replay must give, bit for bit,
    what the same step gives eagerly on a twin cache through the workspace entry point; the steps
    cross a flush of both Q-buffers."""
    from kitty_amd.kvcache.kernels import kitty_attention_forward
    B, H_KV, H_Q, T, steps = 2, 2, 8, 32 + 128 + 100, 40
    k, v = make_kv(B, H_KV, T + steps, seed=71)
    twins = []
    for _ in range(2):
        c = K.KittyCache(K.u.cfg(H_KV, H_Q), B, 1024)
        assert c.update(K.u.to_dev(k[:, :, :T]), K.u.to_dev(v[:, :, :T]), 0) is True
        c.quantize_prefill(0)
        c.enable_device_counters()
        twins.append(c)
    eager, graphed = twins
    lib = K.lib.lib()
    L = graphed.kv_cache[0]
    kin = torch.zeros((B, H_KV, 1, 128), dtype=torch.float16, device="cuda")
    vin, qin = torch.zeros_like(kin), torch.zeros((B, H_Q, 1, 128), dtype=torch.float16, device="cuda")
    out = torch.zeros((B, 1, H_Q, 128), dtype=torch.float16, device="cuda")
    desc = L.descriptor()

    def step(stream):
        rc = lib.kitty_append_token(desc, kin.data_ptr(), vin.data_ptr(), kin.stride(0) * 2, kin.stride(1) * 2,
                                    None, None, 0, B, stream)
        rc = rc or lib.kitty_decode_attn_static(desc, qin.data_ptr(), B, H_Q, SC, out.data_ptr(), 0, 0, stream)
        return rc or lib.kitty_flush_full(desc, B, stream)

    # the first call on a device asks the runtime where the library's array lies: not under capture
    assert lib.kitty_decode_attn_static(desc, qin.data_ptr(), B, H_Q, SC, out.data_ptr(), 0, 0,
                                        K.lib.current_stream_ptr(qin.device)) == 0
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):   # capture records, it does not run: the cache is untouched until the first replay
        rc = step(torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.kitty_last_error()
    mod = K.u.module(H_KV, H_Q)
    for s in range(steps):
        kn, vn = K.u.to_dev(k[:, :, T + s:T + s + 1]), K.u.to_dev(v[:, :, T + s:T + s + 1])
        q = K.u.to_dev(make_q(B, H_Q, seed=200 + s))
        assert eager.update(kn, vn, 0) is False
        want, _ = kitty_attention_forward(mod, q, eager.kv_cache[0], SC)
        eager.quantize_decode(0)
        kin.copy_(kn), vin.copy_(vn), qin.copy_(q)
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"step {s}"
    a, b = eager.kv_cache[0], L
    assert torch.equal(a.seq_counts, b.seq_counts)
    assert int(a.seq_counts[0, 1]) == 2 and int(a.seq_counts[0, 3]) == 1          # both Q-buffers were flushed
    for name in ("KeyCache", "KeyCache_metadata", "ValueCache", "ValueCache_metadata", "Q_Buffer_K", "Local_Buffer_V"):
        assert torch.equal(getattr(a, name), getattr(b, name)), name


def test_first_call_on_a_capturing_stream_is_refused_with_a_reason():
    """The first call on a device looks the array's address up in the runtime, which a stream capture
    must not contain.  In a fresh process, a first call under capture is rejected (KITTY_E_RANGE, nothing
    recorded), and after one eager call the same capture works."""
    import os
    import subprocess
    import sys
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    code = r"""
import sys, torch
sys.path.insert(0, %r)
import kitty_amd
from kitty_amd import _lib
from tests import gpu_util as u
from tests.helpers import make_kv, make_q
lib = _lib.lib()
k, v = make_kv(1, 2, 32 + 128 * 2 + 5, seed=5)
c = kitty_amd.KittyCache(u.cfg(2, 8), 1, 1024)
c.update(u.to_dev(k), u.to_dev(v), 0)
c.quantize_prefill(0)
L = c.kv_cache[0]
q = u.to_dev(make_q(1, 8, seed=5))
out = torch.zeros((1, 1, 8, 128), dtype=torch.float16, device="cuda")
call = lambda: lib.kitty_decode_attn_static(L.descriptor(), q.data_ptr(), 1, 8, 128 ** -0.5, out.data_ptr(), 2, 0,
                                            _lib.current_stream_ptr(q.device))
torch.cuda.synchronize()
g = torch.cuda.CUDAGraph()
with torch.cuda.graph(g):
    rc = call()
msg = lib.kitty_last_error().decode()
assert rc == -3 and "before capturing" in msg, (rc, msg)
assert call() == 0
torch.cuda.synchronize()
eager = out.clone()
out.zero_()
g2 = torch.cuda.CUDAGraph()
with torch.cuda.graph(g2):
    assert call() == 0
g2.replay()
torch.cuda.synchronize()
assert torch.equal(out, eager) and bool(out.abs().sum() > 0)
print("ok")
""" % os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "ok" in r.stdout, r.stdout + r.stderr
