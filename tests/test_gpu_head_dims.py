"""Head dimensions 64 and 256 on the GPU (the reference takes ``config.head_dim`` and boosts a quarter of the
channels, src/kitty/kvcache/kitty.py:39-44; its kernels take D as a parameter): quantizer, cache plugin,
decode attention and chunked-prefill attention against the oracle, whose quantizer is pinned at these sizes
by the reference's own output (tests/golden/quant_k_v_d64.npz, quant_k_v_d256.npz).  These sizes run on
plain kernels of their own; packed bytes bit-exact, attention within 2e-3 of float64 attention over the
reference's twice-rounded fp16 dequantization."""
import numpy as np
import pytest
import torch

from oracle import kitty_oracle as O
from tests.helpers import make_kv

pytestmark = pytest.mark.gpu
ATOL = 2e-3
DIMS = [64, 256]


@pytest.fixture(scope="module")
def K():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import kitty_amd
    from kitty_amd import _lib
    _lib.lib()
    from kitty_amd.kvcache.kernels import (kitty_attention_forward, kitty_prefill_attention, quantize_pack_k,
                                           quantize_pack_v, select_boost_k)
    from tests import gpu_util
    return type("NS", (), dict(KittyCache=kitty_amd.KittyCache, attn=kitty_attention_forward,
                               prefill=kitty_prefill_attention, qk=quantize_pack_k, qv=quantize_pack_v,
                               sel=select_boost_k, u=gpu_util))


def _np(t):
    return t.detach().cpu().numpy()


def _q(B, HQ, T, D, seed):
    return np.random.default_rng(seed).standard_normal((B, HQ, T, D)).astype(np.float16)


@pytest.mark.parametrize("D", DIMS)
@pytest.mark.parametrize("student_t", [False, True])
def test_quantize_pack_bit_exact(K, D, student_t):
    """Both quantizers into permuted pages at an offset: fused selection, a given slot map, selection alone."""
    B, H, P, DB = 2, 2, 2, D // 4
    x, _ = make_kv(B, H, 32 + 128 * P + 9, D=D, seed=3 + D, student_t=student_t)
    rng = np.random.default_rng(D)
    max_page = 4
    pt = rng.permutation(B * max_page).reshape(B, max_page).astype(np.int64)
    lay = O.Layout(H_KV=H, D=D, D_BOOSTED=DB)
    kc = torch.zeros((B * max_page, lay.bytes_per_page_K), dtype=torch.uint8, device="cuda")
    km = torch.zeros((B * max_page, H, D, 2), dtype=torch.float16, device="cuda")
    vc = torch.zeros((B * max_page, lay.bytes_per_page_V), dtype=torch.uint8, device="cuda")
    vm = torch.zeros((B * max_page, H, 128, 2), dtype=torch.float16, device="cuda")
    xd, ptd = K.u.to_dev(x), K.u.to_dev(pt)
    K.qk(xd, 32, P, ptd, 1, kc, km, 128, DB)
    K.qv(xd, 32, P, ptd, 1, vc, vm, 128)
    sm = K.sel(xd, 32, P, 128, DB)
    torch.cuda.synchronize()
    okc, okm = np.zeros(tuple(kc.shape), np.uint8), np.zeros(tuple(km.shape), np.float16)
    ovc, ovm = np.zeros(tuple(vc.shape), np.uint8), np.zeros(tuple(vm.shape), np.float16)
    O.quantize_pack_k(x, 32, P, pt, 1, okc, okm, 128, DB)
    O.quantize_pack_v(x, 32, P, pt, 1, ovc, ovm, 128)
    assert np.array_equal(_np(kc), okc) and np.array_equal(_np(km).view(np.uint16), okm.view(np.uint16))
    assert np.array_equal(_np(vc), ovc) and np.array_equal(_np(vm).view(np.uint16), ovm.view(np.uint16))
    osm = np.stack([[[O.select_boost(x[b, h, 32 + 128 * p: 32 + 128 * (p + 1)], DB) for p in range(P)]
                     for h in range(H)] for b in range(B)])
    assert np.array_equal(_np(sm), osm)
    # a caller's own map (here: the boosted channels reversed) is consumed as the reference's kernel consumes it
    sm2 = np.where(osm < DB, DB - 1 - osm, DB).astype(np.uint8)
    kc2, km2 = torch.zeros_like(kc), torch.zeros_like(km)
    K.qk(xd, 32, P, ptd, 1, kc2, km2, 128, DB, slot_map=K.u.to_dev(sm2))
    torch.cuda.synchronize()
    okc2, okm2 = np.zeros_like(okc), np.zeros_like(okm)
    O.quantize_pack_k(x, 32, P, pt, 1, okc2, okm2, 128, DB, slot_map=sm2)
    assert np.array_equal(_np(kc2), okc2) and np.array_equal(_np(km2).view(np.uint16), okm2.view(np.uint16))


def _build(K, D, B, H_KV, H_Q, T, max_len, seed):
    k, v = make_kv(B, H_KV, T, D=D, seed=seed)
    cache = K.KittyCache(K.u.cfg(H_KV, H_Q, D=D), B, max_len)
    assert cache.update(K.u.to_dev(k), K.u.to_dev(v), 0) is True
    cache.quantize_prefill(0)
    ol = O.OracleLayer(B, max_len, H_KV, D=D, D_BOOSTED=D // 4)
    assert ol.update(k, v) is True
    ol.quantize_prefill()
    return cache, ol


def _check(got, ol, q, D, what):
    sc = D ** -0.5
    ref = O.decode_attention(ol, q, sc, reference_rounding=False, dequant="two")
    err = np.abs(got - ref).max()
    assert err <= ATOL, f"{what}: {err:.3e} vs float64 attention over fp16-dequantized KV"
    lit = O.decode_attention(ol, q, sc, reference_rounding=True, dequant="two").astype(np.float64)
    assert np.abs(got - lit).max() <= 6.5e-3, f"{what}: vs the reference's own fp16 logits and probabilities"


@pytest.mark.parametrize("D", DIMS)
def test_cache_roundtrip_decode_steps_and_attention(K, D):
    """Prefill, then decode steps across both flushes in the caller's order update -> attend -> flush: every
    byte and counter of the layer equals the oracle's, attention is within tolerance along the way."""
    B, H_KV, H_Q = 2, 2, 8
    T0 = 32 + 128 * 2 + 70
    cache, ol = _build(K, D, B, H_KV, H_Q, T0, 1024, seed=21 + D)
    L = cache.kv_cache[0]
    assert L.D == D and L.D_BOOSTED == D // 4
    assert not K.u.layer_bytes_equal(L, ol)
    mod = K.u.module(H_KV, H_Q)
    kn, vn = make_kv(B, H_KV, 140, D=D, seed=22 + D)
    for s in range(140):
        ks, vs = kn[:, :, s:s + 1], vn[:, :, s:s + 1]
        assert cache.update(K.u.to_dev(ks), K.u.to_dev(vs), 0) is False and ol.update(ks, vs) is False
        if s % 35 == 0 or s in (57, 58, 59):
            q = _q(B, H_Q, 1, D, 100 + s)
            out, _ = K.attn(mod, K.u.to_dev(q), L, D ** -0.5)
            torch.cuda.synchronize()
            assert tuple(out.shape) == (B, 1, H_Q, D)
            _check(_np(out).astype(np.float64), ol, q, D, f"D={D} step {s}")
        cache.quantize_decode(0)
        ol.quantize_decode()
    torch.cuda.synchronize()
    assert (L.PageCount_K, L.PageCount_V) == (ol.PageCount_K, ol.PageCount_V) == (3, 2)
    bad = K.u.layer_bytes_equal(L, ol)
    assert not bad, bad


@pytest.mark.parametrize("D", DIMS)
@pytest.mark.parametrize("G", [1, 3, 8, 16])
def test_group_sizes_and_split_counts(K, D, G):
    H_KV = 1 if G == 16 else 2
    cache, ol = _build(K, D, 1, H_KV, H_KV * G, 32 + 128 * 3 + 17, 1024, seed=31 + D + G)
    L = cache.kv_cache[0]
    q = _q(1, H_KV * G, 1, D, 7 + G)
    mod = K.u.module(H_KV, H_KV * G)
    outs = []
    for splits in (None, 1, 3, 9):
        out, _ = K.attn(mod, K.u.to_dev(q), L, D ** -0.5, num_splits=splits)
        torch.cuda.synchronize()
        _check(_np(out).astype(np.float64), ol, q, D, f"D={D} G={G} splits={splits}")
        outs.append(out.float())
    for o in outs[1:]:
        assert (o - outs[0]).abs().max().item() <= 1e-3


@pytest.mark.parametrize("D", DIMS)
@pytest.mark.parametrize("T0,G", [(0, 4), (20, 4), (32 + 128 + 50, 4), (32 + 128 + 50, 3), (32 + 128 + 50, 16), (200, 1)])
def test_chunked_prefill_attention(K, D, T0, G):
    """A chunk of new tokens over an empty layer (plain causal attention), a sink-only layer and a layer with
    packed pages, against the oracle's chunk attention; then the chunk is appended and the layer compared."""
    B, H_KV, Tq = 1, 2, 37
    H_Q = H_KV * G
    k, v = make_kv(B, H_KV, T0 + Tq, D=D, seed=41 + D + T0)
    cache = K.KittyCache(K.u.cfg(H_KV, H_Q, D=D), B, 1024)
    ol = O.OracleLayer(B, 1024, H_KV, D=D, D_BOOSTED=D // 4)
    if T0:
        cache.update(K.u.to_dev(k[:, :, :T0]), K.u.to_dev(v[:, :, :T0]), 0)
        cache.quantize_prefill(0)
        ol.update(k[:, :, :T0], v[:, :, :T0])
        ol.quantize_prefill()
    q = _q(B, H_Q, Tq, D, 5 + T0)
    kc, vc = k[:, :, T0:], v[:, :, T0:]
    out, _ = K.prefill(K.u.module(H_KV, H_Q), K.u.to_dev(q), K.u.to_dev(kc), K.u.to_dev(vc), cache.kv_cache[0], D ** -0.5)
    torch.cuda.synchronize()
    assert tuple(out.shape) == (B, Tq, H_Q, D)
    ref = O.chunk_attention(ol, q, kc, vc, D ** -0.5, dequant="two")
    err = np.abs(_np(out).astype(np.float64) - ref).max()
    assert err <= ATOL, f"D={D} T0={T0}: {err:.3e}"
    cache.append(K.u.to_dev(kc), K.u.to_dev(vc), 0)
    ol.append(kc, vc)
    torch.cuda.synchronize()
    bad = K.u.layer_bytes_equal(cache.kv_cache[0], ol, live_q_rows_only=True)
    assert not bad, bad


@pytest.mark.parametrize("D", DIMS)
def test_device_counters_and_page_pools_say_what_they_need(K, D):
    import kitty_amd
    cache, _ = _build(K, D, 1, 2, 8, 100, 512, seed=5)
    with pytest.raises(ValueError, match="head_dim 128"):
        cache.enable_device_counters()
    with pytest.raises(ValueError, match="head_dim 128"):
        kitty_amd.PagedKittyCache(K.u.cfg(2, 8, D=D), 2, 512, pool_pages=4)
