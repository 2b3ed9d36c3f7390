"""GPU parity of chunked-prefill attention (through the Python API, i.e. the C ABI) against the
oracle: float64 causal attention over [cache dequantized as decode does | the chunk in fp16].

Tolerance: max-abs 2e-3 on fp16 outputs.  The kernel dequantizes a page exactly as the reference's
expression fp16(code)*scale+zero evaluates eagerly (two fp16 roundings, the oracle's "two" mode),
so unlike decode there is no dequantization ambiguity in this comparison; what remains is the fp16
rounding of the probabilities and of the output."""
import numpy as np
import pytest
import torch

from oracle import kitty_oracle as O
from tests.helpers import make_kv

pytestmark = pytest.mark.gpu
ATOL = 2e-3
SC = 128 ** -0.5


@pytest.fixture(scope="module")
def K():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import kitty_amd
    from kitty_amd import _lib
    _lib.lib()
    from kitty_amd.kvcache.kernels import kitty_attention_forward, kitty_prefill_attention
    from tests import gpu_util
    return type("NS", (), dict(KittyCache=kitty_amd.KittyCache, attn=kitty_attention_forward,
                               pre=kitty_prefill_attention, u=gpu_util))


def _q(B, HQ, Tq, seed):
    return np.random.default_rng(seed + 31337).standard_normal((B, HQ, Tq, 128)).astype(np.float16)


def _state(K, B, H_KV, H_Q, T0, steps, max_len, seed, student_t=False):
    """Device cache and oracle after a prefill of T0 tokens and `steps` decode steps."""
    cache = K.KittyCache(K.u.cfg(H_KV, H_Q), B, max_len)
    ol = O.OracleLayer(B, max_len, H_KV)
    if T0 == 0:
        return cache, ol
    k, v = make_kv(B, H_KV, T0 + steps, seed=seed, student_t=student_t)
    kd, vd = K.u.to_dev(k), K.u.to_dev(v)
    cache.update(kd[:, :, :T0], vd[:, :, :T0], 0)
    cache.quantize_prefill(0)
    ol.update(k[:, :, :T0], v[:, :, :T0])
    ol.quantize_prefill()
    for s in range(steps):
        t = T0 + s
        cache.update(kd[:, :, t:t + 1], vd[:, :, t:t + 1], 0)
        cache.quantize_decode(0)
        ol.update(k[:, :, t:t + 1], v[:, :, t:t + 1])
        ol.quantize_decode()
    assert K.u.layer_bytes_equal(cache.kv_cache[0], ol) == []
    return cache, ol


def _run(K, cache, ol, H_KV, H_Q, B, Tq, seed, student_t=False, what=""):
    kc, vc = make_kv(B, H_KV, Tq, seed=seed + 1, student_t=student_t)
    q = _q(B, H_Q, Tq, seed)
    out, w = K.pre(K.u.module(H_KV, H_Q), K.u.to_dev(q), K.u.to_dev(kc), K.u.to_dev(vc), cache.kv_cache[0], SC)
    assert w is None and tuple(out.shape) == (B, Tq, H_Q, 128) and out.dtype == torch.float16
    torch.cuda.synchronize()
    got = out.cpu().numpy().astype(np.float64)
    want = O.chunk_attention(ol, q, kc, vc, SC)
    assert np.isfinite(got).all(), what
    err = np.abs(got - want).max()
    assert err <= ATOL, f"{what}: {err:.3e}"
    return got, q, kc, vc


@pytest.mark.parametrize("Tq", [1, 5, 64, 65, 130, 300])
def test_empty_cache_is_plain_causal_attention(K, Tq):
    B, H_KV, H_Q = 2, 2, 8
    cache, ol = _state(K, B, H_KV, H_Q, 0, 0, 1024, seed=1)
    got, q, kc, vc = _run(K, cache, ol, H_KV, H_Q, B, Tq, seed=Tq, what=f"Tq={Tq}")
    # the same thing from torch (fp32, CPU): textbook reference independent of the oracle
    qt, kt, vt = (torch.from_numpy(a).float() for a in (q, kc, vc))
    ref = torch.nn.functional.scaled_dot_product_attention(
        qt, kt.repeat_interleave(H_Q // H_KV, 1), vt.repeat_interleave(H_Q // H_KV, 1), is_causal=True, scale=SC)
    assert np.abs(got - ref.transpose(1, 2).numpy()).max() <= ATOL


@pytest.mark.parametrize("T0,steps", [(7, 0), (32, 0), (33, 0), (100, 3), (161, 0), (32 + 128 * 3 + 50, 0),
                                      (32 + 128 * 2 + 120, 140), (20, 200)])
@pytest.mark.parametrize("Tq", [1, 33, 200])
def test_chunk_over_cached_prefix(K, T0, steps, Tq):
    """Sink only, sink + residual, pages with a mixed K-packed / V-fp16 tile, ring offset != 0."""
    B, H_KV, H_Q = 2, 2, 8
    cache, ol = _state(K, B, H_KV, H_Q, T0, steps, 2048, seed=T0 + steps)
    _run(K, cache, ol, H_KV, H_Q, B, Tq, seed=T0 + Tq, what=f"T0={T0} steps={steps} Tq={Tq}")


@pytest.mark.parametrize("G", [1, 2, 3, 4, 8, 16])
def test_chunk_group_sizes(K, G):
    B, H_KV, T0, Tq = 1, 2, 32 + 128 * 2 + 77, 150
    cache, ol = _state(K, B, H_KV, H_KV * G, T0, 0, 1024, seed=G)
    _run(K, cache, ol, H_KV, H_KV * G, B, Tq, seed=G, what=f"G={G}")


def test_chunk_without_boosted_channels(K):
    """D_BOOSTED = 0: the other instantiation of the kernel (the reference's cache always boosts
    head_dim / 4 channels, so the layer is built by hand); the append of the chunk too."""
    from kitty_amd.kvcache.utils_kv_per_layer import KVCache_Layer
    B, H_KV, H_Q, T0, Tq, max_len = 2, 2, 8, 32 + 128 * 3 + 40, 170, 1024
    cache = K.KittyCache(K.u.cfg(H_KV, H_Q), B, max_len)
    cache.d_boosted = 0
    cache.kv_cache[0] = KVCache_Layer(MAX_BS=B, MAX_LEN=max_len, H_KV=H_KV, D=128, D_BOOSTED=0, LOW_BIT=2, HIGH_BIT=4,
                                      PAGE_SIZE=128, S=32, device="cuda")
    ol = O.OracleLayer(B, max_len, H_KV, D_BOOSTED=0)
    k, v = make_kv(B, H_KV, T0, seed=91)
    cache.update(K.u.to_dev(k), K.u.to_dev(v), 0)
    cache.quantize_prefill(0)
    ol.update(k, v)
    ol.quantize_prefill()
    assert K.u.layer_bytes_equal(cache.kv_cache[0], ol) == []
    got, q, kc, vc = _run(K, cache, ol, H_KV, H_Q, B, Tq, seed=92, what="no boosted channels")
    cache.append(K.u.to_dev(kc), K.u.to_dev(vc), 0)
    for t in range(Tq):
        ol.update(kc[:, :, t:t + 1], vc[:, :, t:t + 1])
        ol.quantize_decode()
    torch.cuda.synchronize()
    assert K.u.layer_bytes_equal(cache.kv_cache[0], ol) == []


def test_one_token_chunk_equals_decode(K):
    """T_q = 1 is a decode step: same result as appending the token and calling decode attention."""
    B, H_KV, H_Q, T0 = 2, 2, 8, 32 + 128 * 4 + 9
    cache, ol = _state(K, B, H_KV, H_Q, T0, 0, 1024, seed=3)
    got, q, kc, vc = _run(K, cache, ol, H_KV, H_Q, B, 1, seed=3)
    cache.update(K.u.to_dev(kc), K.u.to_dev(vc), 0)
    ol.update(kc, vc)
    kw = dict(reference_rounding=False)
    d = np.abs(O.decode_attention(ol, q, SC, dequant="two", **kw)
               - O.decode_attention(ol, q, SC, dequant="affine", **kw)).max()
    for variant in (0, 1):
        out, _ = K.attn(K.u.module(H_KV, H_Q), K.u.to_dev(q), cache.kv_cache[0], SC, variant=variant)
        dec = out.cpu().numpy().astype(np.float64)
        # two kernels, each within ATOL of its oracle; the matrix-core decode kernel's oracle is the
        # affine dequantization, d away from the two-rounding one this kernel follows
        bound = 2 * ATOL + (d if variant == 0 else 0.0)
        err = np.abs(dec - got).max()
        assert err <= bound, f"variant {variant}: {err:.3e} > {bound:.3e}"


def test_strided_query_and_chunk(K):
    """[B, T, H, D] projections viewed as [B, H, T, D] (what an attention module holds): no copy."""
    B, H_KV, H_Q, T0, Tq = 1, 2, 8, 32 + 128 + 40, 70
    cache, ol = _state(K, B, H_KV, H_Q, T0, 0, 1024, seed=8)
    kc, vc = make_kv(B, H_KV, Tq, seed=9)
    q = _q(B, H_Q, Tq, 9)
    qd = K.u.to_dev(q.transpose(0, 2, 1, 3)).transpose(1, 2)
    kd = K.u.to_dev(kc.transpose(0, 2, 1, 3)).transpose(1, 2)
    vd = K.u.to_dev(vc.transpose(0, 2, 1, 3)).transpose(1, 2)
    assert not qd.is_contiguous() and not kd.is_contiguous()
    out, _ = K.pre(K.u.module(H_KV, H_Q), qd, kd, vd, cache.kv_cache[0], SC)
    want = O.chunk_attention(ol, q, kc, vc, SC)
    assert np.abs(out.cpu().numpy().astype(np.float64) - want).max() <= ATOL


def test_ragged_prefix_per_sequence_counts(K):
    B, H_KV, H_Q, Tq = 3, 2, 8, 90
    max_len = 32 + 128 * 8
    cache = K.KittyCache(K.u.cfg(H_KV, H_Q), B, max_len)
    L = cache.kv_cache[0]
    rng = np.random.default_rng(5)
    ols, counts, dicts = [], [], []
    for b in range(B):
        T = int(rng.integers(40, max_len - 200))
        k, v = make_kv(1, H_KV, T + 60, seed=700 + b)
        ol = O.OracleLayer(1, max_len, H_KV)
        ol.update(k[:, :, :T], v[:, :, :T])
        ol.quantize_prefill()
        for s in range(int(rng.integers(0, 60))):
            ol.update(k[:, :, T + s:T + s + 1], v[:, :, T + s:T + s + 1])
            ol.quantize_decode()
        ols.append(ol)
        for name in ("Sink_Buffer_K", "Sink_Buffer_V", "Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V"):
            getattr(L, name)[b].copy_(K.u.to_dev(getattr(ol, name)[0]))
        for name in ("KeyCache", "KeyCache_metadata", "ValueCache", "ValueCache_metadata"):
            getattr(L, name)[b * L.MAX_PAGE:(b + 1) * L.MAX_PAGE].copy_(K.u.to_dev(getattr(ol, name)))
        counts.append([ol.Sink_Count, ol.PageCount_K, ol.Q_Buffer_Count_K, ol.PageCount_V, ol.Q_Buffer_Count_V,
                       ol.Local_Count_V, ol.Write_Offset_Local_V, 0])
    L.seq_counts = torch.tensor(counts, dtype=torch.int32, device="cuda")
    kc, vc = make_kv(B, H_KV, Tq, seed=55)
    q = _q(B, H_Q, Tq, 55)
    out, _ = K.pre(K.u.module(H_KV, H_Q), K.u.to_dev(q), K.u.to_dev(kc), K.u.to_dev(vc), L, SC)
    got = out.cpu().numpy().astype(np.float64)
    for b in range(B):
        want = O.chunk_attention(ols[b], q[b:b + 1], kc[b:b + 1], vc[b:b + 1], SC)
        assert np.abs(got[b:b + 1] - want).max() <= ATOL, b


def test_config3_scaled_down_student_t(K):
    """BASELINE config 3 at a size the oracle finishes in seconds: heavy-tailed keys, a packed
    prefix with residual, a chunk of several tiles."""
    B, H_KV, H_Q, T0, Tq = 2, 2, 8, 32 + 128 * 20 + 96, 512
    cache, ol = _state(K, B, H_KV, H_Q, T0, 0, 4096, seed=1003, student_t=True)
    _run(K, cache, ol, H_KV, H_Q, B, Tq, seed=1003, student_t=True, what="config 3 scaled")


@pytest.mark.parametrize("T0,steps,chunks", [(5, 0, [1, 30, 200]), (100, 0, [60, 300]), (32 + 128 * 2 + 96, 7, [25, 256, 131]),
                                             (0, 0, [50, 500])])
def test_append_on_device_equals_single_steps(K, T0, steps, chunks):
    """KittyCache.append: same counters, same packed pages bit for bit, same fp16 rows in the same
    slots as one update + quantize_decode per token (the oracle's definition)."""
    B, H_KV, H_Q = 2, 2, 8
    cache, ol = _state(K, B, H_KV, H_Q, T0, steps, 2048, seed=T0 + 11, student_t=True)
    k, v = make_kv(B, H_KV, sum(chunks), seed=T0 + 12, student_t=True)
    kd, vd = K.u.to_dev(k), K.u.to_dev(v)
    t = 0
    for c in chunks:
        cache.append(kd[:, :, t:t + c], vd[:, :, t:t + c], 0)
        ol.append(k[:, :, t:t + c], v[:, :, t:t + c])
        t += c
        assert K.u.layer_bytes_equal(cache.kv_cache[0], ol, live_q_rows_only=True) == []
    assert cache.get_seq_length(0) == T0 + steps + t


def test_chunk_then_append_then_decode(K):
    """The chunked-prefill call order: attend the chunk over the cache, append it, decode."""
    B, H_KV, H_Q, T0, Tq = 1, 2, 8, 32 + 128 * 3 + 96, 160
    cache, ol = _state(K, B, H_KV, H_Q, T0, 0, 2048, seed=21)
    got, q, kc, vc = _run(K, cache, ol, H_KV, H_Q, B, Tq, seed=21)
    cache.append(K.u.to_dev(kc), K.u.to_dev(vc), 0)
    ol.append(kc, vc)
    assert K.u.layer_bytes_equal(cache.kv_cache[0], ol, live_q_rows_only=True) == []
    q1 = _q(B, H_Q, 1, 22)
    out, _ = K.attn(K.u.module(H_KV, H_Q), K.u.to_dev(q1), cache.kv_cache[0], SC, variant=1)
    want = O.decode_attention(ol, q1, SC, reference_rounding=False, dequant="two")
    assert np.abs(out.cpu().numpy().astype(np.float64) - want).max() <= ATOL


def test_config3_full_size(K):
    """BASELINE config 3 at its real shape: B=4, 32 Q / 8 KV heads, a 2048-token chunk over a
    30720-token packed prefix (Student-t keys), then the append of the chunk.  The oracle cannot
    attend 8192 x 32768 scores per head in seconds, so: (i) sampled query rows of two batch rows
    are checked in float64 against the dequantized device cache, every cached and chunk token
    included; (ii) after the append the counters have the closed form, and sampled new pages are
    bit-exact against the oracle's quantizer."""
    B, H_KV, H_Q, T0, Tq = 4, 8, 32, 30720, 2048
    max_len = 32768 + 128
    gen = torch.Generator(device="cuda").manual_seed(1003)
    chi = torch.randn(B, H_KV, T0 + Tq, 128, 3, generator=gen, device="cuda").square_().sum(-1).div_(3).sqrt_()
    k = torch.randn(B, H_KV, T0 + Tq, 128, generator=gen, device="cuda") / chi          # Student-t, nu = 3
    del chi
    for h in range(H_KV):
        ch = torch.randperm(128, generator=torch.Generator().manual_seed(h))[:8]
        k[:, h, :, ch] *= 10.0
    k = k.clamp_(-6e4, 6e4).half()
    v = torch.randn(B, H_KV, T0 + Tq, 128, generator=gen, device="cuda").half()
    q = torch.randn(B, H_Q, Tq, 128, generator=gen, device="cuda").half()
    cache = K.KittyCache(K.u.cfg(H_KV, H_Q), B, max_len)
    cache.update(k[:, :, :T0], v[:, :, :T0], 0)
    cache.quantize_prefill(0)
    L = cache.kv_cache[0]
    assert (L.PageCount_K, L.PageCount_V, L.Q_Buffer_Count_K, L.Q_Buffer_Count_V, L.Local_Count_V) == (239, 238, 96, 96, 128)
    kc, vc = k[:, :, T0:], v[:, :, T0:]
    out, _ = K.pre(K.u.module(H_KV, H_Q), q, kc, vc, L, SC)
    torch.cuda.synchronize()
    got = out.cpu().numpy().astype(np.float64)
    assert np.isfinite(got).all()
    ol = K.u.oracle_from_layer(L, max_len)
    rows = np.array([0, 1, 63, 64, 127, 128, 1000, 1999, 2047])
    G = H_Q // H_KV
    for b in (0, 3):
        Kd, Vd = O.gather_dense_kv(ol, b, dequant="two")                    # [H_KV, T0, D]
        Kc = np.concatenate([Kd.astype(np.float64), kc[b].cpu().numpy().astype(np.float64)], axis=1)
        Vc = np.concatenate([Vd.astype(np.float64), vc[b].cpu().numpy().astype(np.float64)], axis=1)
        qb = q[b].cpu().numpy().astype(np.float64)
        for hq in range(H_Q):
            s = qb[hq, rows] @ Kc[hq // G].T * SC                           # [rows, T0 + Tq]
            s = np.where(np.arange(T0 + Tq)[None, :] > (T0 + rows)[:, None], -np.inf, s)
            e = np.exp(s - s.max(axis=1, keepdims=True))
            want = (e / e.sum(axis=1, keepdims=True)) @ Vc[hq // G]
            err = np.abs(got[b, rows, hq] - want).max()
            assert err <= ATOL, f"b={b} hq={hq}: {err:.3e}"
    # the append: 2048 tokens, 16 K pages and 16 V pages per (b, h), residuals unchanged
    qk_before = L.Q_Buffer_K.cpu().numpy().copy()
    cache.append(kc, vc, 0)
    torch.cuda.synchronize()
    assert (L.PageCount_K, L.PageCount_V, L.Q_Buffer_Count_K, L.Q_Buffer_Count_V, L.Local_Count_V) == (255, 254, 96, 96, 128)
    assert cache.get_seq_length(0) == T0 + Tq
    lay = O.Layout(H_KV=H_KV)
    kcn = kc.cpu().numpy()
    KC, KM = L.KeyCache.cpu().numpy(), L.KeyCache_metadata.cpu().numpy()
    for b, h, page in ((0, 0, 239), (1, 3, 240), (3, 7, 254)):
        if page == 239:      # the page completed from the 96 buffered rows and the first 32 chunk rows
            x = np.concatenate([qk_before[b, h, :96], kcn[b, h, :32]], axis=0)
        else:
            lo = 32 + (page - 240) * 128
            x = kcn[b, h, lo:lo + 128]
        oc = np.zeros((1, lay.k_stride_h), np.uint8)
        om = np.zeros((1, 1, 128, 2), np.float16)
        O.quantize_pack_k(x[None, None], 0, 1, np.zeros((1, 1), np.int64), 0, oc, om, 128, 32)
        pg = b * L.MAX_PAGE + page
        assert np.array_equal(KC[pg, h * lay.k_stride_h:(h + 1) * lay.k_stride_h], oc[0]), (b, h, page)
        assert np.array_equal(KM[pg, h].view(np.uint16), om[0, 0].view(np.uint16)), (b, h, page)
    assert np.array_equal(L.Q_Buffer_K.cpu().numpy()[:, :, :96].view(np.uint16), kcn[:, :, -96:].view(np.uint16))


def test_prefill_rejects_bad_arguments(K):
    cache = K.KittyCache(K.u.cfg(2, 8), 1, 512)
    L = cache.kv_cache[0]
    z = lambda *s: torch.zeros(*s, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        K.pre(K.u.module(2, 8), z(1, 8, 4, 128), z(1, 2, 5, 128), z(1, 2, 5, 128), L, SC)     # chunk length
    with pytest.raises(ValueError):
        K.pre(K.u.module(2, 8), z(1, 8, 4, 128).float(), z(1, 2, 4, 128), z(1, 2, 4, 128), L, SC)
    with pytest.raises(AssertionError):
        K.pre(K.u.module(1, 32), z(1, 32, 4, 128), z(1, 1, 4, 128), z(1, 1, 4, 128), L, SC)   # group of 32
    with pytest.raises(RuntimeError):
        K.pre(K.u.module(2, 8), z(1, 8, 4, 128).cpu(), z(1, 2, 4, 128), z(1, 2, 4, 128), L, SC)
