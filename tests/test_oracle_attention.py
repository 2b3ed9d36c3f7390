"""The oracle's attention restatement against textbook attention and closed forms."""
import numpy as np
import pytest

from oracle import kitty_oracle as O
from tests.helpers import make_kv, make_q


def _layer(T, H_KV=2, seed=0, steps=0, B=1):
    k, v = make_kv(B, H_KV, T + steps, seed=seed)
    ol = O.OracleLayer(B, 2048, H_KV)
    ol.update(k[:, :, :T], v[:, :, :T])
    ol.quantize_prefill()
    for s in range(steps):
        ol.update(k[:, :, T + s:T + s + 1], v[:, :, T + s:T + s + 1])
        ol.quantize_decode()
    return ol, k, v


def _softmax_attention(q, K, V, scaling):
    s = K.astype(np.float64) @ q.astype(np.float64) * scaling
    e = np.exp(s - s.max())
    return (e / e.sum()) @ V.astype(np.float64)


@pytest.mark.parametrize("T", [1, 5, 32])
def test_short_prompt_is_plain_fp16_attention(T):
    """With at most 32 tokens everything sits in the fp16 sink: no quantization is involved."""
    ol, k, v = _layer(T, seed=T)
    q = make_q(1, 8, seed=T)
    out = O.decode_attention(ol, q, 128 ** -0.5, reference_rounding=False)
    for hq in range(8):
        want = _softmax_attention(q[0, hq, 0], k[0, hq // 4, :T], v[0, hq // 4, :T], 128 ** -0.5)
        assert np.allclose(out[0, 0, hq], want, atol=1e-12)


def test_token_order_sink_pages_qbuffer_ring():
    """gather_dense_kv returns tokens in chronological order on both sides, ring offset included:
    every fp16 row equals the original token, every packed row is within half a step of it."""
    ol, k, v = _layer(32 + 128 * 2 + 70, seed=3, steps=200)
    assert ol.Write_Offset_Local_V != 0
    T = ol.get_total_length()
    Kd, Vd = O.gather_dense_kv(ol, 0)
    assert Kd.shape == (2, T, 128) and Vd.shape == (2, T, 128)
    nk = 32 + 128 * ol.PageCount_K
    nv = 32 + 128 * ol.PageCount_V
    assert np.array_equal(Kd[:, :32], k[0, :, :32]) and np.array_equal(Kd[:, nk:], k[0, :, nk:T])
    assert np.array_equal(Vd[:, :32], v[0, :, :32]) and np.array_equal(Vd[:, nv:], v[0, :, nv:T])
    assert np.abs(Vd[:, 32:nv].astype(np.float64) - v[0, :, 32:nv].astype(np.float64)).max() < 1.6   # range/3/2 of N(0,1)
    err = np.abs(Kd[:, 32:nk].astype(np.float64) - k[0, :, 32:nk].astype(np.float64))
    assert err.max() < 0.5 * 100 / 3 and np.median(err) < 0.6


def test_dequant_modes_are_ordered():
    """'fma' and 'two' are roundings of 'affine': each within one fp16 ulp of it per element."""
    ol, _, _ = _layer(32 + 128 * 2 + 10, seed=9)
    lay = ol.lay
    by, meta = ol.KeyCache[0, : lay.k_stride_h], ol.KeyCache_metadata[0, 0]
    a = O.dequant_k_page(by, meta, lay, "affine")
    f = O.dequant_k_page(by, meta, lay, "fma").astype(np.float64)
    t = O.dequant_k_page(by, meta, lay, "two").astype(np.float64)
    ulp = np.maximum(np.abs(a), 2.0 ** -14) * 2.0 ** -10
    assert np.all(np.abs(f - a) <= ulp / 2 + 1e-12)
    s = meta[:, 0].astype(np.float64)[None, :]
    assert np.all(np.abs(t - a) <= ulp / 2 + 15 * s * 2.0 ** -11 + 1e-12)
    assert a.dtype == np.float64 and O.dequant_k_page(by, meta, lay, "two").dtype == np.float16


def test_reference_rounding_stays_close_to_float64():
    ol, _, _ = _layer(32 + 128 * 4 + 3, seed=21)
    q = make_q(1, 8, seed=2)
    ref = O.decode_attention(ol, q, 128 ** -0.5).astype(np.float64)
    exact = O.decode_attention(ol, q, 128 ** -0.5, reference_rounding=False)
    assert ref.shape == (1, 1, 8, 128) and np.abs(ref - exact).max() < 2e-2


def test_per_sequence_counts_override():
    ol, _, _ = _layer(32 + 128 * 3 + 20, seed=4, B=2)
    q = make_q(2, 8, seed=4)
    full = O.decode_attention(ol, q, 0.1, reference_rounding=False)
    same = O.decode_attention(ol, q, 0.1, reference_rounding=False, seq_counts=[None, {}])
    assert np.array_equal(full, same)
    short = O.decode_attention(ol, q, 0.1, reference_rounding=False,
                               seq_counts=[dict(pk=1, rk=0, pv=0, rv=0, lv=128, off=0), None])
    assert not np.allclose(short[0], full[0]) and np.array_equal(short[1], full[1])


def test_prefill_attention_is_causal():
    rng = np.random.default_rng(0)
    H_Q, H_KV, T0, Tq, D = 4, 2, 10, 6, 16
    K = rng.standard_normal((H_KV, T0 + Tq, D)).astype(np.float16)
    V = rng.standard_normal((H_KV, T0 + Tq, D)).astype(np.float16)
    q = rng.standard_normal((H_Q, Tq, D)).astype(np.float16)
    out = O.prefill_attention(q, K, V, 0.3, T0)
    for hq in range(H_Q):
        for i in range(Tq):
            n = T0 + i + 1
            want = _softmax_attention(q[hq, i], K[hq // 2, :n], V[hq // 2, :n], 0.3)
            assert np.allclose(out[hq, i], want, atol=1e-12)


def test_sim_baseline_shapes_and_levels():
    import torch
    from oracle import sim_baseline as S
    torch.manual_seed(0)
    K = torch.randn(1, 2, 32 + 128 * 2 + 9, 128).half()
    V = torch.randn(1, 2, 32 + 128 * 2 + 9, 128).half()
    K0, V0 = K.clone(), V.clone()
    S.simulate_prefill(K, V)
    assert torch.equal(K[:, :, :32], K0[:, :, :32]) and torch.equal(K[:, :, -9:], K0[:, :, -9:])
    assert torch.equal(V[:, :, -128:], V0[:, :, -128:])
    grp = K[0, 0, 32:160].float()
    levels = [len(torch.unique(grp[:, d])) for d in range(128)]
    assert max(levels) <= 16 and sorted(levels)[64] <= 4          # 25 % of channels at 4 bit, the rest at 2
    assert len(torch.unique(V[0, 0, 40].float())) <= 4
    out = S.eager_attention(torch.randn(1, 8, 1, 128).half(), K, V, 128 ** -0.5, 4)
    assert tuple(out.shape) == (1, 1, 8, 128)


def test_rope_restatement_equals_torch_fp16_operators():
    """oracle.rope_fp16 against the caller's expression evaluated by torch's own fp16 operators
    (modeling_qwen3.py:98-102, 125-128: q * cos + rotate_half(q) * sin on fp16 tensors), bit for bit,
    and the two closed forms a rotation has: angle 0 is the identity, angle pi/2 swaps the halves."""
    import torch
    rng = np.random.default_rng(5)
    B, H, T, D = 3, 2, 4, 128
    x = (rng.standard_normal((B, H, T, D)) * 4).astype(np.float16)
    pos = rng.integers(0, 100000, size=(B, T)).astype(np.float64)
    inv = 1.0 / (500000.0 ** (np.arange(0, D, 2) / D))
    ang = pos[..., None] * inv
    cos = np.concatenate([np.cos(ang), np.cos(ang)], -1).astype(np.float16)       # [B, T, D]
    sin = np.concatenate([np.sin(ang), np.sin(ang)], -1).astype(np.float16)
    got = O.rope_fp16(x, cos, sin)
    xt, ct, st = torch.from_numpy(x), torch.from_numpy(cos).unsqueeze(1), torch.from_numpy(sin).unsqueeze(1)
    rot = torch.cat((-xt[..., D // 2:], xt[..., : D // 2]), dim=-1)
    want = (xt * ct) + (rot * st)
    assert want.dtype == torch.float16
    assert np.array_equal(got.view(np.uint16), want.numpy().view(np.uint16))
    one, zero = np.ones((B, T, D), np.float16), np.zeros((B, T, D), np.float16)
    assert np.array_equal(O.rope_fp16(x, one, zero), x)
    quarter = O.rope_fp16(x, zero, one)
    assert np.array_equal(quarter[..., : D // 2], -x[..., D // 2:]) and np.array_equal(quarter[..., D // 2:], x[..., : D // 2])
