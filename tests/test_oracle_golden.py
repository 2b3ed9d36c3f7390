"""The oracle against the reference's own outputs (golden vectors) and against closed forms.

The golden files hold what the reference's quantize_pack_k / quantize_pack_v
(kitty_quant_pack.py:253-356) wrote for seeded inputs when run through Triton's CPU
interpreter (tests/golden/make_quant_golden.py).
"""
import glob
import os

import numpy as np
import pytest

from oracle import kitty_oracle as O

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "quant_*.npz")))


def _slot_maps(g, lay):
    x = g["x"]
    B, H, _, D = x.shape
    P, po, pt = int(g["pages"]), int(g["page_offset"]), g["page_table"]
    sm = np.zeros((B, H, P, D), np.uint8)
    for b in range(B):
        for p in range(P):
            for h in range(H):
                o = h * lay.k_stride_h
                sm[b, h, p] = g["key_cache"][pt[b, po + p], o + lay.k_off_idx: o + lay.k_stride_h]
    return sm


def test_golden_files_present():
    assert len(GOLDEN) == 6
    dims = sorted(int(np.load(p)["x"].shape[-1]) for p in GOLDEN)
    assert dims == [64, 128, 128, 128, 128, 256]     # head dimensions 64 and 256 boost 16 and 64 channels


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_quantizer_matches_reference_output(path):
    g = np.load(path)
    x = g["x"]
    B, H, _, D = x.shape
    P, t0, po, pt = int(g["pages"]), int(g["t_offset"]), int(g["page_offset"]), g["page_table"]
    DB = int(g["d_boost"])
    assert DB == D // 4
    lay = O.Layout(H_KV=H, D=D, D_BOOSTED=DB)
    sm = _slot_maps(g, lay)
    kc, km = np.zeros_like(g["key_cache"]), np.zeros_like(g["key_meta"])
    vc, vm = np.zeros_like(g["value_cache"]), np.zeros_like(g["value_meta"])
    O.quantize_pack_k(x, t0, P, pt, po, kc, km, 128, DB, slot_map=sm)
    O.quantize_pack_v(x, t0, P, pt, po, vc, vm, 128)
    # V: bytes and metadata bit-exact, including untouched pages (zeros)
    assert np.array_equal(vc, g["value_cache"])
    assert np.array_equal(vm.view(np.uint16), g["value_meta"].view(np.uint16))
    # K: metadata bit-exact; low plane and slot map bit-exact on every page
    assert np.array_equal(km.view(np.uint16), g["key_meta"].view(np.uint16))
    gk = g["key_cache"].reshape(-1, H, lay.k_stride_h)
    ok = kc.reshape(-1, H, lay.k_stride_h)
    assert np.array_equal(ok[:, :, : lay.k_off_hi], gk[:, :, : lay.k_off_hi])
    assert np.array_equal(ok[:, :, lay.k_off_idx:], gk[:, :, lay.k_off_idx:])
    # K high plane.  The reference computes the row offset as uint8(slot) * 32 in uint8
    # arithmetic (kitty_quant_pack.py:140), so slot s lands in row s % 8 and four boosted
    # channels collide per row; the CPU interpreter keeps the last writer (largest channel).
    # This build stores slot s in row s.  What the reference kept must equal our row of the
    # winning slot, and its rows 8 .. d_boost - 1 were never written (the same wrap for 16 and 64 slots).
    for b in range(B):
        for p in range(P):
            pg = pt[b, po + p]
            for h in range(H):
                ghi = gk[pg, h, lay.k_off_hi: lay.k_off_idx].reshape(DB, 32)
                ohi = ok[pg, h, lay.k_off_hi: lay.k_off_idx].reshape(DB, 32)
                assert not ghi[8:].any()
                idx = sm[b, h, p]
                for r in range(8):
                    chans = [d for d in range(D) if idx[d] < DB and idx[d] % 8 == r]
                    winner = idx[max(chans)]
                    assert np.array_equal(ghi[r], ohi[winner]), (b, p, h, r)


TIE_FREE = [p for p in GOLDEN if any(k in p for k in ("spread", "d64", "d256"))]


@pytest.mark.parametrize("path", TIE_FREE, ids=[os.path.basename(p) for p in TIE_FREE])
def test_selection_matches_reference_when_tie_free(path):
    g = np.load(path)
    x = g["x"]
    B, H, _, D = x.shape
    DB, t0 = int(g["d_boost"]), int(g["t_offset"])
    lay = O.Layout(H_KV=H, D=D, D_BOOSTED=DB)
    sm = _slot_maps(g, lay)
    n = 0
    for b in range(B):
        for p in range(int(g["pages"])):
            for h in range(H):
                xx = x[b, h, t0 + p * 128: t0 + (p + 1) * 128]
                assert O.boost_is_tie_free(xx, DB)
                assert np.array_equal(O.select_boost(xx, DB), sm[b, h, p])
                n += 1
    assert n == B * H * int(g["pages"]) >= 1


def test_selection_same_scores_on_tied_pages():
    """On tied pages torch.topk's order is unspecified, but the *scores* of the channels the
    reference picked must be the 32 largest of the oracle's scores (as a multiset)."""
    for path in GOLDEN:
        g = np.load(path)
        x = g["x"]
        B, H, _, D = x.shape
        DB = int(g["d_boost"])
        lay = O.Layout(H_KV=H, D=D, D_BOOSTED=DB)
        sm = _slot_maps(g, lay)
        t0 = int(g["t_offset"])
        for b in range(B):
            for p in range(int(g["pages"])):
                for h in range(H):
                    xx = x[b, h, t0 + p * 128: t0 + (p + 1) * 128]
                    sc = O.boost_score(xx).astype(np.float64)
                    ref_sorted = np.sort(sc[sm[b, h, p] < DB])[::-1]
                    ours_sorted = np.sort(sc)[::-1][:DB]
                    assert np.array_equal(ref_sorted, ours_sorted)
                    # the reference's slot order is descending in score as well
                    by_slot = sc[np.argsort(np.where(sm[b, h, p] < DB, sm[b, h, p], 255))[:DB]]
                    assert np.all(np.diff(by_slot) <= 0)


# ---- closed-form known answers ------------------------------------------------------------------
def test_layout_sizes():
    lay = O.Layout(H_KV=8)
    assert (lay.k_stride_d, lay.k_off_hi, lay.k_off_idx, lay.k_stride_h) == (32, 4096, 5120, 5248)
    assert lay.bytes_per_page_K == 41984 and lay.bytes_per_page_V == 32768
    assert lay.v_stride_t == 32 and lay.v_stride_h == 4096


def test_v_known_answer_bytes():
    lay = O.Layout(H_KV=1)
    x = np.zeros((128, 128), np.float16)
    x[:] = (np.arange(128) % 4) * 0.25            # 4 equally spaced levels -> codes 0,1,2,3
    by, meta = O.pack_v_page(x, lay)
    assert np.all(by == 0xE4)
    assert np.all(meta[:, 0] == np.float16(0.25)) and np.all(meta[:, 1] == 0)


def test_k_known_answer_bytes():
    lay = O.Layout(H_KV=1)
    x = np.zeros((128, 128), np.float16)
    x[:, 5] = (np.arange(128) % 16) * 0.5          # boosted: 16 levels -> codes 0..15 over tokens
    x[:, 9] = (np.arange(128) % 4) * 2.0           # not boosted: codes 0..3
    idx = np.full(128, 32, np.uint8)
    idx[5] = 7
    by, meta = O.pack_k_page(x, idx, lay)
    assert np.all(by[5 * 32: 6 * 32] == 0xE4)                       # low bits of 0..15 cycle 0,1,2,3
    hi = by[4096 + 7 * 32: 4096 + 8 * 32]
    assert np.array_equal(hi, np.tile(np.array([0x00, 0x55, 0xAA, 0xFF], np.uint8), 8))
    assert np.all(by[9 * 32: 10 * 32] == 0xE4)
    assert not by[4096: 4096 + 7 * 32].any() and not by[4096 + 8 * 32: 5120].any()
    assert np.array_equal(by[5120:], idx)
    assert meta[5, 0] == np.float16(0.5) and meta[9, 0] == np.float16(2.0)
    # constant channel: scale floors at 1e-6 (fp16 subnormal 0x0011), codes 0
    assert meta[0].view(np.uint16)[0] == 0x0011 and not by[:32].any()


def test_brute_force_scalar_loop():
    """A scalar Python restatement (one element at a time, struct-free fp32 via numpy scalars)."""
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((128, 128)) * rng.uniform(0.1, 20, size=(1, 128))).astype(np.float16)
    lay = O.Layout(H_KV=1)
    idx = O.select_boost(x, 32)
    by, meta = O.pack_k_page(x, idx, lay)
    f = np.float32
    for d in [0, 1, 17, 64, 127] + list(np.nonzero(idx < 32)[0][:3]):
        col = [f(v) for v in x[:, d]]
        mn, mx = min(col), max(col)
        qmax = f(15.0) if idx[d] < 32 else f(3.0)
        s = f(f(mx - mn) / qmax)
        if s < f(1e-6):
            s = f(1e-6)
        assert np.float16(s) == meta[d, 0] and np.float16(mn) == meta[d, 1]
        for t in range(128):
            q = int(min(max(np.floor(f(f(col[t] - mn) / s) + f(0.5)), f(0)), qmax))
            lo = (by[d * 32 + t // 4] >> (2 * (t % 4))) & 3
            assert lo == (q & 3)
            if idx[d] < 32:
                hi = (by[4096 + int(idx[d]) * 32 + t // 4] >> (2 * (t % 4))) & 3
                assert hi == (q >> 2)
            else:
                assert q < 4
    vb, vmeta = O.pack_v_page(x, lay)
    for t in [0, 3, 127]:
        row = [f(v) for v in x[t]]
        mn, mx = min(row), max(row)
        s = f(f(mx - mn) / f(3.0))
        s = f(1e-6) if s < f(1e-6) else s
        assert np.float16(s) == vmeta[t, 0] and np.float16(mn) == vmeta[t, 1]
        for d in range(128):
            q = int(min(max(np.floor(f(f(row[d] - mn) / s) + f(0.5)), f(0)), f(3)))
            assert ((vb[t * 32 + d // 4] >> (2 * (d % 4))) & 3) == q


def test_quantize_dequantize_error_bound_and_extremes():
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((128, 128)) * rng.uniform(0.5, 12, size=(1, 128))).astype(np.float16)
    lay = O.Layout(H_KV=1)
    idx = O.select_boost(x, 32)
    by, meta = O.pack_k_page(x, idx, lay)
    codes = O.k_codes_from_page(by, lay)
    xf = x.astype(np.float64)
    qmax = np.where(idx < 32, 15, 3)
    assert np.all(codes[xf.argmin(axis=0), np.arange(128)] == 0)          # min -> code 0
    assert np.all(codes[xf.argmax(axis=0), np.arange(128)] == qmax)       # max -> qmax
    deq = O.dequant_k_page(by, meta, lay).astype(np.float64)
    s = meta[:, 0].astype(np.float64)[None, :]
    # half a step + fp16 rounding of scale, product and sum
    bound = s / 2 + np.abs(xf) * 2.0 ** -9 + s * qmax[None, :] * 2.0 ** -10
    assert np.all(np.abs(deq - xf) <= bound)
    # boosted channels really are finer: their step is range/15
    rng_ = (xf.max(axis=0) - xf.min(axis=0))
    assert np.allclose(s[0][idx < 32], (rng_ / 15)[idx < 32], rtol=2e-3)
    assert np.allclose(s[0][idx >= 32], (rng_ / 3)[idx >= 32], rtol=2e-3)
    vb, vmeta = O.pack_v_page(x, lay)
    vdeq = O.dequant_v_page(vb, vmeta, lay).astype(np.float64)
    vs = vmeta[:, 0].astype(np.float64)[:, None]
    assert np.all(np.abs(vdeq - xf) <= vs / 2 + np.abs(xf) * 2.0 ** -9 + vs * 3 * 2.0 ** -10)


def test_high_plane_of_unboosted_slots_is_preserved():
    lay = O.Layout(H_KV=1, D_BOOSTED=32)
    x = np.random.default_rng(1).standard_normal((128, 128)).astype(np.float16)
    idx = np.full(128, 32, np.uint8)
    idx[3] = 0                                     # a single boosted channel in slot 0
    prev = np.full(lay.k_stride_h, 0x5A, np.uint8)
    by, _ = O.pack_k_page(x, idx, lay, prev=prev)
    assert np.all(by[4096 + 32: 5120] == 0x5A)     # slots 1..31 untouched
    by0, _ = O.pack_k_page(x, idx, lay)
    assert not by0[4096 + 32: 5120].any()


def test_d_boost_zero_is_pure_two_bit():
    lay = O.Layout(H_KV=1, D_BOOSTED=0)
    x = np.random.default_rng(2).standard_normal((128, 128)).astype(np.float16)
    idx = O.select_boost(x, 0)
    assert np.all(idx == 0)
    by, meta = O.pack_k_page(x, idx, lay)
    assert by.shape[0] == 4096 + 128
    assert O.k_codes_from_page(by, lay).max() <= 3
