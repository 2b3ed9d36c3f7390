"""CPU oracle for Kitty's quantized-KV hot path (numpy).  TEST INFRASTRUCTURE ONLY.

This file restates, on the CPU, the arithmetic of the reference's packed-KV
path so that the HIP kernels can be checked against it.  It is the checker,
never the product: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it.  Nothing under
``kitty_amd/`` imports it and the product path has no CPU fallback.

Reference files restated here (paths relative to the reference checkout):

* ``src/kitty/kvcache/utils_kv_per_layer.py:12-95``   storage layout, counters
* ``src/kitty/kvcache/kernels/kitty_quant_pack.py``    quantize + bit-pack (K and V)
* ``src/kitty/kvcache/kernels/kitty_attention.py``     decode attention over packed KV
* ``src/kitty/kvcache/kitty.py:63-241``                append / flush state machine

How each function is pinned (what a wrong restatement would fail):

* ``quantize_group`` / ``pack_k_page`` / ``pack_v_page`` / ``quantize_pack_k`` /
  ``quantize_pack_v``: golden vectors under ``tests/golden/quant_*.npz`` produced
  by the reference's own ``quantize_pack_k/v`` run through Triton's CPU
  interpreter (script ``tests/golden/make_quant_golden.py``; head dimension 128
  with 32 boosted channels in four cases, 64 with 16 and 256 with 64 in one each),
  plus closed-form known-answer bytes and a scalar brute-force loop.
* ``select_boost``: the score is pinned by the golden slot maps wherever the
  reference's scores are tie-free; the tie rule (descending score, then
  ascending channel) is this build's canonical choice because ``torch.topk``
  leaves tie order unspecified - the *order among tied channels* is therefore
  "parity unpinned" against the reference and is documented as such.
* ``dequant_*`` / ``decode_attention``: floating point; pinned by reduction to
  textbook GQA attention in float64 over the dequantized cache, by special
  cases (all-equal keys, short prompts, d_boost=0) and by quantize/dequantize
  error bounds.  Tolerance for the HIP path is max-abs 2e-3 in fp16.
* ``OracleLayer`` (state machine): conservation and closed-form occupancy
  properties in ``tests/test_state_machine.py``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Optional

import numpy as np

F16 = np.float16
F32 = np.float32


# ----------------------------------------------------------------------------------------------
# layout (utils_kv_per_layer.py:33-46, kitty_quant_pack.py:42-45,180-181)
# ----------------------------------------------------------------------------------------------
@dataclass(frozen=True)
class Layout:
    H_KV: int
    D: int = 128
    D_BOOSTED: int = 32
    PAGE_SIZE: int = 128

    @property
    def k_stride_d(self) -> int:          # bytes per channel row of a 2-bit plane
        return self.PAGE_SIZE * 2 // 8

    @property
    def k_off_hi(self) -> int:
        return self.k_stride_d * self.D

    @property
    def k_off_idx(self) -> int:
        return self.k_stride_d * (self.D + self.D_BOOSTED)

    @property
    def k_stride_h(self) -> int:
        return self.k_off_idx + self.D

    @property
    def v_stride_t(self) -> int:
        return self.D * 2 // 8

    @property
    def v_stride_h(self) -> int:
        return self.v_stride_t * self.PAGE_SIZE

    @property
    def bytes_per_page_K(self) -> int:
        return self.H_KV * self.k_stride_h

    @property
    def bytes_per_page_V(self) -> int:
        return self.H_KV * self.v_stride_h


# ----------------------------------------------------------------------------------------------
# quantizer arithmetic (kitty_quant_pack.py:75-82,106-112 for K; :201-204,227-230 for V)
# ----------------------------------------------------------------------------------------------
def quantize_group(x: np.ndarray, qmax: np.ndarray, axis: int):
    """Asymmetric min/max quantization of fp16 ``x`` along ``axis``.

    ``qmax`` broadcasts against the reduced shape (keepdims).  All arithmetic is
    IEEE fp32: Triton promotes fp16 reductions and ``fp16 / python-float`` to fp32,
    so ``max-min``, the divide, ``x-min`` and the second divide are fp32 operations
    and only the *stored* scale is rounded to fp16.
    Returns (codes uint8, scale fp16, zero fp16) with scale/zero keepdims-shaped.
    """
    assert x.dtype == F16
    xf = x.astype(F32)
    mx = xf.max(axis=axis, keepdims=True)
    mn = xf.min(axis=axis, keepdims=True)
    qmax = np.asarray(qmax, dtype=F32)
    scale = ((mx - mn).astype(F32) / qmax).astype(F32)
    scale = np.where(scale < F32(1e-6), F32(1e-6), scale).astype(F32)
    xq = np.floor(((xf - mn).astype(F32) / scale).astype(F32) + F32(0.5)).astype(F32)
    xq = np.minimum(np.maximum(xq, F32(0.0)), qmax)
    return xq.astype(np.uint8), scale.astype(F16), mn.astype(F16)


def pack2(codes: np.ndarray) -> np.ndarray:
    """Pack 2-bit codes along the last axis, 4 per byte, element i in bits 2*(i%4) (LSB first)."""
    c = (codes & 3).astype(np.uint8).reshape(*codes.shape[:-1], codes.shape[-1] // 4, 4)
    return (c[..., 0] | (c[..., 1] << 2) | (c[..., 2] << 4) | (c[..., 3] << 6)).astype(np.uint8)


def unpack2(b: np.ndarray) -> np.ndarray:
    out = np.stack([(b >> s) & 3 for s in (0, 2, 4, 6)], axis=-1)
    return out.reshape(*b.shape[:-1], b.shape[-1] * 4).astype(np.uint8)


def pack_k_page(x: np.ndarray, idx: np.ndarray, lay: Layout, prev: Optional[np.ndarray] = None):
    """One K page-head.  x fp16 [PAGE, D]; idx uint8 [D] (slot, or D_BOOSTED = not boosted).

    Returns (bytes uint8 [k_stride_h], meta fp16 [D, 2]).  ``prev`` is the previous content
    of the page-head (the reference writes the high plane with a mask, so slots no channel
    maps to keep their old bytes - kitty_quant_pack.py:137-144).
    """
    PAGE, D, DB = lay.PAGE_SIZE, lay.D, lay.D_BOOSTED
    assert x.shape == (PAGE, D) and idx.shape == (D,)
    boost = idx < DB
    qmax = np.where(boost, F32(15.0), F32(3.0))[None, :]
    codes, scale, zero = quantize_group(x, qmax, axis=0)          # codes [PAGE, D]
    out = np.zeros(lay.k_stride_h, np.uint8) if prev is None else prev.copy()
    lo = pack2(codes.T)                                           # [D, PAGE/4]
    out[: lay.k_off_hi] = lo.reshape(-1)
    hi = pack2((codes.T >> 2) & 3)                                # [D, PAGE/4]
    hi_view = out[lay.k_off_hi: lay.k_off_idx].reshape(DB, lay.k_stride_d)
    for d in np.nonzero(boost)[0]:
        hi_view[int(idx[d])] = hi[d]
    out[lay.k_off_idx:] = idx
    meta = np.stack([scale[0], zero[0]], axis=-1).astype(F16)     # [D, 2]
    return out, meta


def pack_v_page(x: np.ndarray, lay: Layout):
    """One V page-head.  x fp16 [PAGE, D].  Returns (bytes [v_stride_h], meta fp16 [PAGE, 2])."""
    codes, scale, zero = quantize_group(x, F32(3.0), axis=1)      # per token over channels
    out = pack2(codes).reshape(-1)                                # token-major, 4 channels per byte
    meta = np.stack([scale[:, 0], zero[:, 0]], axis=-1).astype(F16)
    return out, meta


# ----------------------------------------------------------------------------------------------
# channel-boost selection (kitty_quant_pack.py:280-288)
# ----------------------------------------------------------------------------------------------
def boost_score(x: np.ndarray) -> np.ndarray:
    """score[d] = fp16( mean_t |x[t, d]| ): exact sum (float64 holds it exactly) rounded once."""
    return (np.abs(x.astype(np.float64)).sum(axis=-2) / x.shape[-2]).astype(F16)


def select_boost(x: np.ndarray, d_boost: int) -> np.ndarray:
    """Slot map for one page-head (x fp16 [PAGE, D]): idx[ch] = rank in the top-``d_boost``
    by score, else ``d_boost``.  Ties: higher score first, then lower channel index."""
    score = boost_score(x)
    D = score.shape[-1]
    order = np.argsort(-score.astype(np.float64), kind="stable")
    idx = np.full(D, d_boost, np.uint8)
    idx[order[:d_boost]] = np.arange(d_boost, dtype=np.uint8)
    return idx


def boost_is_tie_free(x: np.ndarray, d_boost: int) -> bool:
    """True when the top-(d_boost+1) scores are pairwise distinct, i.e. any correct top-k agrees."""
    s = np.sort(boost_score(x).astype(np.float64))[::-1][: d_boost + 1]
    return bool(np.all(np.diff(s) < 0))


# ----------------------------------------------------------------------------------------------
# wrappers with the reference's signatures (kitty_quant_pack.py:253-266, 315-327)
# ----------------------------------------------------------------------------------------------
def quantize_pack_k(key_states, key_states_t_offset, key_states_page_count, page_table_k, page_offset_k,
                    cache, cache_metadata, page_size, d_boost, slot_map=None):
    """numpy arrays in place of tensors.  ``slot_map`` uint8 [B,H,P,D] overrides the selection
    (the reference kernel's own boundary: it consumes the map, kitty_quant_pack.py:58-65)."""
    B, H, _, D = key_states.shape
    lay = Layout(H_KV=H, D=D, D_BOOSTED=d_boost, PAGE_SIZE=page_size)
    used = np.zeros((B, H, key_states_page_count, D), np.uint8)
    for b in range(B):
        for p in range(key_states_page_count):
            pg = int(page_table_k[b, page_offset_k + p])
            t0 = key_states_t_offset + p * page_size
            for h in range(H):
                x = np.ascontiguousarray(key_states[b, h, t0: t0 + page_size, :])
                idx = select_boost(x, d_boost) if slot_map is None else slot_map[b, h, p]
                used[b, h, p] = idx
                o = h * lay.k_stride_h
                by, meta = pack_k_page(x, idx, lay, prev=cache[pg, o: o + lay.k_stride_h])
                cache[pg, o: o + lay.k_stride_h] = by
                cache_metadata[pg, h] = meta
    return used


def quantize_pack_v(value_states, t_offset, page_count, page_table_v, page_offset_v,
                    cache, cache_metadata, page_size):
    B, H, _, D = value_states.shape
    lay = Layout(H_KV=H, D=D, PAGE_SIZE=page_size)
    for b in range(B):
        for p in range(page_count):
            pg = int(page_table_v[b, page_offset_v + p])
            t0 = t_offset + p * page_size
            for h in range(H):
                x = np.ascontiguousarray(value_states[b, h, t0: t0 + page_size, :])
                by, meta = pack_v_page(x, lay)
                o = h * lay.v_stride_h
                cache[pg, o: o + lay.v_stride_h] = by
                cache_metadata[pg, h] = meta


# ----------------------------------------------------------------------------------------------
# dequantization as the attention kernels see it (kitty_attention.py:130-165, 307-320)
# ----------------------------------------------------------------------------------------------
def k_codes_from_page(by: np.ndarray, lay: Layout) -> np.ndarray:
    """uint8 codes [PAGE, D] (0..15 on boosted channels, 0..3 elsewhere) of one K page-head."""
    lo = unpack2(by[: lay.k_off_hi].reshape(lay.D, lay.k_stride_d))              # [D, PAGE]
    idx = by[lay.k_off_idx: lay.k_off_idx + lay.D]
    hi_plane = unpack2(by[lay.k_off_hi: lay.k_off_idx].reshape(lay.D_BOOSTED, lay.k_stride_d))
    hi = np.zeros_like(lo)
    boost = idx < lay.D_BOOSTED
    hi[boost] = hi_plane[idx[boost].astype(np.int64)]
    return (lo | (hi << 2)).T.copy()


DEQUANT_MODES = ("two", "fma", "affine")


def _dequant(codes: np.ndarray, scale: np.ndarray, zero: np.ndarray, mode: str) -> np.ndarray:
    """``code * scale + zero`` on the stored fp16 scale / zero, in one of three roundings:

    ``"two"``    product and sum each rounded to fp16 - how eager torch and the Triton interpreter
                 evaluate kitty_attention.py:162-165 / :317-320 (the reference semantics; fp16 out);
    ``"fma"``    rounded once - what a compiled kernel that contracts the expression produces (fp16);
    ``"affine"`` not rounded at all - the value both of the above approximate (float64 out).
    """
    c64, s64, z64 = codes.astype(np.float64), scale.astype(np.float64), zero.astype(np.float64)
    if mode == "two":
        return ((codes.astype(F16) * scale).astype(F16) + zero).astype(F16)
    if mode == "fma":
        return (c64 * s64 + z64).astype(F16)          # exact in float64, then one rounding
    if mode == "affine":
        return c64 * s64 + z64
    raise ValueError(mode)


def dequant_k_page(by: np.ndarray, meta: np.ndarray, lay: Layout, mode: str = "two") -> np.ndarray:
    """[PAGE, D] dequantized keys of one page-head (see ``_dequant`` for ``mode``)."""
    codes = k_codes_from_page(by, lay)
    return _dequant(codes, meta[:, 0][None, :], meta[:, 1][None, :], mode)


def dequant_v_page(by: np.ndarray, meta: np.ndarray, lay: Layout, mode: str = "two") -> np.ndarray:
    codes = unpack2(by.reshape(lay.PAGE_SIZE, lay.v_stride_t))                    # [PAGE, D]
    return _dequant(codes, meta[:, 0][:, None], meta[:, 1][:, None], mode)


# ----------------------------------------------------------------------------------------------
# per-layer storage + append state machine (utils_kv_per_layer.py:12-95, kitty.py:63-236)
# ----------------------------------------------------------------------------------------------
@dataclass
class OracleLayer:
    MAX_BS: int
    MAX_LEN: int
    H_KV: int
    D: int = 128
    D_BOOSTED: int = 32
    PAGE_SIZE: int = 128
    S: int = 32
    lay: Layout = field(init=False)

    def __post_init__(self):
        assert self.PAGE_SIZE % 128 == 0
        self.lay = Layout(self.H_KV, self.D, self.D_BOOSTED, self.PAGE_SIZE)
        self.MAX_PAGE = math.ceil(self.MAX_LEN / self.PAGE_SIZE)
        n = self.MAX_BS * self.MAX_PAGE
        self.KeyCache = np.zeros((n, self.lay.bytes_per_page_K), np.uint8)
        self.KeyCache_metadata = np.zeros((n, self.H_KV, self.D, 2), F16)
        self.ValueCache = np.zeros((n, self.lay.bytes_per_page_V), np.uint8)
        self.ValueCache_metadata = np.zeros((n, self.H_KV, self.PAGE_SIZE, 2), F16)
        ident = (np.arange(self.MAX_PAGE)[None, :] + np.arange(self.MAX_BS)[:, None] * self.MAX_PAGE)
        self.PageTable_K = ident.astype(np.int64)
        self.PageTable_V = ident.astype(np.int64).copy()
        self.PageCount_K = 0
        self.PageCount_V = 0
        win = lambda n_: np.zeros((self.MAX_BS, self.H_KV, n_, self.D), F16)
        self.Sink_Buffer_K, self.Sink_Buffer_V = win(self.S), win(self.S)
        self.Sink_Count = 0
        self.Q_Buffer_K, self.Q_Buffer_V = win(self.PAGE_SIZE), win(self.PAGE_SIZE)
        self.Q_Buffer_Count_K = 0
        self.Q_Buffer_Count_V = 0
        self.Local_Buffer_V = win(self.PAGE_SIZE)
        self.Local_Count_V = 0
        self.Write_Offset_Local_V = 0
        self.key_states = None
        self.value_states = None

    # utils_kv_per_layer.py:85-95
    def get_total_length(self) -> int:
        k = self.PageCount_K * self.PAGE_SIZE + self.Sink_Count + self.Q_Buffer_Count_K
        v = (self.PageCount_V * self.PAGE_SIZE + self.Sink_Count + self.Q_Buffer_Count_V
             + self.Local_Count_V)
        assert k == v, f"seqlen_K: {k}, seqlen_V: {v}"
        return k

    # kitty.py:63-124
    def update(self, key_states: np.ndarray, value_states: np.ndarray) -> bool:
        if self.Sink_Count == 0:
            self.key_states = np.ascontiguousarray(key_states)
            self.value_states = np.ascontiguousarray(value_states)
            return True
        assert key_states.shape[-2] == 1 and value_states.shape[-2] == 1
        B = key_states.shape[0]
        if self.Sink_Count < self.S:
            i = self.Sink_Count
            self.Sink_Buffer_K[:B, :, i, :] = key_states[:, :, 0, :]
            self.Sink_Buffer_V[:B, :, i, :] = value_states[:, :, 0, :]
            self.Sink_Count += 1
        else:
            assert self.Q_Buffer_Count_K < self.PAGE_SIZE
            self.Q_Buffer_K[:B, :, self.Q_Buffer_Count_K, :] = key_states[:, :, 0, :]
            self.Q_Buffer_Count_K += 1
            assert self.Local_Count_V <= self.PAGE_SIZE
            if self.Local_Count_V < self.PAGE_SIZE:
                self.Local_Buffer_V[:B, :, self.Local_Count_V, :] = value_states[:, :, 0, :]
                self.Local_Count_V += 1
            else:
                assert self.Q_Buffer_Count_V < self.PAGE_SIZE
                w = self.Write_Offset_Local_V
                self.Q_Buffer_V[:B, :, self.Q_Buffer_Count_V, :] = self.Local_Buffer_V[:B, :, w, :]
                self.Q_Buffer_Count_V += 1
                self.Local_Buffer_V[:B, :, w, :] = value_states[:, :, 0, :]
                self.Write_Offset_Local_V = (w + 1) % self.PAGE_SIZE
        return False

    def append(self, key_states: np.ndarray, value_states: np.ndarray) -> None:
        """A chunk of T tokens, by definition T single-token steps of the reference's decode path
        (update, then quantize_decode: modeling_qwen3.py:225-251); an empty layer takes the
        reference's prefill path instead, as its update() would (kitty.py:91-95)."""
        if self.get_total_length() == 0:
            self.update(key_states, value_states)
            self.quantize_prefill()
            return
        for t in range(key_states.shape[-2]):
            self.update(key_states[:, :, t:t + 1], value_states[:, :, t:t + 1])
            self.quantize_decode()

    # kitty.py:126-192
    def quantize_prefill(self) -> None:
        if self.key_states is None or self.value_states is None:
            raise ValueError("No key_states or value_states to quantize. Please call update() first.")
        K, V = self.key_states, self.value_states
        B, T = K.shape[0], K.shape[-2]
        P = self.PAGE_SIZE
        ls = min(self.S, T)
        lq = max(0, T - ls) % P
        pk = (T - ls - lq) // P
        self.Sink_Buffer_K[:B, :, :ls, :] = K[:, :, :ls, :]
        self.Sink_Count = ls
        if lq > 0:
            self.Q_Buffer_K[:B, :, :lq, :] = K[:, :, T - lq:, :]
            self.Q_Buffer_Count_K = lq
        if pk > 0:
            quantize_pack_k(K, ls, pk, self.PageTable_K, 0, self.KeyCache, self.KeyCache_metadata,
                            P, self.D_BOOSTED)
            self.PageCount_K += pk
        ll = max(0, min(P, T - ls))
        lqv = max(0, T - ls - ll) % P
        pv = (T - ls - ll - lqv) // P
        self.Sink_Buffer_V[:B, :, :ls, :] = V[:, :, :ls, :]
        if ll > 0:
            self.Local_Buffer_V[:B, :, :ll, :] = V[:, :, T - ll:, :]
            self.Local_Count_V = ll
        if lqv > 0:
            self.Q_Buffer_V[:B, :, :lqv, :] = V[:, :, T - ll - lqv: T - ll, :]
            self.Q_Buffer_Count_V = lqv
        if pv > 0:
            quantize_pack_v(V, ls, pv, self.PageTable_V, 0, self.ValueCache, self.ValueCache_metadata, P)
            self.PageCount_V += pv
        self.key_states = None
        self.value_states = None

    # kitty.py:194-236
    def quantize_decode(self) -> None:
        P = self.PAGE_SIZE
        if self.Q_Buffer_Count_K == P:
            quantize_pack_k(self.Q_Buffer_K, 0, 1, self.PageTable_K, self.PageCount_K, self.KeyCache,
                            self.KeyCache_metadata, P, self.D_BOOSTED)
            self.PageCount_K += 1
            self.Q_Buffer_Count_K = 0
        if self.Q_Buffer_Count_V == P:
            quantize_pack_v(self.Q_Buffer_V, 0, 1, self.PageTable_V, self.PageCount_V, self.ValueCache,
                            self.ValueCache_metadata, P)
            self.PageCount_V += 1
            self.Q_Buffer_Count_V = 0


# ----------------------------------------------------------------------------------------------
# decode attention (kitty_attention.py:403-526; qk_kernel :16-207; softmax :473; sv_kernel :210-399)
# ----------------------------------------------------------------------------------------------
def gather_dense_kv(layer: OracleLayer, b: int, counts: Optional[dict] = None, dequant: str = "two"):
    """K̂ [H_KV, T, D] and V̂ [H_KV, T, D] of sequence ``b`` in chronological order (fp16, or
    float64 for ``dequant="affine"``):
    K = [sink | pages | Q-buffer], V = [sink | pages | Q-buffer | local ring in age order].
    ``counts`` overrides the layer-wide counters (ragged batches: per-sequence occupancy)."""
    c = dict(sink=layer.Sink_Count, pk=layer.PageCount_K, rk=layer.Q_Buffer_Count_K,
             pv=layer.PageCount_V, rv=layer.Q_Buffer_Count_V, lv=layer.Local_Count_V,
             off=layer.Write_Offset_Local_V)
    if counts:
        c.update(counts)
    lay, P = layer.lay, layer.PAGE_SIZE
    Ks, Vs = [], []
    for h in range(layer.H_KV):
        kparts = [layer.Sink_Buffer_K[b, h, : c["sink"]]]
        for p in range(c["pk"]):
            pg = int(layer.PageTable_K[b, p])
            o = h * lay.k_stride_h
            kparts.append(dequant_k_page(layer.KeyCache[pg, o: o + lay.k_stride_h],
                                         layer.KeyCache_metadata[pg, h], lay, dequant))
        kparts.append(layer.Q_Buffer_K[b, h, : c["rk"]])
        vparts = [layer.Sink_Buffer_V[b, h, : c["sink"]]]
        for p in range(c["pv"]):
            pg = int(layer.PageTable_V[b, p])
            o = h * lay.v_stride_h
            vparts.append(dequant_v_page(layer.ValueCache[pg, o: o + lay.v_stride_h],
                                         layer.ValueCache_metadata[pg, h], lay, dequant))
        vparts.append(layer.Q_Buffer_V[b, h, : c["rv"]])
        ring = (np.arange(c["lv"]) + c["off"]) % P
        vparts.append(layer.Local_Buffer_V[b, h, ring])
        dt = np.float64 if dequant == "affine" else F16
        Ks.append(np.concatenate([p_.astype(dt) for p_ in kparts], axis=0))
        Vs.append(np.concatenate([p_.astype(dt) for p_ in vparts], axis=0))
    return np.stack(Ks), np.stack(Vs)


def attend_dense(q: np.ndarray, K: np.ndarray, V: np.ndarray, scaling: float,
                 reference_rounding: bool = True) -> np.ndarray:
    """q fp16 [H_Q, D]; K, V fp16 [H_KV, T, D] -> out fp16 [H_Q, D].

    ``reference_rounding`` applies the reference's rounding points: logits = fp16(fp32 dot *
    scaling) (kitty_attention.py:100-102,167-169), probabilities = fp16(softmax in fp32) (:473),
    output = fp16(fp32 accumulation) (:389).  Without it everything stays float64 (the textbook
    value the reference approximates)."""
    H_Q, D = q.shape
    H_KV, T, _ = K.shape
    G = H_Q // H_KV
    out = np.zeros((H_Q, D), np.float64)
    for hq in range(H_Q):
        h = hq // G
        if reference_rounding:
            logits = (K[h].astype(F32) @ q[hq].astype(F32)).astype(F32)
            logits = (logits * F32(scaling)).astype(F16).astype(F32)
            m = logits.max() if T else F32(0)
            e = np.exp((logits - m).astype(F32)).astype(F32)
            p = (e / e.sum(dtype=F32)).astype(F16)
            out[hq] = (p.astype(F32)[None, :] @ V[h].astype(F32))[0]
        else:
            logits = K[h].astype(np.float64) @ q[hq].astype(np.float64) * float(scaling)
            e = np.exp(logits - logits.max())
            out[hq] = (e / e.sum()) @ V[h].astype(np.float64)
    return out.astype(F16) if reference_rounding else out


def rope_fp16(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """The caller-side rotation of the keys (modeling_qwen3.py:98-102, 125-128, applied at :215-220
    before ``update``): ``x * cos + rotate_half(x) * sin`` on fp16 tensors, i.e. both products and
    the sum rounded to fp16.  x fp16 [B, H, T, D]; cos / sin fp16 [B, T, D] (unsqueezed over the
    heads as the reference does).  numpy's float16 operators round each result once, like torch's.
    Pinned by torch's own fp16 operators on the same inputs (tests/test_oracle_attention.py)."""
    x = x.astype(F16)
    cos, sin = cos.astype(F16)[:, None], sin.astype(F16)[:, None]
    half = x.shape[-1] // 2
    rot = np.concatenate([-x[..., half:], x[..., :half]], axis=-1)
    return ((x * cos).astype(F16) + (rot * sin).astype(F16)).astype(F16)


def decode_attention(layer: OracleLayer, query: np.ndarray, scaling: float,
                     seq_counts: Optional[list] = None, reference_rounding: bool = True,
                     dequant: str = "two") -> np.ndarray:
    """query fp16 [B, H_Q, 1, D] -> [B, 1, H_Q, D] (fp16, or float64 without reference rounding).

    ``dequant`` picks how the packed pages are turned into numbers (``_dequant``);
    ``reference_rounding`` additionally applies the reference's fp16 roundings of logits,
    probabilities and output.  ``reference_rounding=False`` is plain dequantize-then-attend in
    float64.

    Uses the runtime ``Sink_Count`` for the probability offsets on the V side as well (the
    reference's sv_kernel uses the constant S there, kitty_attention.py:327,343,368, which only
    differs for prompts shorter than S tokens where it mis-indexes)."""
    B, H_Q, tq, D = query.shape
    assert tq == 1
    outs = []
    for b in range(B):
        K, V = gather_dense_kv(layer, b, None if seq_counts is None else seq_counts[b], dequant)
        assert K.shape[1] == V.shape[1]
        if reference_rounding:
            K, V = K.astype(F16), V.astype(F16)
        outs.append(attend_dense(query[b, :, 0, :], K, V, scaling, reference_rounding))
    return np.stack(outs)[:, None, :, :]


def prefill_attention(query: np.ndarray, K: np.ndarray, V: np.ndarray, scaling: float,
                      q_start: int) -> np.ndarray:
    """Causal chunk attention in float64.  query [H_Q, Tq, D] holds tokens q_start..q_start+Tq-1;
    K, V [H_KV, T, D] hold tokens 0..T-1 (T >= q_start+Tq).  Query i sees keys 0..q_start+i."""
    H_Q, Tq, D = query.shape
    H_KV, T, _ = K.shape
    G = H_Q // H_KV
    out = np.zeros((H_Q, Tq, D), np.float64)
    for hq in range(H_Q):
        h = hq // G
        s = query[hq].astype(np.float64) @ K[h].astype(np.float64).T * float(scaling)   # [Tq, T]
        mask = np.arange(T)[None, :] > (q_start + np.arange(Tq))[:, None]
        s = np.where(mask, -np.inf, s)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        out[hq] = (e / e.sum(axis=1, keepdims=True)) @ V[h].astype(np.float64)
    return out


def chunk_attention(layer: OracleLayer, query: np.ndarray, key_chunk: np.ndarray, value_chunk: np.ndarray,
                    scaling: float, seq_counts: Optional[list] = None, dequant: str = "two") -> np.ndarray:
    """Chunked-prefill attention over a cache (an extension; the reference attends one token at a
    time, kitty_attention.py:411).  query [B, H_Q, Tq, D]; key_chunk / value_chunk [B, H_KV, Tq, D]
    are the chunk's own fp16 keys / values, not yet appended.  Query i sees every cached token (in
    decode's order, dequantized as decode does) and chunk tokens 0..i.  Float64 throughout after the
    dequantization.  Returns [B, Tq, H_Q, D] float64.  Pinned by: reduction to `prefill_attention`
    (textbook causal attention) over `gather_dense_kv`, both pinned on their own; with Tq == 1 it
    equals decode attention after appending the token."""
    B, H_Q, Tq, D = query.shape
    out = np.zeros((B, Tq, H_Q, D), np.float64)
    for b in range(B):
        K, V = gather_dense_kv(layer, b, None if seq_counts is None else seq_counts[b], dequant)   # [H_KV, T0, D]
        T0 = K.shape[1]
        Kc = np.concatenate([K.astype(np.float64), key_chunk[b].astype(np.float64)], axis=1)
        Vc = np.concatenate([V.astype(np.float64), value_chunk[b].astype(np.float64)], axis=1)
        out[b] = prefill_attention(query[b], Kc, Vc, scaling, T0).transpose(1, 0, 2)
    return out
