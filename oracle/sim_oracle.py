"""CPU oracle of the reference's accuracy simulator (fake quantization of a dense fp16 KV cache).
TEST INFRASTRUCTURE ONLY: nothing in ``kitty_amd`` imports it.

numpy restatement, one function per reference function:

* ``fake_quant_groupwise_lastdim``  - src/kitty_sim/utils_quant.py:64-114
* ``build_promote_mask``            - src/kitty_sim/utils_quant.py:12-61 (strategies 1 and 2; the
                                       random strategy 0 has no arithmetic to restate)
* ``SimCache.update``               - src/kitty_sim/kitty_simulate.py:170-252

The reference runs these on fp16 tensors, where every torch operator computes in fp32 and rounds its
result to fp16; ``_h`` is that rounding and appears once per operator of the reference's chain.  One
operator differs between devices: a tensor divided by a Python scalar (``/ (2 ** bit - 1)``, :96-97,
:106) is a true division on the CPU and a multiplication by the scalar's fp32 reciprocal on a GPU
(torch's kernels for a host-scalar divisor); ``scalar_div`` selects which, default the GPU's.

Pinned by tests/test_sim_oracle.py: against torch's own fp16 operators evaluating the reference's
chain on the CPU (``scalar_div="true"``), against a scalar loop in numpy float16 arithmetic, and by
closed forms (levels reproduce, constant groups, clamp before round, half to even).  The reference
holds no fixtures for these functions, and ``torch.topk``'s order among equal scores is not pinned
by anything (tests use data without ties at the selection boundary).
"""
from typing import Optional

import numpy as np


def _h(a):
    """Round to fp16 and continue in fp32: the store of one torch operator on an fp16 tensor."""
    return np.asarray(a, dtype=np.float32).astype(np.float16).astype(np.float32)


def fake_quant_groupwise_lastdim(data: np.ndarray, group_size: int, bit: int, promote_mask: Optional[np.ndarray] = None,
                                 promote_bit: int = 4, scalar_div: str = "reciprocal") -> np.ndarray:
    """data fp16 [B, nh, D, T], groups of ``group_size`` along the last dim; promote_mask bool [B, nh, D]."""
    assert data.ndim == 4 and data.dtype == np.float16
    B, nh, D, T = data.shape
    assert T % group_size == 0, "T must be divisible by group_size"
    if bit >= 16:
        return data
    x = data.astype(np.float32).reshape(B, nh, D, T // group_size, group_size)
    mn = x.min(axis=-1, keepdims=True)                                   # :90
    mx = x.max(axis=-1, keepdims=True)                                   # :91
    rng = _h(np.maximum(_h(mx - mn), np.float32(1e-4)))                  # (mx - mn).clamp(min=eps), eps = 1e-4 for fp16 (:92)

    def over(levels):
        if scalar_div == "reciprocal":
            return _h(rng * (np.float32(1.0) / np.float32(levels)))
        assert scalar_div == "true"
        return _h(rng / np.float32(levels))

    scale = over(2 ** bit - 1)                                           # :106
    max_val = np.full_like(scale, 2 ** bit - 1)
    if promote_mask is not None:
        assert promote_mask.shape == (B, nh, D)
        pm = promote_mask.reshape(B, nh, D, 1, 1).astype(bool)
        scale = np.where(pm, over(2 ** promote_bit - 1), scale)          # :96-99
        max_val = np.where(pm, np.float32(2 ** promote_bit - 1), max_val)    # :100-104
    q = _h(_h(x - mn) / scale)                                           # :112, two operators
    q = np.rint(np.clip(q, 0.0, max_val))                                # clamp, then round half to even
    dq = _h(_h(q * scale) + mn)                                          # :113, two operators
    return dq.reshape(B, nh, D, T).astype(np.float16)


def promote_scores(key_states: np.ndarray, channel_selection: int) -> np.ndarray:
    """The score ``build_promote_mask`` ranks channels by; key_states fp16 [B, nh, D, T]."""
    x = key_states.astype(np.float32)
    T = x.shape[-1]
    if channel_selection == 1:                                           # magnitude (:43-45)
        return _h(np.abs(x).sum(axis=-1, dtype=np.float32) / np.float32(T))
    if channel_selection == 2:                                           # variance (:48-50)
        mean = _h(x.sum(axis=-1, keepdims=True, dtype=np.float32) / np.float32(T))
        diff = _h(x - mean)
        return _h(_h(diff * diff).sum(axis=-1, dtype=np.float32) / np.float32(T))
    raise ValueError(f"Invalid channel_selection strategy: {channel_selection}")


def promote_count(D: int, promote_ratio: float) -> int:
    return max(0, min(int(D * promote_ratio + 1e-6), D))                 # :34-35


def build_promote_mask(key_states: np.ndarray, promote_ratio: float, channel_selection: int) -> np.ndarray:
    B, nh, D, _ = key_states.shape
    assert 0.0 <= promote_ratio <= 1.0
    k = promote_count(D, promote_ratio)
    if k == 0:
        return np.zeros((B, nh, D), dtype=bool)
    if k >= D:
        return np.ones((B, nh, D), dtype=bool)
    score = promote_scores(key_states, channel_selection)
    order = np.argsort(-score, axis=-1, kind="stable")                   # ties: lower channel first (not pinned)
    mask = np.zeros((B, nh, D), dtype=bool)
    np.put_along_axis(mask, order[..., :k], True, axis=-1)
    return mask


def selection_is_tie_free(key_states: np.ndarray, promote_ratio: float, channel_selection: int) -> bool:
    k = promote_count(key_states.shape[2], promote_ratio)
    if k == 0 or k >= key_states.shape[2]:
        return True
    s = -np.sort(-promote_scores(key_states, channel_selection), axis=-1)
    return bool((s[..., k - 1] > s[..., k]).all())


class SimCache:
    """One layer of the simulator's cache (kitty_simulate.py:170-252): dense fp16 K / V
    [B, nh, T, D] that are fake-quantized in place as tokens age; ``update`` returns what the
    attention of that step sees."""

    def __init__(self, sink_length=32, buffer_length=128, group_size=128, kbits=2, vbits=2, promote_ratio=0.1,
                 promote_bit=4, channel_selection=1, VCache_BitDecoding=False, PostQuant=True,
                 scalar_div="reciprocal", mask_fn=None):
        self.sink, self.buf, self.group = sink_length, buffer_length, group_size
        self.kbits, self.vbits, self.ratio, self.pbit = kbits, vbits, promote_ratio, promote_bit
        self.sel, self.bitdec, self.post = channel_selection, VCache_BitDecoding, PostQuant
        self.div = scalar_div
        self.mask_fn = mask_fn or (lambda ks: build_promote_mask(ks, self.ratio, self.sel))
        self.K = self.V = None

    def _quant_k(self, lo, hi):
        ks = np.ascontiguousarray(self.K[:, :, lo:hi, :].transpose(0, 1, 3, 2))
        out = fake_quant_groupwise_lastdim(ks, self.group, self.kbits, self.mask_fn(ks), self.pbit, self.div)
        self.K[:, :, lo:hi, :] = out.transpose(0, 1, 3, 2)

    def _quant_v(self, lo, hi):
        if hi > lo:
            self.V[:, :, lo:hi, :] = fake_quant_groupwise_lastdim(self.V[:, :, lo:hi, :], self.group, self.vbits,
                                                                  scalar_div=self.div)

    def update(self, key_states: np.ndarray, value_states: np.ndarray):
        if self.K is None:                                               # prefill (:183-215)
            self.K, self.V = key_states.copy(), value_states.copy()
            L = self.K.shape[-2]
            k_ret, v_ret = self.K.copy(), self.V.copy()
            assert L > self.sink
            if L > self.sink + self.buf:
                n = L - self.sink
                nq = n - n % self.buf
                for i in range(self.sink, self.sink + nq, self.buf):
                    self._quant_k(i, i + self.buf)
                self._quant_v(self.sink, self.sink + (nq if self.bitdec else n - self.buf))
        else:                                                            # decode (:217-247)
            self.K = np.concatenate([self.K, key_states], axis=-2)
            self.V = np.concatenate([self.V, value_states], axis=-2)
            L = self.K.shape[-2]
            k_ret, v_ret = self.K.copy(), self.V.copy()
            n = L - self.sink - self.buf
            if n > 0 and n % self.buf == 1:
                self._quant_k(L - self.buf - 1, L - 1)
                if self.bitdec:
                    self._quant_v(L - self.buf - 1, L - 1)
            if not self.bitdec and n > 0:
                self._quant_v(L - self.buf - 1, L - self.buf)
        if self.post:
            return k_ret, v_ret
        return self.K, self.V
