"""The reference's accuracy simulator on the GPU: a dense fp16 KV cache whose older tokens are
fake-quantized in place (quantize, dequantize, keep fp16), with configurable bit widths, promote
ratio and channel-selection strategy, for accuracy sweeps on the box that runs the packed path.

Mirrors src/kitty_sim (same names, argument meaning and results):

* ``fake_quant_groupwise_lastdim(data, group_size, bit, promote_mask=None, promote_bit=4)`` -
  utils_quant.py:64-114, here one HIP kernel (``kitty_fake_quant``) instead of a dozen torch
  operators with fp16 temporaries;
* ``build_promote_mask(key_states, promote_ratio, channel_selection)`` - utils_quant.py:12-61
  (0 random, 1 magnitude, 2 variance), the reference's torch operators on the device;
* ``KittyKVCacheConfig`` / ``KittyKVCache.update`` - kitty_simulate.py:22-121, 170-252.  The
  reference concatenates the new token to the whole cache and clones the whole cache on every step
  (PostQuant); here the layer's K / V live in buffers allocated once, ``update`` returns views, and
  under PostQuant the step's quantization is applied when the layer is touched next, so that the
  attention of the step sees the same fp16 values the reference's clone holds.

Head dimension 128, ``buffer_length`` 128 and ``group_size`` 32 / 64 / 128 only (the kernels'
tile).  The product path needs the HIP library; there is no torch fallback.
"""
from __future__ import annotations

from typing import Any, Optional

import torch

try:  # usable as past_key_values of a stock transformers model when transformers is importable
    from transformers.cache_utils import Cache as _HFCache
except Exception:  # pragma: no cover - transformers is optional for the kernels themselves
    _HFCache = object

from . import _lib

__all__ = ["build_promote_mask", "fake_quant_groupwise_lastdim", "fake_quant_tokens_", "KittyKVCacheConfig",
           "KittyKVCache"]


def build_promote_mask(key_states: torch.Tensor, promote_ratio: float, channel_selection: int) -> torch.Tensor:
    """key_states [..., D, T] -> bool [..., D]: the channels to promote (leading dims are batch
    dims; the reference passes [B, nh, D, T])."""
    assert key_states.dim() >= 3
    D = key_states.shape[-2]
    assert 0. <= promote_ratio <= 1.0, f"promote_ratio must be in [0, 1], got {promote_ratio}"
    k_chan = max(0, min(int(D * promote_ratio + 1e-6), D))
    lead = key_states.shape[:-1]
    if k_chan == 0:
        return torch.zeros(lead, dtype=torch.bool, device=key_states.device)
    if k_chan >= D:
        return torch.ones(lead, dtype=torch.bool, device=key_states.device)
    mask = torch.zeros(lead, dtype=torch.bool, device=key_states.device)
    if channel_selection == 0:
        if key_states.dim() != 4:
            raise ValueError("random selection draws one permutation per head of a [B, nh, D, T] tensor")
        for i in range(key_states.shape[1]):
            mask[:, i, torch.randperm(D, device=key_states.device)[:k_chan]] = True
        return mask
    if channel_selection == 1:
        score = key_states.abs().mean(dim=-1)
    elif channel_selection == 2:
        score = (key_states - key_states.mean(dim=-1, keepdim=True)).pow(2).mean(dim=-1)
    else:
        raise ValueError(f"Invalid channel_selection strategy: {channel_selection}")
    _, top_idx = score.topk(k_chan, dim=-1)
    mask.scatter_(-1, top_idx, True)
    return mask


def fake_quant_tokens_(x: torch.Tensor, t_offset: int, n_tokens: int, axis: int, group_size: int, bit: int,
                       promote_mask: Optional[torch.Tensor] = None, promote_bit: int = 4) -> torch.Tensor:
    """In place on tokens ``[t_offset, t_offset + n_tokens)`` of ``x`` fp16 [B, H, T, 128].
    axis 0: groups along the tokens (keys), ``promote_mask`` bool [B, H, D] or, one mask per
    128-token block, [B, H, n_tokens / 128, D]; axis 1: groups along the channels (values)."""
    _lib.require_hip(x, "x")
    if x.dtype != torch.float16 or x.dim() != 4 or x.stride(-1) != 1:
        raise ValueError("x must be float16 [B, H, T, D] with D contiguous")
    if bit >= 16:
        return x
    B, H, T, D = x.shape
    m_ptr, m_sb, m_sh, m_st = None, 0, 0, 0
    if promote_mask is not None:
        _lib.require_hip(promote_mask, "promote_mask")
        tiles = -(-n_tokens // 128)
        if promote_mask.dtype != torch.bool or tuple(promote_mask.shape) not in ((B, H, D), (B, H, tiles, D)):
            raise ValueError(f"promote_mask must be bool [B, H, D] or [B, H, {tiles}, D]")
        promote_mask = promote_mask.contiguous()
        m_ptr, m_sb, m_sh = promote_mask.data_ptr(), promote_mask.stride(0), promote_mask.stride(1)
        m_st = promote_mask.stride(2) if promote_mask.dim() == 4 else 0
    rc = _lib.lib().kitty_fake_quant(x.data_ptr(), x.stride(0) * 2, x.stride(1) * 2, x.stride(2) * 2, B, H, T, D,
                                     t_offset, n_tokens, axis, group_size, bit, m_ptr, m_sb, m_sh, m_st, promote_bit,
                                     _lib.current_stream_ptr(x.device))
    _lib.check(rc, "fake_quant")
    return x


def fake_quant_groupwise_lastdim(data: torch.Tensor, group_size: int, bit: int,
                                 promote_mask: Optional[torch.Tensor] = None, promote_bit: int = 4) -> torch.Tensor:
    """The reference's signature: ``data`` fp16 [B, nh, M, N], groups of ``group_size`` along the
    last dim, optional ``promote_mask`` [B, nh, M]; returns a new tensor of the same shape.  Two
    layouts are served: N == 128 contiguous (values, [B, nh, T, D]) and the transposed view of keys
    the reference builds (``k.transpose(2, 3)``: M == 128 channels, tokens last)."""
    assert data.dim() == 4, "Expected input shape [B, nh, D, T]"
    B, nh, M, N = data.shape
    assert N % group_size == 0, "T must be divisible by group_size"
    if bit >= 16:
        return data
    if M == 128 and (N != 128 or promote_mask is not None or data.stride(-2) == 1):
        # keys: [B, nh, D, T] -> token-major copy, groups along the tokens
        x = data.transpose(2, 3).contiguous()
        if x.data_ptr() == data.data_ptr():
            x = x.clone()
        fake_quant_tokens_(x, 0, N, 0, group_size, bit, promote_mask, promote_bit)
        return x.transpose(2, 3)
    if N != 128:
        raise ValueError("the kernels serve head_dim 128: [B, nh, T, 128] or [B, nh, 128, T]")
    if promote_mask is not None:
        raise ValueError("a promote mask goes with the transposed key layout [B, nh, 128, T]")
    x = data.contiguous()
    if x.data_ptr() == data.data_ptr():
        x = x.clone()
    return fake_quant_tokens_(x, 0, M, 1, group_size, bit)


class KittyKVCacheConfig:
    """Fields and defaults of the reference's configuration (kitty_simulate.py:22-48)."""

    def __init__(self, sink_length: int = 32, buffer_length: int = 128, group_size: int = 128, kbits: int = 2,
                 vbits: int = 2, promote_ratio: float = 0.1, promote_bit: int = 4, channel_selection: int = 1,
                 VCache_BitDecoding: bool = False, PostQuant: bool = True):
        self.sink_length, self.buffer_length, self.group_size = sink_length, buffer_length, group_size
        self.kbits, self.vbits = kbits, vbits
        self.promote_ratio, self.promote_bit, self.channel_selection = promote_ratio, promote_bit, channel_selection
        self.VCache_BitDecoding, self.PostQuant = VCache_BitDecoding, PostQuant
        self.validate()

    def validate(self):
        """The reference's checks (kitty_simulate.py:50-121) plus the kernels' tile constraints."""
        if self.channel_selection not in (0, 1, 2):
            raise ValueError(f"channel_selection must be 0, 1 or 2, got {self.channel_selection}")
        if self.buffer_length != 128 or self.group_size not in (32, 64, 128):
            raise ValueError("the kernels serve buffer_length 128 and group_size 32, 64 or 128")
        if self.sink_length < 0:
            raise ValueError(f"sink_length must be >= 0, got {self.sink_length}")
        for name in ("kbits", "vbits"):
            b = getattr(self, name)
            if b < 1 or b > 16 or 8 < b < 16:
                raise ValueError(f"{name} must be in [1, 8] or 16 (no quantization), got {b}")
        if not 0.0 <= self.promote_ratio <= 1.0:
            raise ValueError(f"promote_ratio must be in [0, 1], got {self.promote_ratio}")
        if self.promote_ratio > 0 and (self.promote_bit < self.kbits or self.promote_bit > 8):
            raise ValueError(f"promote_bit must be in [kbits, 8], got {self.promote_bit}")


class KittyKVCache(_HFCache):
    """The simulator's cache: ``update(key_states, value_states, layer_idx)`` appends and returns
    the keys and values the attention of this step sees ([B, nh, T, D] views of the layer's
    buffers, valid until the layer's next ``update``).  A ``transformers`` cache like the
    reference's (a ``DynamicCache`` subclass there): stock models with any dense attention
    implementation take it as ``past_key_values``."""
    is_compileable = False

    def __init__(self, cache_config: KittyKVCacheConfig, max_length: Optional[int] = None):
        """``KittyKVCache(cache_config)`` as in the reference (kitty_simulate.py:151).  ``max_length``
        (optional) sizes a layer's buffers once for good; without it they start at twice the prompt
        and double when full (the reference re-allocates on every step through ``torch.cat``)."""
        if _HFCache is not object:
            try:
                super().__init__(layers=[])          # transformers >= 4.54
            except TypeError:
                super().__init__()
        self.cfg = cache_config
        self.max_length = max_length
        self.key_cache: list[torch.Tensor] = []
        self.value_cache: list[torch.Tensor] = []
        self._len: list[int] = []
        self._pending: list[list] = []        # per layer: quantizations the last step left for later

    def get_seq_length(self, layer_idx: int = 0) -> int:
        return self._len[layer_idx] if layer_idx < len(self._len) else 0

    def get_mask_sizes(self, query_length, layer_idx: int = 0):
        """(kv_length, kv_offset) of the mask a stock model prepares for ``query_length`` new tokens."""
        n = query_length if isinstance(query_length, int) else int(query_length.shape[0])
        return self.get_seq_length(layer_idx) + n, 0

    # -- the three quantization steps of the reference, on [lo, hi) of a layer's buffers ----------
    def _quant_k(self, layer: int, lo: int, hi: int) -> None:
        c, K = self.cfg, self.key_cache[layer]
        # one mask per 128-token block, from the block as it is before quantization (:204-206, :236-237)
        blocks = K[:, :, lo:hi, :].unflatten(2, (-1, c.buffer_length)).transpose(-1, -2)    # [B, nh, blocks, D, 128]
        if c.channel_selection == 0:          # a fresh permutation per head and block, as the reference draws them
            mask = torch.stack([build_promote_mask(blocks[:, :, i], c.promote_ratio, 0)
                                for i in range(blocks.shape[2])], dim=2)
        else:
            mask = build_promote_mask(blocks, c.promote_ratio, c.channel_selection)
        fake_quant_tokens_(K, lo, hi - lo, 0, c.group_size, c.kbits, mask, c.promote_bit)

    def _quant_v(self, layer: int, lo: int, hi: int) -> None:
        if hi > lo:
            fake_quant_tokens_(self.value_cache[layer], lo, hi - lo, 1, self.cfg.group_size, self.cfg.vbits)

    def _run(self, layer: int, jobs: list) -> None:
        for kind, lo, hi in jobs:
            (self._quant_k if kind == "k" else self._quant_v)(layer, lo, hi)

    def flush_pending(self, layer_idx: Optional[int] = None) -> None:
        """Apply the quantizations PostQuant deferred (all layers by default)."""
        for l in ([layer_idx] if layer_idx is not None else range(len(self._pending))):
            self._run(l, self._pending[l])
            self._pending[l] = []

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[dict[str, Any]] = None):
        c = self.cfg
        if len(self.key_cache) < layer_idx:
            raise ValueError("QuantizedCache does not support model usage where layers are skipped. Use DynamicCache.")
        jobs = []
        if len(self.key_cache) == layer_idx:                                   # prefill
            B, nh, L, D = key_states.shape
            _lib.require_hip(key_states, "key_states")
            if key_states.dtype != torch.float16 or D != 128 or value_states.shape != key_states.shape:
                raise ValueError("key_states / value_states must be float16 [B, nh, T, 128]")
            assert L > c.sink_length, "Kitty-KV: sequence length must be greater than sink_length, currently."
            if self.max_length is not None and L > self.max_length:
                raise ValueError(f"prompt of {L} tokens exceeds max_length={self.max_length}")
            cap = self.max_length if self.max_length is not None else max(2 * L, L + 1024)
            for store, x in ((self.key_cache, key_states), (self.value_cache, value_states)):
                buf = torch.empty((B, nh, cap, D), dtype=torch.float16, device=key_states.device)
                buf[:, :, :L].copy_(x)
                store.append(buf)
            self._len.append(L)
            self._pending.append([])
            if L > c.sink_length + c.buffer_length:
                n = L - c.sink_length
                nq = n - n % c.buffer_length
                jobs.append(("k", c.sink_length, c.sink_length + nq))
                jobs.append(("v", c.sink_length, c.sink_length + (nq if c.VCache_BitDecoding else n - c.buffer_length)))
            self._run(layer_idx, jobs)
            if c.PostQuant:
                return key_states, value_states        # the prompt's attention sees the prompt as it came
            return self.key_cache[layer_idx][:, :, :L], self.value_cache[layer_idx][:, :, :L]
        # decode
        self.flush_pending(layer_idx)
        L = self._len[layer_idx]
        T_new = key_states.shape[-2]
        assert T_new == 1, "decode appends one token per step"
        if self.max_length is not None and L + 1 > self.max_length:
            raise ValueError(f"cache is full (max_length={self.max_length})")
        if L + 1 > self.key_cache[layer_idx].shape[2]:                         # no max_length given: double
            for store in (self.key_cache, self.value_cache):
                old = store[layer_idx]
                buf = torch.empty((old.shape[0], old.shape[1], 2 * old.shape[2], old.shape[3]), dtype=old.dtype,
                                  device=old.device)
                buf[:, :, :L].copy_(old[:, :, :L])
                store[layer_idx] = buf
        K, V = self.key_cache[layer_idx], self.value_cache[layer_idx]
        K[:, :, L:L + 1].copy_(key_states)
        V[:, :, L:L + 1].copy_(value_states)
        L += 1
        self._len[layer_idx] = L
        n = L - c.sink_length - c.buffer_length
        if n > 0 and n % c.buffer_length == 1:
            jobs.append(("k", L - c.buffer_length - 1, L - 1))
            if c.VCache_BitDecoding:
                jobs.append(("v", L - c.buffer_length - 1, L - 1))
        if not c.VCache_BitDecoding and n > 0:
            jobs.append(("v", L - c.buffer_length - 1, L - c.buffer_length))
        if c.PostQuant:
            self._pending[layer_idx] = jobs
        else:
            self._run(layer_idx, jobs)
        return K[:, :, :L], V[:, :, :L]
