"""Helpers for the GPU parity tests: build the same cache state in the HIP-backed KittyCache and
in the CPU oracle from the same seeded inputs."""
import types

import numpy as np
import torch

from oracle import kitty_oracle as O


def cfg(H_KV, H_Q, layers=1, D=128):
    return types.SimpleNamespace(num_hidden_layers=layers, head_dim=D, num_key_value_heads=H_KV,
                                 num_attention_heads=H_Q, hidden_size=H_Q * D)


def module(H_KV, H_Q):
    return types.SimpleNamespace(num_attention_heads=H_Q, num_key_value_heads=H_KV)


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def layer_bytes_equal(layer, ol: O.OracleLayer, live_q_rows_only: bool = False):
    """Bit-exact comparison of every tensor of a layer with the oracle's; returns list of mismatches.
    ``live_q_rows_only``: compare the Q-buffers up to their fill counts only (rows past the count are
    stale, and a chunked append legitimately leaves other stale rows than single steps do)."""
    bad = []

    def cmp(name, t, a):
        got = t.detach().cpu().numpy()
        if got.dtype == np.float16:
            got, a = got.view(np.uint16), a.view(np.uint16)
        if not np.array_equal(got, a):
            bad.append((name, int((got != a).sum())))

    cmp("KeyCache", layer.KeyCache, ol.KeyCache)
    cmp("KeyCache_metadata", layer.KeyCache_metadata, ol.KeyCache_metadata)
    cmp("ValueCache", layer.ValueCache, ol.ValueCache)
    cmp("ValueCache_metadata", layer.ValueCache_metadata, ol.ValueCache_metadata)
    cmp("Sink_Buffer_K", layer.Sink_Buffer_K, ol.Sink_Buffer_K)
    cmp("Sink_Buffer_V", layer.Sink_Buffer_V, ol.Sink_Buffer_V)
    nk = ol.Q_Buffer_Count_K if live_q_rows_only else ol.PAGE_SIZE
    nv = ol.Q_Buffer_Count_V if live_q_rows_only else ol.PAGE_SIZE
    cmp("Q_Buffer_K", layer.Q_Buffer_K[:, :, :nk], ol.Q_Buffer_K[:, :, :nk])
    cmp("Q_Buffer_V", layer.Q_Buffer_V[:, :, :nv], ol.Q_Buffer_V[:, :, :nv])
    cmp("Local_Buffer_V", layer.Local_Buffer_V, ol.Local_Buffer_V)
    for f in ("Sink_Count", "PageCount_K", "PageCount_V", "Q_Buffer_Count_K", "Q_Buffer_Count_V",
              "Local_Count_V", "Write_Offset_Local_V"):
        if getattr(layer, f) != getattr(ol, f):
            bad.append((f, getattr(layer, f), getattr(ol, f)))
    return bad


def oracle_from_layer(layer, max_len) -> O.OracleLayer:
    """An OracleLayer holding a copy of a device layer's bytes and counters (to check attention at
    sizes where quantizing again on the CPU would take minutes; the quantizer is checked elsewhere)."""
    ol = O.OracleLayer(layer.MAX_BS, max_len, layer.H_KV)
    for name in ("KeyCache", "KeyCache_metadata", "ValueCache", "ValueCache_metadata", "PageTable_K",
                 "PageTable_V", "Sink_Buffer_K", "Sink_Buffer_V", "Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V"):
        a = getattr(layer, name).detach().cpu().numpy()
        assert a.shape == getattr(ol, name).shape, name
        setattr(ol, name, a)
    for f in ("Sink_Count", "PageCount_K", "PageCount_V", "Q_Buffer_Count_K", "Q_Buffer_Count_V",
              "Local_Count_V", "Write_Offset_Local_V"):
        setattr(ol, f, getattr(layer, f))
    return ol


def oracle_head_view(layer, b: int, h: int, max_len: int, counts=None) -> O.OracleLayer:
    """OracleLayer (batch 1, one KV head) holding a copy of row ``b``, head ``h`` of a device layer
    whose page table is the identity; ``counts`` = (sink, pk, rk, pv, rv, lv, off) overrides the
    layer's counters (per-sequence occupancy)."""
    ol = O.OracleLayer(1, max_len, 1)
    lay = O.Layout(H_KV=layer.H_KV)
    mp = layer.MAX_PAGE
    assert ol.MAX_PAGE == mp
    rows = slice(b * mp, (b + 1) * mp)
    ol.KeyCache = layer.KeyCache[rows, h * lay.k_stride_h:(h + 1) * lay.k_stride_h].cpu().numpy().copy()
    ol.ValueCache = layer.ValueCache[rows, h * lay.v_stride_h:(h + 1) * lay.v_stride_h].cpu().numpy().copy()
    ol.KeyCache_metadata = layer.KeyCache_metadata[rows, h:h + 1].cpu().numpy().copy()
    ol.ValueCache_metadata = layer.ValueCache_metadata[rows, h:h + 1].cpu().numpy().copy()
    for name in ("Sink_Buffer_K", "Sink_Buffer_V", "Q_Buffer_K", "Q_Buffer_V", "Local_Buffer_V"):
        setattr(ol, name, getattr(layer, name)[b:b + 1, h:h + 1].cpu().numpy().copy())
    fields = ("Sink_Count", "PageCount_K", "Q_Buffer_Count_K", "PageCount_V", "Q_Buffer_Count_V", "Local_Count_V",
              "Write_Offset_Local_V")
    vals = counts if counts is not None else [getattr(layer, f) for f in fields]
    for f, v in zip(fields, vals):
        setattr(ol, f, int(v))
    return ol
