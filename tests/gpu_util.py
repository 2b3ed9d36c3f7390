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
