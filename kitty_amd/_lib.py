"""ctypes binding of libkitty_hip.so, the C-ABI library that holds every HIP kernel.

There is no fallback: if the library has not been built, or a tensor is not on a HIP device, the
callers raise.  Build it with ``python -m kitty_amd.build``.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_uint8, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libkitty_hip.so")
ABI_VERSION = 2
SEQ_COUNT_FIELDS = 8
STATUS_FIELDS = 4
# order of a status row (KITTY_STATUS_*, include/kitty_hip.h)
STATUS_NAMES = ("tokens_dropped", "flush_skipped", "bad_page_write", "bad_page_read")

# order of kitty_kv_layer.counts / seq_counts rows (include/kitty_hip.h)
CNT_SINK, CNT_PAGES_K, CNT_QBUF_K, CNT_PAGES_V, CNT_QBUF_V, CNT_LOCAL_V, CNT_LOCAL_OFF = range(7)


class KittyKVLayer(ctypes.Structure):
    """struct kitty_kv_layer (include/kitty_hip.h)."""
    _fields_ = [
        ("H_KV", c_int32), ("D", c_int32), ("D_BOOSTED", c_int32), ("PAGE_SIZE", c_int32),
        ("S", c_int32), ("MAX_PAGE", c_int32),
        ("counts", c_int32 * SEQ_COUNT_FIELDS),
        ("seq_counts", c_void_p),
        ("status", c_void_p),
        ("cache_pages_k", c_int64), ("cache_pages_v", c_int64),
        ("key_cache", c_void_p), ("key_cache_stride_page", c_int64),
        ("key_meta", c_void_p), ("key_meta_stride_page", c_int64),
        ("value_cache", c_void_p), ("value_cache_stride_page", c_int64),
        ("value_meta", c_void_p), ("value_meta_stride_page", c_int64),
        ("page_table_k", c_void_p), ("page_table_k_stride_b", c_int64),
        ("page_table_v", c_void_p), ("page_table_v_stride_b", c_int64),
        ("sink_k", c_void_p), ("sink_v", c_void_p),
        ("sink_stride_b", c_int64), ("sink_stride_h", c_int64),
        ("qbuf_k", c_void_p), ("qbuf_v", c_void_p), ("local_v", c_void_p),
        ("win_stride_b", c_int64), ("win_stride_h", c_int64),
    ]


_SIGNATURES = {
    "kitty_abi_version": (c_int, []),
    "kitty_last_error": (c_char_p, []),
    "kitty_select_boost_k": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_int, c_int,
                                     c_int, c_int, c_void_p, c_void_p]),
    "kitty_quant_pack_k": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_int, c_int,
                                   c_int, c_int, c_void_p, c_void_p, c_int64, c_int, c_void_p, c_int64, c_void_p,
                                   c_int64, c_int64, c_void_p, c_void_p]),
    "kitty_quant_pack_v": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_int, c_int,
                                   c_int, c_void_p, c_int64, c_int, c_void_p, c_int64, c_void_p, c_int64, c_int64,
                                   c_void_p, c_void_p]),
    "kitty_decode_attn_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "kitty_decode_attn_default_splits": (c_int, [c_int, c_int, c_int, c_int]),
    "kitty_decode_attn_split": (c_int, [POINTER(KittyKVLayer), c_void_p, c_int, c_int, c_float, c_void_p, c_size_t,
                                        c_int, c_int, c_void_p]),
    "kitty_decode_attn_merge": (c_int, [c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "kitty_profile_next_split": (c_int, [c_void_p, c_void_p]),
    "kitty_decode_attn": (c_int, [POINTER(KittyKVLayer), c_void_p, c_int, c_int, c_float, c_void_p, c_void_p,
                                  c_size_t, c_int, c_int, c_void_p]),
    "kitty_decode_attn_static": (c_int, [POINTER(KittyKVLayer), c_void_p, c_int, c_int, c_float, c_void_p, c_int, c_int,
                                         c_void_p]),
    "kitty_prefill_attn": (c_int, [POINTER(KittyKVLayer), c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                   c_int64, c_int64, c_int64, c_int, c_int, c_int, c_float, c_void_p, c_void_p]),
    "kitty_append_token": (c_int, [POINTER(KittyKVLayer), c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p,
                                   c_int64, c_int, c_void_p]),
    "kitty_flush_full": (c_int, [POINTER(KittyKVLayer), c_int, c_void_p]),
    "kitty_append_chunk": (c_int, [POINTER(KittyKVLayer), c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int,
                                   c_void_p]),
    "kitty_fake_quant": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_int, c_int,
                                 c_int, c_int, c_int, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p]),
}

EXPORTS = tuple(_SIGNATURES)
_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP kernels are not built (run `python -m kitty_amd.build`). "
                "There is no CPU or PyTorch fallback for this path.")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        if handle.kitty_abi_version() != ABI_VERSION:
            raise RuntimeError(f"libkitty_hip.so has ABI {handle.kitty_abi_version()}, expected {ABI_VERSION}")
        _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    """0 = ok; negative = argument rejected on the host (ValueError, as the reference's asserts and
    ValueErrors fire before launch); positive = hipError_t (RuntimeError)."""
    if rc == 0:
        return
    msg = lib().kitty_last_error().decode("utf-8", "replace")
    if rc < 0:
        raise ValueError(f"{what}: {msg} (code {rc})")
    raise RuntimeError(f"{what}: HIP error {rc}: {msg}")


def require_hip(t, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} lives on {t.device}; the Kitty kernels are HIP kernels for MI355X and there is no CPU path")


def current_stream_ptr(device) -> int:
    import torch
    return torch.cuda.current_stream(device).cuda_stream
