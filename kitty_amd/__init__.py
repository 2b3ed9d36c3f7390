"""MI355X-native implementation of Kitty's quantized-KV hot path (2-bit KV cache with Dynamic
Channel-wise Precision Boost): hand-written gfx950 kernels behind a C ABI, with the reference's
Python cache-plugin API on top."""
from .kvcache import KittyCache, OutOfPages, PagedKittyCache, PagePool, get_kvcache_kitty  # noqa: F401

__all__ = ["KittyCache", "get_kvcache_kitty", "PagedKittyCache", "PagePool", "OutOfPages"]
