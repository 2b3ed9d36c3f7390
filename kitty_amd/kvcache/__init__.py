"""Kitty KV cache module (the exports of the reference's src/kitty/kvcache/__init__.py, plus the
paged variant)."""
from .kitty import KittyCache, get_kvcache_kitty
from .paging import OutOfPages, PagedKittyCache, PagePool

__all__ = ["KittyCache", "get_kvcache_kitty", "PagedKittyCache", "PagePool", "OutOfPages"]
