"""Kitty KV cache module (same exports as the reference's src/kitty/kvcache/__init__.py)."""
from .kitty import KittyCache, get_kvcache_kitty

__all__ = ["KittyCache", "get_kvcache_kitty"]
