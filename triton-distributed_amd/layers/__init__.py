"""Layers on the flash-decode path (``python/triton_dist/layers/nvidia/__init__.py:25``) and the decode
block that calls it (``python/triton_dist/layers/amd/tp_attn.py``, ``python/triton_dist/models/kv_cache.py``)."""
from .kv_cache import KV_Cache, PagedKV_Cache  # noqa: F401
from .sp_flash_decode_layer import SpGQAFlashDecodeAttention  # noqa: F401
from .tp_attn import TP_Attn, _set_cos_sin_cache, layer_norm  # noqa: F401

__all__ = ["SpGQAFlashDecodeAttention", "TP_Attn", "KV_Cache", "PagedKV_Cache"]
