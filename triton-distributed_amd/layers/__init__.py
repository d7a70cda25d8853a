"""Layers on the flash-decode path (``python/triton_dist/layers/nvidia/__init__.py:25``)."""
from .sp_flash_decode_layer import SpGQAFlashDecodeAttention  # noqa: F401

__all__ = ["SpGQAFlashDecodeAttention"]
