"""KV caches for the decode block.

``PagedKV_Cache`` is the layout the decode path is built for (``[pages, P, Hkv, D]`` pools with an int32
block table, python/triton_dist/test/nvidia/test_decode_attn.py:150-156), optionally fp8-e4m3 with
per-KV-head scales; the reference has no paged owner class, so this one only adds what the kernels need:
the pools, a block table and the ``kv_offset`` bookkeeping.

``KV_Cache`` is the reference's dense cache (``python/triton_dist/models/kv_cache.py:28-69``:
``[layers, B, max_length, Hkv/world, D]`` plus an int32 ``kv_offset [B]``) expressed in that layout: one page of
``max_length`` tokens per sequence with the identity block table, so a layer's slice ``[B, max_length, Hkv, D]`` is
both what the reference's attention call takes as a dense cache and a valid pool for the paged kernels.  It keeps
the reference's constructor arguments, attribute names and methods so the decode block reads the same.
"""
from __future__ import annotations

from typing import Optional

import torch


class PagedKV_Cache:
    """Paged pools shared by all sequences of a layer: ``[layers, pages, P, Hkv, D]`` and one block table
    ``[B, max_length / P]`` whose rows are disjoint slices of a shuffled page list (``shuffle=False``: in
    order).  ``fp8=True`` stores e4m3fn bytes; ``k_scale`` / ``v_scale`` ``[layers, Hkv]`` fp32 then hold the
    dequantisation scales (default 1/16: representable magnitudes up to 28)."""

    def __init__(self, num_layers: int = 32, batch_size: int = 1, max_length: int = 32 * 1024, kv_heads: int = 8,
                 head_dim: int = 128, dtype=torch.bfloat16, world_size: int = 1, page_size: int = 16,
                 fp8: bool = False, shuffle: bool = True, seed: int = 0) -> None:
        assert max_length % page_size == 0
        self.num_layers, self.batch_size, self.max_length = num_layers, batch_size, max_length
        self.kv_heads, self.head_dim, self.world_size, self.page_size = kv_heads, head_dim, world_size, page_size
        self.fp8 = fp8
        self.dtype = torch.uint8 if fp8 else dtype
        pages_per_seq = max_length // page_size
        pages = batch_size * pages_per_seq
        shape = (num_layers, pages, page_size, kv_heads // world_size, head_dim)
        self.k_cache = torch.zeros(shape, device="cuda", dtype=self.dtype)
        self.v_cache = torch.zeros(shape, device="cuda", dtype=self.dtype)
        self.kv_offset = torch.zeros(batch_size, dtype=torch.int32, device="cuda")
        if shuffle:
            order = torch.randperm(pages, generator=torch.Generator().manual_seed(seed))
        else:
            order = torch.arange(pages)
        self.block_table = order.to(torch.int32).view(batch_size, pages_per_seq).cuda()
        self._k_scale = self._v_scale = None
        if fp8:
            self._k_scale = torch.full((num_layers, kv_heads // world_size), 1.0 / 16, device="cuda")
            self._v_scale = torch.full((num_layers, kv_heads // world_size), 1.0 / 16, device="cuda")
        self._layer = 0

    def update_kv_cache(self, new_k_cache: Optional[torch.Tensor], new_v_cache: Optional[torch.Tensor],
                        layer_idx: int):
        self._layer = layer_idx
        return self.k_cache[layer_idx], self.v_cache[layer_idx], self.kv_offset

    @property
    def k_scale(self):
        return self._k_scale[self._layer] if self.fp8 else None

    @property
    def v_scale(self):
        return self._v_scale[self._layer] if self.fp8 else None

    def set_scales(self, k_scale: torch.Tensor, v_scale: torch.Tensor):
        """``[layers, Hkv]`` fp32 dequantisation scales of an fp8 cache."""
        assert self.fp8 and k_scale.shape == self._k_scale.shape and v_scale.shape == self._v_scale.shape
        self._k_scale.copy_(k_scale)
        self._v_scale.copy_(v_scale)

    def inc_offset(self):
        self.kv_offset += 1

    def clear(self):
        self.kv_offset.zero_()

    def get_kv_len(self):
        return self.kv_offset


class KV_Cache(PagedKV_Cache):
    """Dense cache = ``PagedKV_Cache`` with ``page_size == max_length`` and pages in sequence order."""

    def __init__(self, num_layers: int = 32, batch_size: int = 1, max_length: int = 32 * 1024, kv_heads: int = 8,
                 head_dim: int = 128, dtype=torch.bfloat16, world_size: int = 8) -> None:
        super().__init__(num_layers=num_layers, batch_size=batch_size, max_length=max_length, kv_heads=kv_heads,
                         head_dim=head_dim, dtype=dtype, world_size=world_size, page_size=max_length, fp8=False,
                         shuffle=False)
        # the attention call derives the table of a dense cache itself ([b] -> page b)
        self.block_table = None

    def rand_fill_kv_cache(self, offset: int):
        """Uniform values in [0, 0.1) in the first ``offset`` positions of every layer and sequence (the range the
        reference's benchmark fill uses, models/kv_cache.py:52-57); ``kv_offset`` is left alone, as there."""
        for cache in (self.k_cache, self.v_cache):
            cache[:, :, :offset].uniform_(0.0, 0.1)
