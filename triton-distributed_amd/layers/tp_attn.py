"""One GPU's share of the reference's attention block at decode time.

``TP_Attn`` keeps the reference's constructor, parameter layout and forward signature
(``python/triton_dist/layers/amd/tp_attn.py:171-308``): fused QKV projection, optional per-head RMS norm of
q and k, rotary embedding, cache update, attention, output projection.  What changes is the middle: the
q/k norms, the rotary embedding of q and k and the cache update are ONE launch of the append kernel, and the attention is
the split-KV decode of this package instead of the flash-attn package (tp_attn.py:262-269).  The two
projections stay plain ``torch.nn.functional.linear`` calls (hipBLASLt), as in the reference's
``torch_fwd``.

Only the decode step (one new token per sequence) on one GPU is covered: ``world_size`` must be 1 -- the
all-gather / reduce-scatter GEMMs of ``dist_triton_fwd`` (tp_attn.py:278-306) and the prefill attention are
other paths -- and anything else raises.
"""
from __future__ import annotations

import torch
from torch import nn

from ..kernels.kv_append import flash_attn_with_kvcache


def layer_norm(hidden_states: torch.Tensor, eps: float, w: torch.Tensor):
    """Per-row RMS norm over the last dimension with weight ``w``: the reference's helper of this name
    (tp_attn.py:52-59), used on q and k when the model has q_norm / k_norm."""
    width = hidden_states.shape[-1]
    rows = hidden_states.reshape(-1, width)
    return nn.functional.rms_norm(rows, (width,), w, eps).reshape(hidden_states.shape)


def _set_cos_sin_cache(inv_freq: torch.Tensor, max_length: int):
    """fp32 ``[max_length, 2 * len(inv_freq)]``: cosines then sines of ``t * inv_freq`` (tp_attn.py:62-69, which
    hard-codes 64 = head_dim / 2 columns of each)."""
    t = torch.arange(max_length, device=inv_freq.device, dtype=inv_freq.dtype)
    freqs = torch.outer(t, inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1).to(torch.float32).contiguous()


class TP_Attn:
    """Attention block; QKV weights column-sharded over heads, output weights row-sharded (world_size 1 here)."""

    def __init__(self, rank=0, world_size=1, group=None):
        if world_size != 1:
            raise NotImplementedError("TP_Attn: this build runs one GPU's share only (world_size == 1)")
        self.rank = rank
        self.world_size = world_size
        self.group = group
        self.head_dim = 128
        self.wqkv = None
        self.wo = None

    def _init_parameters(self, self_attn: nn.Module, verbose=False):
        """Takes ``q_proj / k_proj / v_proj / o_proj`` (and ``q_norm / k_norm`` if present) of a HF attention module
        (tp_attn.py:186-209)."""
        self.init_from_weights(self_attn.q_proj.weight.detach(), self_attn.k_proj.weight.detach(),
                               self_attn.v_proj.weight.detach(), self_attn.o_proj.weight.detach())
        if hasattr(self_attn, "q_norm"):
            self.q_norm_eps = self_attn.q_norm.variance_epsilon
            self.q_norm_w = self_attn.q_norm.weight.detach().to("cuda", non_blocking=True)
        if hasattr(self_attn, "k_norm"):
            self.k_norm_eps = self_attn.k_norm.variance_epsilon
            self.k_norm_w = self_attn.k_norm.weight.detach().to("cuda", non_blocking=True)
        if verbose:
            print(f"[RANK {self.rank}] Attn initialized with parameters: qkv ({self.wqkv.shape}, o ({self.wo.shape}))")

    def init_from_weights(self, wq, wk, wv, wo, head_dim: int = 128):
        self.head_dim = head_dim
        self.q_size = wq.shape[0]
        self.kv_size = wk.shape[0]
        self.wqkv = torch.cat((wq, wk, wv), dim=0).to("cuda", non_blocking=True)   # [qkv_dim, hidden_size]
        self.wo = wo.to("cuda", non_blocking=True)
        self.K = self.wqkv.shape[1]
        self.dtype = self.wqkv.dtype

    def _init_ctx(self, *args, **kwargs):
        """The reference builds its all-gather / reduce-scatter GEMM contexts here (tp_attn.py:211-230); one GPU
        needs none."""

    @torch.inference_mode()
    def fwd(self, x: torch.Tensor, position_ids: torch.Tensor, cos_sin_cache: torch.Tensor, kv_cache, layer_idx: int,
            **decode_kw):
        """x ``[B, 1, hidden]`` -> ``[B, 1, hidden]``; appends the token's K/V to ``kv_cache`` at its offsets.
        The caller advances the offsets afterwards (``kv_cache.inc_offset()``), as the reference's engine does
        (models/engine.py:168)."""
        bsz, q_len, _ = x.size()
        if q_len != 1:
            raise NotImplementedError("TP_Attn.fwd: decode step only (one new token per sequence)")
        qkv = nn.functional.linear(x, self.wqkv)
        q, k, v = qkv.split([self.q_size, self.kv_size, self.kv_size], dim=-1)
        q = q.view(bsz, q_len, -1, self.head_dim)
        k = k.view(bsz, q_len, -1, self.head_dim)
        v = v.view(bsz, q_len, -1, self.head_dim)
        # the per-head RMS norms of q and k (tp_attn.py:252-258) run inside the append launch
        q_norm = (self.q_norm_w, self.q_norm_eps) if hasattr(self, "q_norm_eps") else None
        k_norm = (self.k_norm_w, self.k_norm_eps) if hasattr(self, "k_norm_eps") else None
        k_cache, v_cache, kv_offset = kv_cache.update_kv_cache(k, v, layer_idx)
        out = flash_attn_with_kvcache(q, k_cache, v_cache, k=k, v=v, cache_seqlens=kv_offset,
                                      block_table=kv_cache.block_table, causal=True, cos_sin_cache=cos_sin_cache,
                                      position_ids=position_ids, k_scale=kv_cache.k_scale, v_scale=kv_cache.v_scale,
                                      q_norm=q_norm, k_norm=k_norm, **decode_kw)
        return nn.functional.linear(out.view(bsz, q_len, -1), self.wo)

    torch_fwd = fwd
    dist_triton_fwd = fwd
