"""Write side of the paged KV cache and the decode call that uses it.

``rope_kv_append`` is one launch that does what the reference's decode block does in three
steps right before attention (``python/triton_dist/layers/amd/tp_attn.py:262-265``): rotary
embedding of Q, rotary embedding of K, and the cache update -- here an append into the
paged pool ``[pages, P, Hkv, D]`` that the decode kernel reads, with fp8-e4m3 quantisation
when the cache is fp8.  ``apply_rotary_pos_emb`` has the reference's signature
(tp_attn.py:128-168).  ``flash_attn_with_kvcache`` is the call the reference's attention
block makes (tp_attn.py:268-269, the flash-attn package's function), for one query token
per sequence.

Every function enqueues hand-written HIP kernels through the C ABI in
``include/flash_decode.h``; there is no CPU path.
"""
from __future__ import annotations

from ctypes import byref
from typing import Optional, Tuple, Union

import torch

from .._lib import FdParams, FdQkPrep, check, fd_dtype_of, load_library, stream_handle
from .._lib import (FD_ORDER_ITEMS, FD_ORDER_SEQUENCES, FD_STEP_EXACT_SPLITS, FD_STEP_FUSED,
                    FD_STEP_ORDER_FROM_APPEND)
from .flash_decode import _decode, _require_cuda, decode_plan, item_order_buffer


def _ptr(t: Optional[torch.Tensor]):
    return t.data_ptr() if t is not None else None


def _prep_struct(cos_sin, position_ids, head_dim, bsz, seq) -> FdQkPrep:
    r = FdQkPrep()
    if cos_sin is None:
        return r
    assert cos_sin.dtype == torch.float32 and cos_sin.dim() == 2 and cos_sin.stride(1) == 1
    assert cos_sin.shape[1] == head_dim, "cos_sin rows hold head_dim/2 cosines then head_dim/2 sines"
    assert position_ids.dim() == 2 and tuple(position_ids.shape) == (bsz, seq)
    assert position_ids.dtype in (torch.int32, torch.int64)
    r.cos_sin = cos_sin.data_ptr()
    r.stride_cos_sin = cos_sin.stride(0)
    r.position_ids = position_ids.data_ptr()
    r.position_dtype = 1 if position_ids.dtype == torch.int64 else 0
    r.max_positions = cos_sin.shape[0]
    r.stride_pos_b, r.stride_pos_t = position_ids.stride(0), position_ids.stride(1)
    return r


def rope_kv_append(k_new: Optional[torch.Tensor], v_new: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                   v_cache: Optional[torch.Tensor], block_table: Optional[torch.Tensor],
                   kv_lens: Optional[torch.Tensor], *, kv_lens_out: Optional[torch.Tensor] = None,
                   seq_order_out: Optional[torch.Tensor] = None, item_order_out: Optional[torch.Tensor] = None,
                   item_plan: Optional[Tuple[int, int, int]] = None,
                   k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None,
                   cos_sin: Optional[torch.Tensor] = None, position_ids: Optional[torch.Tensor] = None,
                   q: Optional[torch.Tensor] = None, q_out: Optional[torch.Tensor] = None,
                   q_norm: Optional[Tuple[torch.Tensor, float]] = None,
                   k_norm: Optional[Tuple[torch.Tensor, float]] = None, stream=None):
    """Appends ``k_new`` / ``v_new`` ``[B, T, Hkv, D]`` at positions ``kv_lens[b] .. +T-1`` of the paged pool.

    With ``cos_sin`` (fp32 ``[max_pos, D]``) and ``position_ids`` (``[B, T]`` int32/int64) K is rotated before it
    is stored and ``q`` ``[B, T, Hq, D]`` (if given) is rotated into ``q_out`` (default: a new tensor; may be
    ``q``) in the same launch.  ``q_norm`` / ``k_norm`` = ``(weight [D], eps)`` apply the per-head RMS norm of the
    reference's block (tp_attn.py:252-258) to q / k before the rotation.  A uint8 / float8_e4m3fn cache with
    ``k_scale`` / ``v_scale`` ``[Hkv]`` stores ``clamp(x / scale, +-448)`` rounded to e4m3fn.  ``kv_lens_out``
    (int32 ``[B]``, not ``kv_lens``) receives the grown lengths; ``seq_order_out`` (int32 ``[2, B]``,
    ``B <= 4096``) the longest-first issue order for the decode that follows (row 0: what ``schedule_sequences``
    would compute, without a launch of its own) and the grown lengths in that order (row 1: the decode's
    ``seq_order_lens``).  ``item_order_out`` (``item_order_buffer(B, num_splits, device)``, ``B <= 256``) with
    ``item_plan = (num_splits, split_align, split_adapt)`` instead receives the work-item order of the decode that
    follows (what ``fd_schedule_items`` would compute for the grown lengths; pass it on as ``item_order=``).
    Returns ``q_out`` (or ``None`` without ``q``).
    """
    lib = load_library()
    append = k_new is not None
    src = k_new if append else q
    if src is None:
        raise RuntimeError("rope_kv_append: neither k_new nor q given")
    _require_cuda(k_new, v_new, k_cache, v_cache, block_table, kv_lens, kv_lens_out, seq_order_out, item_order_out,
                  cos_sin, position_ids, q, q_out)
    bsz, seq, _, head_dim = src.shape
    p = FdParams()
    p.head_dim = head_dim
    p.q_dtype = fd_dtype_of(src)
    p.q_heads = q.shape[2] if q is not None else 1
    p.kv_heads = k_new.shape[2] if append else 1
    skn = svn = (0, 0, 0)
    sk = sv = (0, 0)
    sbt = 0
    if append:
        assert v_new is not None and k_new.shape == v_new.shape and k_new.dtype == v_new.dtype
        assert k_new.stride(-1) == 1 and v_new.stride(-1) == 1 and k_cache.stride(-1) == 1 and v_cache.stride(-1) == 1
        assert k_cache.shape == v_cache.shape and k_cache.shape[2] == k_new.shape[2] and k_cache.shape[3] == head_dim
        page_size = k_cache.shape[1]
        assert k_cache.stride(0) == page_size * k_cache.stride(1) and v_cache.stride(0) == page_size * v_cache.stride(1)
        assert block_table.dtype == torch.int32 and kv_lens.dtype == torch.int32 and block_table.stride(1) == 1
        assert block_table.shape[0] == bsz and kv_lens.numel() == bsz and kv_lens.is_contiguous()
        if (k_scale is None) != (v_scale is None):
            raise RuntimeError("k_scale and v_scale must be given together")
        if kv_lens_out is not None:
            assert kv_lens_out.dtype == torch.int32 and kv_lens_out.is_contiguous() and kv_lens_out.numel() == bsz
        if seq_order_out is not None:
            assert item_order_out is None
            assert seq_order_out.dtype == torch.int32 and seq_order_out.is_contiguous()
            assert seq_order_out.numel() == 2 * bsz
        if item_order_out is not None:
            num_splits, split_align, split_adapt = item_plan
            assert item_order_out.dtype == torch.int32 and item_order_out.is_contiguous()
            assert item_order_out.numel() >= 2 * bsz * num_splits
            p.num_splits, p.split_align, p.split_adapt, p.seq_order_items = num_splits, split_align, split_adapt, 1
            seq_order_out = item_order_out
        p.page_size = page_size
        p.num_pages = k_cache.shape[0]
        p.max_pages_per_seq = block_table.shape[1]
        p.kv_dtype = fd_dtype_of(k_cache, fp8_bytes=k_scale is not None)
        p.k_scale, p.v_scale = _ptr(k_scale), _ptr(v_scale)
        skn, svn = k_new.stride()[:3], v_new.stride()[:3]
        sk, sv = (k_cache.stride(1), k_cache.stride(2)), (v_cache.stride(1), v_cache.stride(2))
        sbt = block_table.stride(0)
    prep = None
    if cos_sin is not None or q_norm is not None or k_norm is not None:
        prep = _prep_struct(cos_sin, position_ids, head_dim, bsz, seq)
        for name, norm in (("q", q_norm), ("k", k_norm)):
            if norm is not None:
                w, eps = norm
                _require_cuda(w)
                assert w.dtype == src.dtype and w.is_contiguous() and w.numel() == head_dim
                setattr(prep, name + "_norm_weight", w.data_ptr())
                setattr(prep, name + "_norm_eps", float(eps))
        if q is not None:
            assert q.dim() == 4 and q.shape[0] == bsz and q.shape[1] == seq and q.shape[3] == head_dim
            assert q.dtype == src.dtype and q.stride(-1) == 1
            if q_out is None:
                q_out = torch.empty_like(q)
            assert q_out.shape == q.shape and q_out.dtype == q.dtype and q_out.stride(-1) == 1
            prep.q, prep.q_out = q.data_ptr(), q_out.data_ptr()
            prep.stride_q_b, prep.stride_q_t, prep.stride_q_h = q.stride()[:3]
            prep.stride_qo_b, prep.stride_qo_t, prep.stride_qo_h = q_out.stride()[:3]
    elif q is not None:
        raise RuntimeError("rope_kv_append: q is only processed together with cos_sin / position_ids or a norm")
    check(lib.fd_kv_append(
        stream_handle(stream, src.device.index), _ptr(k_new), _ptr(v_new), _ptr(k_cache), _ptr(v_cache),
        _ptr(block_table), _ptr(kv_lens), _ptr(kv_lens_out), _ptr(seq_order_out), bsz, seq, *skn, *svn, *sk, *sv, sbt,
        byref(prep) if prep is not None else None, byref(p)))
    return q_out if q is not None else None


def paged_kv_append(k_new, v_new, k_cache, v_cache, block_table, kv_lens, *, kv_lens_out=None, seq_order_out=None,
                    k_scale=None, v_scale=None, stream=None):
    """``rope_kv_append`` without the rotation: the plain cache update (models/kv_cache.py:43-50 for a paged pool)."""
    rope_kv_append(k_new, v_new, k_cache, v_cache, block_table, kv_lens, kv_lens_out=kv_lens_out,
                   seq_order_out=seq_order_out, k_scale=k_scale, v_scale=v_scale, stream=stream)


def apply_rotary_pos_emb(x: torch.Tensor, cos_sin: torch.Tensor, position_ids: torch.Tensor) -> torch.Tensor:
    """Rotary embedding of ``x [bsz, seq, heads, head_dim]`` -> new tensor (tp_attn.py:128-168)."""
    assert x.dim() == 4, "Input tensor x must be 4-dimensional"
    assert position_ids.dim() == 2, "position_ids must be 2-dimensional"
    x = x.contiguous()
    return rope_kv_append(None, None, None, None, None, None, cos_sin=cos_sin.contiguous(),
                          position_ids=position_ids, q=x)


_ARANGE = {}


def _dense_block_table(device, n):
    key = (device.index, n)
    t = _ARANGE.get(key)
    if t is None:
        t = torch.arange(n, dtype=torch.int32, device=device).view(n, 1)
        _ARANGE[key] = t
    return t


def flash_attn_with_kvcache(q, k_cache, v_cache, k=None, v=None, rotary_cos=None, rotary_sin=None,
                            cache_seqlens: Union[int, torch.Tensor, None] = None, cache_batch_idx=None,
                            cache_leftpad=None, block_table=None, softmax_scale=None, causal=False,
                            window_size=(-1, -1), softcap=0.0, rotary_interleaved=True, alibi_slopes=None,
                            num_splits=0, return_softmax_lse=False, *, cos_sin_cache=None, position_ids=None,
                            k_scale=None, v_scale=None, kv_lens_out=None, q_norm=None, k_norm=None, stream=None,
                            **decode_kw):
    """Decode-step drop-in for the flash-attn call of the reference's attention block (tp_attn.py:268-269).

    ``q [B, 1, Hq, D]``; ``k_cache`` / ``v_cache`` either dense ``[B_cache, L, Hkv, D]`` (the reference's
    ``KV_Cache`` slice, models/kv_cache.py:36-44) or paged ``[pages, P, Hkv, D]`` with ``block_table``;
    ``k`` / ``v [B, T, Hkv, D]`` are appended in place at ``cache_seqlens`` first and attention then covers
    ``cache_seqlens + T`` tokens (with one query token ``causal`` changes nothing).  ``cache_seqlens`` itself
    is not modified, as in flash-attn.  Returns ``out [B, 1, Hq, D]`` (and the natural-log LSE
    ``[B, Hq, 1]`` fp32 with ``return_softmax_lse``).

    Beyond flash-attn: ``cos_sin_cache`` + ``position_ids`` (the reference's rotary format) rotate q and k
    on the way in, in the append launch, after the per-head RMS norms ``q_norm`` / ``k_norm`` =
    ``(weight, eps)``; ``k_scale`` / ``v_scale`` select an fp8-e4m3 cache;
    ``kv_lens_out`` receives ``cache_seqlens + T``.  ``num_splits`` 0 lets the library choose.
    Not covered, and refused: more than one query token, flash-attn's own rotary arguments, left padding,
    sliding windows and ALiBi.
    """
    if q.dim() != 4 or q.shape[1] != 1:
        raise NotImplementedError("flash_attn_with_kvcache: this library covers the decode step (seqlen_q == 1)")
    if rotary_cos is not None or rotary_sin is not None:
        raise NotImplementedError("flash_attn_with_kvcache: pass cos_sin_cache= / position_ids= for rotary")
    if cache_leftpad is not None or alibi_slopes is not None or tuple(window_size) != (-1, -1):
        raise NotImplementedError("flash_attn_with_kvcache: cache_leftpad, alibi_slopes and window_size")
    if cache_seqlens is None:
        raise RuntimeError("flash_attn_with_kvcache: cache_seqlens is required")
    bsz, _, q_heads, head_dim = q.shape
    dev = q.device
    if isinstance(cache_seqlens, int):
        cache_seqlens = torch.full((bsz,), cache_seqlens, dtype=torch.int32, device=dev)
    assert cache_seqlens.dtype == torch.int32 and cache_seqlens.numel() == bsz
    if block_table is None:
        if cache_batch_idx is not None:
            block_table = cache_batch_idx.to(torch.int32).view(bsz, 1)
        else:
            assert k_cache.shape[0] >= bsz
            block_table = _dense_block_table(dev, bsz)
    elif cache_batch_idx is not None:
        raise RuntimeError("flash_attn_with_kvcache: cache_batch_idx is not used with a paged cache")
    scale = head_dim ** -0.5 if softmax_scale is None else softmax_scale

    kv_lens = cache_seqlens
    q_rot = q
    if k is not None:
        assert v is not None
        if kv_lens_out is None:
            kv_lens_out = torch.empty_like(cache_seqlens)
        order = items = item_plan = None
        if "seq_order" not in decode_kw and "item_order" not in decode_kw and decode_kw.get("auto_order", True):
            # the append launch can also compute the decode's issue order, at no launch of its own: the library's
            # plan says whether that pays for this batch and which kind -- (sequence, range) items, largest first, or
            # sequences, longest first
            plan = decode_plan(q[:, 0], k_cache, block_table, num_splits if num_splits > 0 else -1,
                               flags=FD_STEP_ORDER_FROM_APPEND
                               | (0 if decode_kw.get("plan_splits", True) else FD_STEP_EXACT_SPLITS)
                               | (FD_STEP_FUSED if decode_kw.get("fuse_combine") else 0),
                               out_dtype=fd_dtype_of(q), fp8=k_scale is not None, path=decode_kw.get("path", "auto"),
                               waves_per_block=decode_kw.get("waves_per_block", 0),
                               max_kv_len=decode_kw.get("max_kv_len"), v_head_dim=v_cache.shape[-1])
            if plan.order_kind == FD_ORDER_ITEMS:
                items = item_order_buffer(bsz, plan.num_splits, dev)
                item_plan = (plan.num_splits, plan.split_align, plan.split_adapt)
                decode_kw["item_order"] = items
            elif plan.order_kind == FD_ORDER_SEQUENCES:
                order = torch.empty((2, bsz), dtype=torch.int32, device=dev)
                decode_kw["seq_order"], decode_kw["seq_order_lens"] = order[0], order[1]
        prep_q = cos_sin_cache is not None or q_norm is not None
        q_rot = rope_kv_append(k, v, k_cache, v_cache, block_table, cache_seqlens, kv_lens_out=kv_lens_out,
                               seq_order_out=order, item_order_out=items, item_plan=item_plan,
                               k_scale=k_scale, v_scale=v_scale,
                               cos_sin=cos_sin_cache, position_ids=position_ids, q=q if prep_q else None,
                               q_norm=q_norm, k_norm=k_norm, stream=stream)
        if q_rot is None:
            q_rot = q
        kv_lens = kv_lens_out
    elif cos_sin_cache is not None or q_norm is not None:
        q_rot = rope_kv_append(None, None, None, None, None, None, cos_sin=cos_sin_cache, position_ids=position_ids,
                               q=q, q_norm=q_norm, stream=stream)

    out = torch.empty_like(q)
    lse = torch.empty((bsz, q_heads), dtype=torch.float32, device=dev) if return_softmax_lse else None
    _decode(q_rot.view(bsz, q_heads, head_dim) if q_rot.is_contiguous() else q_rot[:, 0], k_cache, v_cache, None,
            kv_lens, block_table, scale, softcap, None, out.view(bsz, q_heads, head_dim),
            num_splits if num_splits > 0 else -1, with_lse_column=False, lse_out=lse, k_scale=k_scale, v_scale=v_scale,
            stream=stream, **decode_kw)
    if return_softmax_lse:
        return out, lse.view(bsz, q_heads, 1)
    return out
