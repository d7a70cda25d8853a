"""Host wrappers of the gfx950 flash-decode kernels.

Same names, argument order and return values as the reference's
``python/triton_dist/kernels/nvidia/flash_decode.py`` wrappers
(``gqa_fwd_batch_decode`` :763-844, ``gqa_fwd_batch_decode_intra_rank`` :847-928,
``gqa_fwd_batch_decode_persistent`` :931-1005 and the ``*_aot`` twins
:1008-1161), so the reference's call sites work unchanged.  Every function
enqueues hand-written HIP kernels through the C ABI in
``include/flash_decode.h`` on the current (or given) torch stream and returns
``output_combine``; nothing synchronises with the host.

Keyword-only additions that the reference does not have (all default off):
  lse_out         fp32 [B, Hq] tensor that receives the merged natural-log LSE
  k_scale/v_scale fp32 [Hkv] dequantisation scales of an fp8-e4m3 KV cache
  extra_partials  (out [E,B,Hq,Dv], lse [E,B,Hq] fp32): further partials merged by
                  the combine, standing in for what other sequence-parallel ranks
                  would contribute
  seq_order       int32 [B] from ``schedule_sequences``: issue order of the sequences (a batch of 64 sequences or
                  more orders its work itself when none is given -- (sequence, range) items up to 192 sequences,
                  whole sequences beyond; ``auto_order=False`` switches that off)
  seq_order_lens  int32 [B], with ``seq_order``: ``kv_lens[seq_order]`` (``rope_kv_append`` writes both), which
                  saves a workgroup one dependent load before it can start
  path            "auto" | "valu" | "mfma"; waves_per_block 0 | 1 | 2 | 4 | 8
  plan_splits     True (default): when ``output_split`` is not supplied, ``kv_split`` is a hint and the library
                  plans the step (``fd_decode_planned``: same result; usually fewer splits -- fewer workgroup prologues
                  and partials --, more for block tables of more than 16384 tokens); False: exactly ``kv_split``
                  splits.  With a caller-supplied ``output_split`` the split count and ranges are always the
                  reference's.
  workspace       the reference's positional argument; a contiguous GPU tensor of at least ``workspace_bytes(...)``
                  bytes on a 256-byte boundary holds partials, LSEs and issue order of a planned step, which then
                  allocates nothing; anything else is ignored, as in the reference
  no_alloc        True: the split partials live in the library's static device array (``fd_decode_noalloc``, at most
                  16 MiB of them) and the call allocates nothing -- for steps captured into a HIP graph or run where
                  allocation is not allowed; needs ``output_combine``; calls that overlap on one GPU must not share it
  rank_merge      ``(global_kv_lens [R, B] int32, this_rank, local_out or None)`` with ``extra_partials`` of the R - 1
                  other ranks in rank order: the combine treats the extras as those ranks' partials -- rank r counts for
                  sequence b iff ``global_kv_lens[r, b] > 0`` (flash_decode.py:513-515) -- and also writes the merge of
                  the local splits alone, LSE in the last column, to ``local_out [B, Hq, Dv + 1]``: intra-rank
                  combine, staging copy and inter-rank combine of the sequence-parallel layer in one launch
  fuse_combine    True: one launch, the combine runs in the tail of the split kernel (pays off when
                  the groups of a ragged batch finish at different times, or for very short steps launched
                  eagerly, where the second launch's host time counts); False (default): split kernel and
                  combine kernel as two launches

Differences from the reference, on purpose: when ``output_split`` is not
supplied the partials stay inside the library as ``[B,Hq,S,Dv]`` with the LSEs
in their own fp32 buffer -- fp32 values, or the output's 16-bit type once there
are 4 MB of them or the caller insists on exactly ``kv_split`` splits
(``fd_plan_decode`` decides; the reference allocates fp16 ``[B,Hq,S,Dv+1]``,
:783-784); the default ``output_combine`` has the query's dtype (the reference
hard-codes fp16, :785, which is the same thing for the fp16 inputs its tests
use).
"""
from __future__ import annotations

from ctypes import addressof, byref
from typing import Optional

import torch

from .._lib import (FD_COMBINE_RANK, FD_COMBINE_SPLIT, FD_COMBINE_SPLIT_LSE, FD_F32, FD_NOALLOC_SCRATCH_BYTES,
                    FD_ORDER_ITEMS, FD_ORDER_SEQUENCES, FD_PATH_AUTO, FD_PATH_MFMA, FD_PATH_VALU,
                    FD_STEP_CALLER_PARTIALS, FD_STEP_EXACT_SPLITS, FD_STEP_FUSED, FD_STEP_LSE_TWICE, FD_STEP_NO_ORDER,
                    FD_STEP_SCHEDULE, FdDecodeArgs, FdLaunchPlan, FdParams, FdRankMerge, check, fd_dtype_of, load_library,
                    stream_handle)

_PATHS = {"auto": FD_PATH_AUTO, "valu": FD_PATH_VALU, "mfma": FD_PATH_MFMA}
DEFAULT_KV_SPLITS = 32  # flash_decode.py:779


def get_split_kv_algo_info(q_heads, kv_heads, q_head_dim, v_head_dim, page_size, split_kv=32, soft_cap=0.0):
    """Counterpart of ``get_triton_split_kv_algo_info`` (flash_decode.py:103-109).  There the dictionary selects an
    ahead-of-time compiled Triton kernel; here it is informational only -- nothing in this package reads it back:
    the library is compiled for every supported combination and picks kernel, tile, waves per workgroup and work
    items per call inside ``fd_split_kv`` / ``fd_decode`` (``fd_plan_splits`` reports the split count it would use).
    The entries describe the kernel family a shape runs on: token tile, query heads per wave, wave size."""
    group = q_heads // kv_heads
    mfma = q_head_dim in (64, 128, 256)   # 16-bit / fp8 caches; fp32 caches run on the VALU kernel
    return {
        "kv_group_num": group, "q_head_num": q_heads, "NUM_KV_SPLITS": split_kv, "PAGE_SIZE": page_size,
        "soft_cap": soft_cap, "K_DIM": q_head_dim, "V_DIM": v_head_dim,
        "path": "mfma" if mfma else "valu", "TILE_N": {64: 64, 128: 32, 256: 16}[q_head_dim] if mfma else None, "BLOCK_H": min(16, group) if mfma else
        min(4, group), "wave_size": 64,
    }


get_triton_split_kv_algo_info = get_split_kv_algo_info  # reference name (kernels/nvidia/__init__.py:34)


def get_combine_kv_algo_info(split_kv=32, v_head_dim=128, block_dv=512):
    """Counterpart of ``get_triton_combine_kv_algo_info`` (flash_decode.py:281-285); informational only, like
    ``get_split_kv_algo_info``: ``fd_combine`` chooses its own launch shape."""
    return {"NUM_KV_SPLITS": split_kv, "Lv": v_head_dim, "BLOCK_DV": block_dv, "wave_size": 64, "waves": 1}


get_triton_combine_kv_algo_info = get_combine_kv_algo_info


def _require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("flash-decode tensors must live on the GPU; this package has no CPU path")


def schedule_sequences(kv_lens: torch.Tensor, out: Optional[torch.Tensor] = None, stream=None) -> torch.Tensor:
    """Kernel (3): int32 [B] sequence order, longest kv_len first, computed on the device."""
    _require_cuda(kv_lens)
    lib = load_library()
    assert kv_lens.dtype == torch.int32 and kv_lens.is_contiguous()
    if out is None:
        out = torch.empty_like(kv_lens)
    check(lib.fd_schedule(stream_handle(stream, kv_lens.device.index), kv_lens.data_ptr(), kv_lens.numel(),
                          out.data_ptr()))
    return out


def _fill_params(t: FdParams, q, k_cache, block_table, kv_split, soft_cap, mid_dtype, out_dtype, fp8, path,
                 waves_per_block, split_align, split_adapt, seq_order_items, max_kv_len, v_head_dim):
    t.q_heads = q.shape[1]
    t.kv_heads = k_cache.shape[2]
    t.head_dim = q.shape[2]
    t.v_head_dim = v_head_dim if v_head_dim and v_head_dim != q.shape[2] else 0
    t.page_size = k_cache.shape[1]
    t.num_splits = kv_split
    t.num_pages = k_cache.shape[0]
    t.max_pages_per_seq = block_table.shape[1]
    t.q_dtype = fd_dtype_of(q)
    t.kv_dtype = fd_dtype_of(k_cache, fp8_bytes=fp8)
    t.mid_dtype = mid_dtype
    t.out_dtype = out_dtype
    t.soft_cap = float(soft_cap or 0.0)
    t.path = _PATHS[path]
    t.waves_per_block = waves_per_block
    t.split_align = split_align
    t.split_adapt = split_adapt
    t.seq_order_items = seq_order_items
    t.max_kv_len = int(max_kv_len or 0)


def _make_params(q, k_cache, block_table, kv_split, soft_cap, mid_dtype, out_dtype, k_scale, v_scale, path,
                 waves_per_block, seq_order_lens=None, split_align=0, split_adapt=0, seq_order_items=0,
                 max_kv_len=0, v_head_dim=0) -> FdParams:
    """``fd_params`` of an explicit call (``fd_decode`` / ``fd_split_kv`` / ``fd_combine``): every field as given."""
    # the scalar fields are the same from step to step: filled once per combination, copied per call
    v_head_dim = v_head_dim or q.shape[2]
    key = (q.shape, k_cache.shape, block_table.shape[1], q.dtype, k_cache.dtype, k_scale is not None, kv_split, soft_cap,
           mid_dtype, out_dtype, path, waves_per_block, split_align, split_adapt, seq_order_items, max_kv_len,
           v_head_dim)
    template = _PARAMS_CACHE.get(key)
    if template is None:
        t = FdParams()
        _fill_params(t, q, k_cache, block_table, kv_split, soft_cap, mid_dtype, out_dtype, k_scale is not None, path,
                     waves_per_block, split_align, split_adapt, seq_order_items, max_kv_len, v_head_dim)
        if len(_PARAMS_CACHE) > 4096:
            _PARAMS_CACHE.clear()
        template = _PARAMS_CACHE[key] = bytes(t)
    p = FdParams.from_buffer_copy(template)
    if k_scale is not None:
        p.k_scale = k_scale.data_ptr()
        p.v_scale = v_scale.data_ptr()
    if seq_order_lens is not None:
        p.seq_order_lens = seq_order_lens.data_ptr()
    return p


_PARAMS_CACHE = {}   # fd_params images by their scalar fields

MAX_ITEM_BATCH = 1024       # sequences fd_schedule_items ranks in one launch
MAX_FUSED_ITEM_BATCH = 256  # ... and fd_kv_append in its trailing workgroup


class DecodePlan:
    """``fd_plan_decode`` for a shape: the library's launch policy as the wrappers see it (read-only)."""
    __slots__ = ("num_splits", "split_adapt", "split_align", "mid_dtype", "direct", "order_kind", "workspace_bytes",
                 "max_kv_len", "launch")

    def __init__(self, lp: FdLaunchPlan):
        self.num_splits, self.split_adapt, self.split_align = lp.num_splits, lp.split_adapt, lp.split_align
        self.mid_dtype, self.direct, self.order_kind = lp.mid_dtype, bool(lp.direct), lp.order_kind
        self.workspace_bytes, self.max_kv_len = lp.workspace_bytes, lp.max_kv_len
        # the launch shape of the split kernel, for tests and reports
        self.launch = dict(mfma=bool(lp.mfma), tile=lp.tile, waves_per_head=lp.waves_per_head, members=lp.members,
                           chunk=lp.chunk, head_block=lp.head_block, grid=tuple(lp.grid),
                           store_through=bool(lp.store_through), partial_bytes=lp.partial_bytes)


def decode_plan(q, k_cache, block_table, kv_split=-1, *, flags=0, out_dtype=None, mid_dtype=FD_F32, num_extra=0,
                fp8=False, path="auto", waves_per_block=0, max_kv_len=None, v_head_dim=0) -> DecodePlan:
    """The library's plan of a decode step of this shape (``fd_plan_decode``; cached by shape): split count and
    ranges, type of the partials, whether the step ranks its work first, workspace size, launch shape.  All launch
    policy lives in the library; the wrappers only carry this out.  ``kv_split`` is the caller's hint (-1: none), or
    the exact count with ``FD_STEP_EXACT_SPLITS`` / ``FD_STEP_CALLER_PARTIALS``."""
    out_dt = fd_dtype_of(q) if out_dtype is None else out_dtype
    hint = -(-max_kv_len // 1024) * 1024 if max_kv_len else 0   # the library plans in steps of 1024 tokens
    key = (q.shape, k_cache.shape[1:], block_table.shape[1], q.dtype, k_cache.dtype, fp8, kv_split, flags, out_dt,
           mid_dtype, num_extra, path, waves_per_block, hint, v_head_dim or q.shape[2])
    plan = _PLAN_CACHE.get(key)
    if plan is None:
        lib = load_library()
        p = FdParams()
        _fill_params(p, q, k_cache, block_table, kv_split, 0.0, mid_dtype, out_dt, fp8, path, waves_per_block, 0, 0, 0,
                     hint, v_head_dim)
        lp = FdLaunchPlan()
        check(lib.fd_plan_decode(byref(p), q.shape[0], num_extra, flags, byref(lp)))
        if len(_PLAN_CACHE) > 4096:
            _PLAN_CACHE.clear()
        plan = _PLAN_CACHE[key] = DecodePlan(lp)
    return plan


def plan_decode(q, k_cache, block_table, kv_split=-1, *, k_scale=None, v_scale=None, path="auto", waves_per_block=0,
                max_kv_len=None, v_head_dim=0):
    """``(num_splits, split_adapt)`` of a decode step whose partials stay inside the library: grid slots per sequence
    and the ranges every sequence gets however short it is (see ``decode_plan``)."""
    plan = decode_plan(q, k_cache, block_table, kv_split, fp8=k_scale is not None, path=path,
                       waves_per_block=waves_per_block, max_kv_len=max_kv_len, v_head_dim=v_head_dim)
    return plan.num_splits, plan.split_adapt


def workspace_bytes(q, k_cache, block_table, kv_split=-1, **kw) -> int:
    """Bytes of workspace a planned decode step of this shape uses (``fd_workspace_bytes``): a contiguous GPU tensor of
    at least that many bytes passed as ``workspace`` makes the step allocation-free.  Keywords as for ``decode_plan``."""
    return decode_plan(q, k_cache, block_table, kv_split, **kw).workspace_bytes


def item_order_buffer(batch, num_splits, device):
    """Storage for the work-item order of ``fd_schedule_items`` / ``rope_kv_append(item_order_out=)``."""
    return torch.empty(2 * batch * num_splits, dtype=torch.int32, device=device)


_STEP_CACHE = {}   # fd_decode_args images of planned steps by everything but the pointers


def _decode(q, k_cache, v_cache, workspace, kv_lens, block_table, scale, soft_cap, output_split, output_combine,
            kv_split, *, with_lse_column: bool, lse_out=None, k_scale=None, v_scale=None, extra_partials=None, seq_order=None,
            seq_order_lens=None, stream=None, path="auto", waves_per_block=0, fuse_combine=False, plan_splits=True,
            schedule_items=False, item_order=None, max_kv_len=None, no_alloc=False, auto_order=True, rank_merge=None,
            _prepare=False):
    batch, q_heads, q_head_dim = q.shape
    _, page_size, kv_heads, k_head_dim = k_cache.shape
    v_shape = v_cache.shape
    assert page_size == v_shape[1] and kv_heads == v_shape[2] and k_head_dim == q_head_dim
    v_head_dim = v_shape[3]
    assert q_heads % kv_heads == 0
    if not (q.is_cuda and k_cache.is_cuda and v_cache.is_cuda and kv_lens.is_cuda and block_table.is_cuda):
        _require_cuda(q, k_cache, v_cache, kv_lens, block_table)
    assert kv_lens.dtype == torch.int32 and block_table.dtype == torch.int32
    q_st, k_st, v_st = q.stride(), k_cache.stride(), v_cache.stride()
    assert q_st[2] == 1 and k_st[3] == 1 and v_st[3] == 1
    # kv_loc = page * P + slot is a flat token index (flash_decode.py:205-206): the pool must be linear in it
    assert k_st[0] == page_size * k_st[1] and v_st[0] == page_size * v_st[1]
    if (k_scale is None) != (v_scale is None):
        raise RuntimeError("k_scale and v_scale must be given together")
    out_cols = v_head_dim + 1 if with_lse_column else v_head_dim
    if output_combine is None:
        if no_alloc:
            raise RuntimeError("no_alloc=True needs output_combine")
        output_combine = torch.empty([batch, q_heads, out_cols], dtype=q.dtype, device=q.device)
    else:
        _require_cuda(output_combine)
    oc_st = output_combine.stride()
    assert output_combine.shape[-1] >= out_cols and oc_st[-1] == 1
    ex_out = ex_lse = None
    n_extra = 0
    if extra_partials is not None:
        ex_out, ex_lse = extra_partials
        _require_cuda(ex_out, ex_lse)
        n_extra = ex_out.shape[0]
        assert tuple(ex_out.shape) == (n_extra, batch, q_heads, v_head_dim) and ex_out.is_contiguous()
        assert tuple(ex_lse.shape) == (n_extra, batch, q_heads) and ex_lse.dtype == torch.float32
        assert ex_lse.is_contiguous() and ex_out.dtype == output_combine.dtype
    if lse_out is not None:
        assert lse_out.dtype == torch.float32 and lse_out.is_contiguous() and lse_out.numel() == batch * q_heads
    rm = None
    if rank_merge is not None:
        # sequence-parallel decode: the extras stand for the other ranks (fd_rank_merge)
        rank_lens, this_rank, local_out = rank_merge
        _require_cuda(rank_lens, local_out)
        assert rank_lens.dtype == torch.int32 and rank_lens.is_contiguous()
        assert tuple(rank_lens.shape) == (n_extra + 1, batch) and 0 <= this_rank <= n_extra
        if fuse_combine:
            raise RuntimeError("rank_merge is not available with fuse_combine")
        rm = FdRankMerge()
        rm.rank_lens, rm.this_rank = rank_lens.data_ptr(), this_rank
        if local_out is not None:
            assert tuple(local_out.shape) == (batch, q_heads, v_head_dim + 1) and local_out.stride(2) == 1
            rm.local_out, rm.local_dtype = local_out.data_ptr(), fd_dtype_of(local_out)
            rm.stride_lb, rm.stride_lh = local_out.stride(0), local_out.stride(1)
    if seq_order_lens is not None:
        assert seq_order is not None and seq_order_lens.dtype == torch.int32 and seq_order_lens.is_contiguous()
        assert seq_order_lens.numel() == batch
    lib = load_library()
    hstream = stream.cuda_stream if stream is not None else stream_handle(None, q.device.index)
    flags = ((0 if plan_splits else FD_STEP_EXACT_SPLITS) | (FD_STEP_SCHEDULE if schedule_items else 0)
             | (0 if auto_order else FD_STEP_NO_ORDER))

    if output_split is None and not fuse_combine and not no_alloc:
        # ---- the planned step: the library chooses splits, ranges, partial type and issue order (fd_decode_planned);
        # partials, LSEs and the order live in one workspace
        if item_order is not None:
            assert item_order.dtype == torch.int32 and item_order.is_contiguous()
            seq_order = item_order
        # (the length hint counts in steps of 1024 tokens, so that a growing batch keeps its prepared step)
        hint = -(-max_kv_len // 1024) * 1024 if max_kv_len else 0
        key = (q.shape, q_st, k_cache.shape, k_st, v_shape, v_st, block_table.shape[1], block_table.stride(0), oc_st,
               q.dtype, k_cache.dtype, output_combine.dtype, kv_split, soft_cap, scale, flags, with_lse_column,
               n_extra, path, waves_per_block, hint, k_scale is not None, item_order is not None)
        cached = _STEP_CACHE.get(key)
        if cached is None:
            a = FdDecodeArgs()
            a.stride_q_bs, a.stride_q_h = q_st[0], q_st[1]
            a.stride_k_tok, a.stride_k_h, a.stride_v_tok, a.stride_v_h = k_st[1], k_st[2], v_st[1], v_st[2]
            a.stride_table_bs, a.stride_obs, a.stride_oh = block_table.stride(0), oc_st[0], oc_st[1]
            a.sm_scale, a.batch, a.num_extra, a.flags = float(scale), batch, n_extra, flags
            a.combine_mode = FD_COMBINE_SPLIT_LSE if with_lse_column else FD_COMBINE_SPLIT
            _fill_params(a.params, q, k_cache, block_table, kv_split, soft_cap, FD_F32, fd_dtype_of(output_combine),
                         k_scale is not None, path, waves_per_block, 0, 0, 1 if item_order is not None else 0,
                         hint, v_head_dim)
            need = lib.fd_workspace_bytes(byref(a.params), batch, n_extra, flags)
            if need < 0:
                check(int(need))
            if len(_STEP_CACHE) > 4096:
                _STEP_CACHE.clear()
            cached = _STEP_CACHE[key] = (bytes(a), need)
        image, need = cached
        a = FdDecodeArgs.from_buffer_copy(image)
        if (workspace is not None and isinstance(workspace, torch.Tensor) and workspace.is_cuda
                and workspace.is_contiguous() and workspace.data_ptr() % 256 == 0
                and workspace.numel() * workspace.element_size() >= need):
            hold = workspace     # the caller's workspace is large enough: no allocation in the call
        else:
            hold = torch.empty(need, dtype=torch.uint8, device=q.device)
            if stream is not None:   # freed on return: keep the allocator from reusing it before `stream` is done
                hold.record_stream(stream)
        a.q, a.k_cache, a.v_cache = q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr()
        a.workspace, a.workspace_bytes = hold.data_ptr(), need
        a.out, a.block_table, a.kv_lens = output_combine.data_ptr(), block_table.data_ptr(), kv_lens.data_ptr()
        if lse_out is not None:
            a.lse_out = lse_out.data_ptr()
        if seq_order is not None:
            a.seq_order = seq_order.data_ptr()
            if seq_order_lens is not None:
                a.params.seq_order_lens = seq_order_lens.data_ptr()
        if n_extra:
            a.extra_out, a.extra_lse = ex_out.data_ptr(), ex_lse.data_ptr()
        if k_scale is not None:
            a.params.k_scale, a.params.v_scale = k_scale.data_ptr(), v_scale.data_ptr()
        if rm is not None:
            a.params.rank_merge = addressof(rm)
        if _prepare:   # PreparedDecode: the marshalled step and what must stay alive with it
            return a, (hold, rm, output_combine)
        rc = lib.fd_decode_planned(hstream, byref(a))
        if rc:
            check(rc)
        return output_combine

    if _prepare:
        raise RuntimeError("PreparedDecode covers the planned step: no output_split, fuse_combine or no_alloc")
    # ---- explicit calls: the caller's own partial buffer (exactly kv_split splits with the reference's ranges, layout
    # [B, Hq, S, Dv + 1]), the fused single launch, or partials in the library's static array.  How the step is issued
    # still comes from the library's plan.
    out_dtype = fd_dtype_of(output_combine)
    lse_twice = FD_STEP_LSE_TWICE if with_lse_column and lse_out is not None else 0
    if item_order is not None or seq_order is not None:
        flags |= FD_STEP_NO_ORDER     # the caller brings the order
    if output_split is not None:
        _require_cuda(output_split)
        assert output_split.shape[-1] == v_head_dim + 1 and output_split.stride(-1) == 1
        num_splits = DEFAULT_KV_SPLITS if kv_split == -1 else kv_split
        assert output_split.shape[2] == num_splits
        if no_alloc:
            raise RuntimeError("no_alloc=True keeps the partials inside the library; output_split cannot be given")
        plan = decode_plan(q, k_cache, block_table, num_splits, flags=flags | FD_STEP_CALLER_PARTIALS | lse_twice
                           | (FD_STEP_FUSED if fuse_combine else 0), out_dtype=out_dtype,
                           mid_dtype=fd_dtype_of(output_split), num_extra=n_extra, fp8=k_scale is not None, path=path,
                           waves_per_block=waves_per_block, max_kv_len=max_kv_len, v_head_dim=v_head_dim)
        hold = None
        mid_ptr, lse_split_ptr = output_split.data_ptr(), None
        so_b, so_h, so_s = output_split.stride(0), output_split.stride(1), output_split.stride(2)
    else:
        if no_alloc and (fuse_combine or schedule_items):
            raise RuntimeError("no_alloc=True needs output_combine and neither fuse_combine nor a scheduling launch")
        plan = decode_plan(q, k_cache, block_table, kv_split, flags=flags | lse_twice | (FD_STEP_NO_ORDER if no_alloc else 0)
                           | (FD_STEP_FUSED if fuse_combine or no_alloc else 0), out_dtype=out_dtype, num_extra=n_extra,
                           fp8=k_scale is not None, path=path, waves_per_block=waves_per_block, max_kv_len=max_kv_len,
                           v_head_dim=v_head_dim)
        num_splits = plan.num_splits
        n_o = batch * q_heads * num_splits * v_head_dim
        n_l = batch * q_heads * num_splits
        if no_alloc:
            # the partials live in the library's static device array (fd_decode_noalloc); nothing is allocated here
            if n_o + n_l > FD_NOALLOC_SCRATCH_BYTES // 4:
                raise RuntimeError(f"no_alloc=True: {4 * (n_o + n_l)} bytes of partials exceed the library's static "
                                   f"workspace of {FD_NOALLOC_SCRATCH_BYTES} bytes")
            hold = None
        elif (isinstance(workspace, torch.Tensor) and workspace.dtype == torch.float32 and workspace.is_cuda
                and workspace.is_contiguous() and workspace.numel() >= n_o + n_l):
            hold = workspace
        else:
            hold = torch.empty(n_o + n_l, dtype=torch.float32, device=q.device)
            if stream is not None:
                hold.record_stream(stream)
        mid_ptr = hold.data_ptr() if hold is not None else None
        lse_split_ptr = mid_ptr + 4 * n_o if hold is not None else None
        so_b, so_h, so_s = q_heads * num_splits * v_head_dim, num_splits * v_head_dim, v_head_dim
    want_items = (item_order is not None and num_splits > 1 and not fuse_combine) or plan.order_kind == FD_ORDER_ITEMS
    if plan.order_kind == FD_ORDER_SEQUENCES:
        seq_order = schedule_sequences(kv_lens, stream=stream)
        if stream is not None:
            seq_order.record_stream(stream)
    p = _make_params(q, k_cache, block_table, num_splits, soft_cap, plan.mid_dtype, out_dtype, k_scale, v_scale, path,
                     waves_per_block, seq_order_lens, plan.split_align, plan.split_adapt, 0, plan.max_kv_len, v_head_dim)
    if want_items:
        # (sequence, range) items, largest first, empty ranges last: given by the caller (the append launch computed
        # it) or computed here by one scheduling launch.  With the caller's exact split count the items are the
        # reference's ranges (every slot of the partial buffer is still written, empty ranges last).
        if item_order is None:
            item_order = item_order_buffer(batch, num_splits, q.device)
            if stream is not None:
                item_order.record_stream(stream)
            check(lib.fd_schedule_items(hstream, kv_lens.data_ptr(), batch, item_order.data_ptr(), byref(p)))
        assert item_order.dtype == torch.int32 and item_order.is_contiguous()
        assert item_order.numel() >= 2 * batch * num_splits
        p.seq_order_items = 1
        p.seq_order_lens = None
        seq_order = item_order
    mode = FD_COMBINE_SPLIT_LSE if with_lse_column else FD_COMBINE_SPLIT
    if rm is not None:
        p.rank_merge = addressof(rm)
    if no_alloc:
        check(lib.fd_decode_noalloc(
            hstream, q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), output_combine.data_ptr(),
            lse_out.data_ptr() if lse_out is not None else None, float(scale), block_table.data_ptr(),
            kv_lens.data_ptr(), batch, q_st[0], q_st[1], k_st[1], k_st[2], v_st[1], v_st[2], block_table.stride(0),
            oc_st[0], oc_st[1], seq_order.data_ptr() if seq_order is not None else None, mode,
            ex_out.data_ptr() if n_extra else None, ex_lse.data_ptr() if n_extra else None, n_extra, byref(p)))
        return output_combine
    tickets = _tickets(q.device, hstream, batch * q_heads) if fuse_combine else None
    check(lib.fd_decode(
        hstream, q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), mid_ptr, lse_split_ptr,
        output_combine.data_ptr(), lse_out.data_ptr() if lse_out is not None else None, float(scale),
        block_table.data_ptr(), kv_lens.data_ptr(), batch,
        q_st[0], q_st[1], k_st[1], k_st[2], v_st[1], v_st[2],
        so_b, so_h, so_s, block_table.stride(0), oc_st[0], oc_st[1],
        seq_order.data_ptr() if seq_order is not None else None, mode,
        ex_out.data_ptr() if n_extra else None, ex_lse.data_ptr() if n_extra else None, n_extra,
        tickets.data_ptr() if tickets is not None else None, byref(p)))
    return output_combine


class PreparedDecode:
    """A planned decode step whose arguments are marshalled once (``fd_decode_args``) and launched many times: a
    serving loop decodes with the same buffers step after step -- the query buffer, the cache pools, the block table,
    ``kv_lens`` and the output keep their addresses, only their contents change -- so all that is left per step is one
    library call (about 6 us on the host with its two launches, against about 10 us through the wrappers, which check
    and marshal two dozen arguments every time, as the reference's do, flash_decode.py:788-844).

        step = PreparedDecode(q, k_cache, v_cache, kv_lens, block_table, scale, output_combine=out, lse_out=lse)
        for _ in range(n):
            ...                       # new contents in q / the caches / kv_lens / block_table
            step()                    # -> out

    ``variant``: "plain" (``gqa_fwd_batch_decode``), "intra_rank" (merged LSE in the output's last column) or
    "persistent" (the scheduled variant).  Every keyword of the planned step is accepted (``kv_split``, ``soft_cap``,
    ``k_scale`` / ``v_scale``, ``extra_partials``, ``seq_order``, ``max_kv_len``, ``workspace`` ...).  The object keeps
    the tensors alive; ``step(k_cache=..., v_cache=...)`` rebinds tensors of the same shape, dtype and strides (a
    rotating pool).  Calls on one object must not overlap: they share its workspace.  Capturable into a HIP graph
    like the wrappers (the step allocates nothing)."""

    _REBINDABLE = {"q": "q", "k_cache": "k_cache", "v_cache": "v_cache", "kv_lens": "kv_lens",
                   "block_table": "block_table", "output_combine": "out", "lse_out": "lse_out"}

    def __init__(self, q, k_cache, v_cache, kv_lens, block_table, scale, soft_cap=0.0, *, variant="plain",
                 output_combine=None, kv_split=-1, workspace=None, stream=None, **kw):
        if variant not in ("plain", "intra_rank", "persistent"):
            raise ValueError(f"variant {variant!r}")
        if variant == "persistent" and kw.get("seq_order") is None and kw.get("item_order") is None and q.shape[0] > 1:
            kw["schedule_items"] = True
        cols = v_cache.shape[-1] + (1 if variant == "intra_rank" else 0)
        if output_combine is None:
            output_combine = torch.empty(q.shape[0], q.shape[1], cols, dtype=q.dtype, device=q.device)
        self._lib = load_library()
        self._stream = stream
        self._device = q.device.index
        self._args, self._keep = _decode(q, k_cache, v_cache, workspace, kv_lens, block_table, scale, soft_cap, None,
                                         output_combine, kv_split, with_lse_column=variant == "intra_rank",
                                         stream=stream, _prepare=True, **kw)
        self._ref = byref(self._args)
        self._tensors = dict(q=q, k_cache=k_cache, v_cache=v_cache, kv_lens=kv_lens, block_table=block_table,
                             output_combine=output_combine, lse_out=kw.get("lse_out"), kw=kw)
        self.output = output_combine

    def __call__(self, stream=None, **rebind):
        for name, t in rebind.items():
            field = self._REBINDABLE[name]
            old = self._tensors[name]
            if old is None or t.shape != old.shape or t.stride() != old.stride() or t.dtype != old.dtype \
                    or t.device != old.device:
                raise RuntimeError(f"PreparedDecode: {name} must keep shape, strides, dtype and device")
            setattr(self._args, field, t.data_ptr())
            self._tensors[name] = t
            if name == "output_combine":
                self.output = t
        s = stream if stream is not None else self._stream
        rc = self._lib.fd_decode_planned(s.cuda_stream if s is not None else stream_handle(None, self._device),
                                         self._ref)
        if rc:
            check(rc)
        return self.output


_PLAN_CACHE = {}   # fd_plan_decode results by problem shape

# Zero-initialised ticket counters of the fused combine, one buffer per (device, stream): calls on
# different streams may overlap and must not share counters; the kernels leave them at zero.
_TICKETS = {}


def _tickets(device, hstream, n):
    key = (device.index, hstream)
    t = _TICKETS.get(key)
    if t is None or t.numel() < n:
        t = torch.zeros(max(n, 4096), dtype=torch.int32, device=device)
        _TICKETS[key] = t
    return t


def gqa_fwd_batch_decode(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale, soft_cap=0.0,
                         output_split=None, output_combine=None, kv_split=-1, **kw):
    """Split-KV decode + plain combine -> ``output_combine [B, Hq, Dv]`` (flash_decode.py:763-844).

    ``q_lens`` is accepted and ignored, as in the reference; so is ``workspace``, unless it is a
    contiguous GPU tensor of at least ``workspace_bytes(...)`` bytes on a 256-byte boundary, in which case partials,
    LSEs and issue order of the step live in it instead of in freshly allocated memory.  Keyword ``max_kv_len=``: an upper bound of
    ``kv_lens`` that the caller knows on the host; the launch shape is then planned for it instead of for the block
    table's capacity (a hint only: longer sequences are still decoded in full).
    """
    return _decode(q, k_cache, v_cache, workspace, kv_lens, block_table, scale, soft_cap, output_split, output_combine, kv_split,
                   with_lse_column=False, **kw)


def gqa_fwd_batch_decode_intra_rank(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale,
                                    soft_cap=0.0, output_split=None, output_combine=None, kv_split=-1, **kw):
    """Split-KV decode + combine that also stores the merged LSE at column Dv:
    ``output_combine [B, Hq, Dv+1]`` (flash_decode.py:847-928)."""
    return _decode(q, k_cache, v_cache, workspace, kv_lens, block_table, scale, soft_cap, output_split, output_combine, kv_split,
                   with_lse_column=True, **kw)


def gqa_fwd_batch_decode_persistent(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale, soft_cap=0,
                                    output_split=None, output_combine=None, kv_split=-1, **kw):
    """Scheduled variant (flash_decode.py:931-1005).  The reference fuses split and combine
    behind a spinning grid barrier on a fixed 132-workgroup grid; here the device-side
    scheduler orders the sequences longest first and the hardware dispatcher balances the
    workgroups over the CUs, so no co-residency assumption is needed."""
    if kw.get("seq_order") is None and kw.get("item_order") is None and q.shape[0] > 1:
        kw["schedule_items"] = True   # a single sequence has nothing to order
    return _decode(q, k_cache, v_cache, workspace, kv_lens, block_table, scale, soft_cap, output_split, output_combine, kv_split,
                   with_lse_column=False, **kw)


def gqa_fwd_batch_decode_aot(stream, q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale, soft_cap=0,
                             output_split=None, output_combine=None, kv_split=-1, **kw):
    """Explicit-stream twin of ``gqa_fwd_batch_decode`` (flash_decode.py:1008-1063).  The library
    is always ahead-of-time compiled, so no environment switch is involved."""
    return gqa_fwd_batch_decode(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale, soft_cap,
                                output_split, output_combine, kv_split, stream=stream, **kw)


def gqa_fwd_batch_decode_intra_rank_aot(stream, q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale,
                                        soft_cap=0, output_split=None, output_combine=None, kv_split=-1, **kw):
    """Explicit-stream twin of ``gqa_fwd_batch_decode_intra_rank`` (flash_decode.py:1066-1121)."""
    return gqa_fwd_batch_decode_intra_rank(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale,
                                           soft_cap, output_split, output_combine, kv_split, stream=stream, **kw)


def gqa_fwd_batch_decode_persistent_aot(stream, q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale,
                                        soft_cap=0, output_split=None, output_combine=None, kv_split=-1, **kw):
    """Explicit-stream twin of ``gqa_fwd_batch_decode_persistent`` (flash_decode.py:1124-1161)."""
    return gqa_fwd_batch_decode_persistent(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale,
                                           soft_cap, output_split, output_combine, kv_split, stream=stream, **kw)


def inter_rank_combine(all_ranks_out: torch.Tensor, final_out: torch.Tensor, global_kv_lens: torch.Tensor,
                       lse_out: Optional[torch.Tensor] = None, stream=None) -> torch.Tensor:
    """Merges per-rank partials ``[R, B, Hq, Dv+1]`` (LSE at column Dv) into ``final_out [B, Hq, Dv]``;
    rank r contributes to sequence b iff ``global_kv_lens[r, b] > 0`` (flash_decode.py:482-532)."""
    R, batch, q_heads, d1 = all_ranks_out.shape
    return _inter_rank_launch(all_ranks_out, final_out, global_kv_lens, batch, q_heads, all_ranks_out.stride(1),
                              all_ranks_out.stride(2), all_ranks_out.stride(0), final_out.stride(0),
                              final_out.stride(1), R, 512, d1 - 1, lse_out=lse_out, stream=stream)


def _inter_rank_launch(Mid_O, o, B_Seqlens, batch, q_heads, stride_mid_ob, stride_mid_oh, stride_mid_os, stride_obs,
                       stride_oh, NUM_KV_SPLITS, BLOCK_DV, Lv, lse_out=None, stream=None):
    _require_cuda(Mid_O, o, B_Seqlens)
    assert B_Seqlens.dtype == torch.int32 and B_Seqlens.is_contiguous()
    assert Mid_O.stride(-1) == 1 and o.stride(-1) == 1
    lib = load_library()
    p = FdParams()
    p.q_heads = q_heads
    p.head_dim = Lv
    p.mid_dtype = fd_dtype_of(Mid_O)
    p.out_dtype = fd_dtype_of(o)
    check(lib.fd_combine(
        stream_handle(stream, o.device.index), Mid_O.data_ptr(), None, o.data_ptr(),
        lse_out.data_ptr() if lse_out is not None else None, B_Seqlens.data_ptr(), batch, q_heads, NUM_KV_SPLITS,
        stride_mid_ob, stride_mid_oh, stride_mid_os, stride_obs, stride_oh, FD_COMBINE_RANK, None, None, 0, byref(p)))
    return o


class _InterRankCombineKernel:
    """Callable with the launch syntax of the reference's Triton kernel
    ``kernel_inter_rank_gqa_fwd_batch_decode_combine_kv[grid](Mid_O, o, B_Seqlens, batch, q_heads,
    stride_mid_ob, stride_mid_oh, stride_mid_os, stride_obs, stride_oh, NUM_KV_SPLITS, BLOCK_DV, Lv)``
    (flash_decode.py:482-497; launched at layers/nvidia/sp_flash_decode_layer.py:173-183).
    The grid and BLOCK_DV are accepted and ignored: the HIP launch derives its own."""

    def __getitem__(self, grid):
        return _inter_rank_launch

    def __call__(self, *args, **kw):
        return _inter_rank_launch(*args, **kw)


kernel_inter_rank_gqa_fwd_batch_decode_combine_kv = _InterRankCombineKernel()
