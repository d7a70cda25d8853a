"""The ctypes binding a maintainer of the reference tree would add for gfx950: a self-contained module (it imports
nothing from this package) that binds ``fd_decode``, ``fd_decode_planned`` and ``fd_kv_append`` of
libflash_decode_gfx950.so and offers

* ``gqa_fwd_batch_decode`` with the reference's signature (flash_decode.py:763-844) -- without ``output_split`` (the
  reference's tests, test_decode_attn.py:158) the library plans the step itself; with it (the perf scripts and the
  sequence-parallel layer, test_decode_attn.py:322-331, sp_flash_decode_layer.py:95-110) the caller gets exactly
  ``kv_split`` partials in the reference's layout -- and
* ``rope_and_update_cache``: the rotary of q and k plus the cache write that precede the attention call in
  ``TP_Attn.torch_fwd`` (layers/amd/tp_attn.py:262-269), as one launch.

In the reference tree the file would live at python/triton_dist/kernels/amd/flash_decode_gfx950.py.  The library is
looked up through ``FD_LIBRARY_PATH`` and then beside this file.  ``kernels/flash_decode.py`` and
``kernels/kv_append.py`` of this package are the complete versions (all wrappers, fp8 scales, extra partials,
scheduler order, fused combine, fp32 LSE output, norms).
"""
import ctypes
import os

import torch
from ctypes import c_void_p, c_int32, c_int64, c_float, POINTER, Structure, byref

class FdParams(Structure):            # struct fd_params, include/flash_decode.h
    _fields_ = [("q_heads", c_int32), ("kv_heads", c_int32), ("head_dim", c_int32), ("page_size", c_int32),
                ("num_splits", c_int32), ("num_pages", c_int32), ("max_pages_per_seq", c_int32),
                ("q_dtype", c_int32), ("kv_dtype", c_int32), ("mid_dtype", c_int32), ("out_dtype", c_int32),
                ("soft_cap", c_float), ("k_scale", c_void_p), ("v_scale", c_void_p),
                ("path", c_int32), ("waves_per_block", c_int32), ("seq_order_lens", c_void_p),
                ("split_align", c_int32), ("split_adapt", c_int32),
                ("max_kv_len", c_int32), ("seq_order_items", c_int32), ("v_head_dim", c_int32),
                ("rank_merge", c_void_p)]

class FdDecodeArgs(Structure):        # struct fd_decode_args, include/flash_decode.h
    _fields_ = [("q", c_void_p), ("k_cache", c_void_p), ("v_cache", c_void_p), ("workspace", c_void_p),
                ("workspace_bytes", c_int64), ("out", c_void_p), ("lse_out", c_void_p), ("block_table", c_void_p),
                ("kv_lens", c_void_p), ("seq_order", c_void_p), ("extra_out", c_void_p), ("extra_lse", c_void_p),
                ("stride_q_bs", c_int64), ("stride_q_h", c_int64), ("stride_k_tok", c_int64), ("stride_k_h", c_int64),
                ("stride_v_tok", c_int64), ("stride_v_h", c_int64), ("stride_table_bs", c_int64),
                ("stride_obs", c_int64), ("stride_oh", c_int64), ("sm_scale", c_float), ("batch", c_int32),
                ("combine_mode", c_int32), ("num_extra", c_int32), ("flags", c_int32), ("params", FdParams)]

_lib = ctypes.CDLL(os.environ.get("FD_LIBRARY_PATH") or
                   os.path.join(os.path.dirname(os.path.abspath(__file__)), "libflash_decode_gfx950.so"))
i64 = c_int64
_lib.fd_decode.restype = c_int32
_lib.fd_decode.argtypes = [c_void_p] * 8 + [c_float, c_void_p, c_void_p, c_int32] + [i64] * 12 + \
                          [c_void_p, c_int32, c_void_p, c_void_p, c_int32, c_void_p, POINTER(FdParams)]
_lib.fd_decode_planned.restype = c_int32
_lib.fd_decode_planned.argtypes = [c_void_p, POINTER(FdDecodeArgs)]
_lib.fd_workspace_bytes.restype = c_int64
_lib.fd_workspace_bytes.argtypes = [POINTER(FdParams), c_int32, c_int32, c_int32]
_lib.fd_last_error.restype = ctypes.c_char_p
FD_F32, FD_F16, FD_BF16, FD_FP8_E4M3 = 0, 1, 2, 3
_DT = {torch.float32: FD_F32, torch.float16: FD_F16, torch.bfloat16: FD_BF16}

def gqa_fwd_batch_decode(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale, soft_cap=0.0,
                         output_split=None, output_combine=None, kv_split=-1):
    B, Hq, D = q.shape
    if output_combine is None:
        output_combine = torch.empty(B, Hq, D, dtype=q.dtype, device=q.device)
    stream = torch.cuda.current_stream().cuda_stream
    if output_split is None:
        # nobody sees the partials (the reference allocates and drops them, flash_decode.py:783-784): the library plans
        # the step -- split count, ranges, partial type, issue order -- and keeps all of it in one workspace
        a = FdDecodeArgs()
        a.params = FdParams(Hq, k_cache.shape[2], D, k_cache.shape[1], kv_split, k_cache.shape[0],
                            block_table.shape[1], _DT[q.dtype], _DT[k_cache.dtype], FD_F32, _DT[output_combine.dtype],
                            float(soft_cap), None, None, 0, 0)
        need = _lib.fd_workspace_bytes(byref(a.params), B, 0, 0)
        if need < 0:
            raise RuntimeError(_lib.fd_last_error().decode())
        if not (torch.is_tensor(workspace) and workspace.is_cuda and workspace.is_contiguous()
                and workspace.data_ptr() % 256 == 0 and workspace.numel() * workspace.element_size() >= need):
            workspace = torch.empty(need, dtype=torch.uint8, device=q.device)   # the reference's is too small to use
        a.q, a.k_cache, a.v_cache, a.out = q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), output_combine.data_ptr()
        a.workspace, a.workspace_bytes = workspace.data_ptr(), need
        a.block_table, a.kv_lens, a.batch, a.sm_scale = block_table.data_ptr(), kv_lens.data_ptr(), B, float(scale)
        a.stride_q_bs, a.stride_q_h = q.stride(0), q.stride(1)
        a.stride_k_tok, a.stride_k_h = k_cache.stride(-3), k_cache.stride(-2)
        a.stride_v_tok, a.stride_v_h = v_cache.stride(-3), v_cache.stride(-2)
        a.stride_table_bs, a.stride_obs, a.stride_oh = block_table.stride(0), output_combine.stride(0), output_combine.stride(1)
        if _lib.fd_decode_planned(stream, byref(a)):
            raise RuntimeError(_lib.fd_last_error().decode())
        return output_combine
    S = 32 if kv_split == -1 else kv_split                                   # flash_decode.py:779
    p = FdParams(Hq, k_cache.shape[2], D, k_cache.shape[1], S, k_cache.shape[0], block_table.shape[1],
                 _DT[q.dtype], _DT[k_cache.dtype], _DT[output_split.dtype], _DT[output_combine.dtype],
                 float(soft_cap), None, None, 0, 0)
    rc = _lib.fd_decode(stream, q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                        output_split.data_ptr(), None, output_combine.data_ptr(), None, float(scale),
                        block_table.data_ptr(), kv_lens.data_ptr(), B,
                        q.stride(0), q.stride(1), k_cache.stride(-3), k_cache.stride(-2),
                        v_cache.stride(-3), v_cache.stride(-2),
                        output_split.stride(0), output_split.stride(1), output_split.stride(2), block_table.stride(0),
                        output_combine.stride(0), output_combine.stride(1),
                        None, 0, None, None, 0, None, byref(p))
    if rc:
        raise RuntimeError(_lib.fd_last_error().decode())
    return output_combine


class FdQkPrep(Structure):              # struct fd_qk_prep, include/flash_decode.h
    _fields_ = [("cos_sin", c_void_p), ("stride_cos_sin", c_int64), ("position_ids", c_void_p),
                ("position_dtype", c_int32), ("max_positions", c_int32), ("stride_pos_b", c_int64),
                ("stride_pos_t", c_int64), ("q", c_void_p), ("q_out", c_void_p),
                ("stride_q_b", c_int64), ("stride_q_t", c_int64), ("stride_q_h", c_int64),
                ("stride_qo_b", c_int64), ("stride_qo_t", c_int64), ("stride_qo_h", c_int64),
                ("q_norm_weight", c_void_p), ("k_norm_weight", c_void_p),     # optional per-head RMS norm before the rotary
                ("q_norm_eps", c_float), ("k_norm_eps", c_float)]

_lib.fd_kv_append.restype = c_int32
_lib.fd_kv_append.argtypes = [c_void_p] * 9 + [c_int32, c_int32] + [i64] * 11 + [POINTER(FdQkPrep), POINTER(FdParams)]

def rope_and_update_cache(q, k, v, k_cache, v_cache, block_table, kv_offset, kv_offset_out, cos_sin, position_ids):
    """q [B,T,Hq,D] rotated in place; k rotated and stored with v at kv_offset[b].. in the paged pools."""
    B, T, Hq, D = q.shape
    r = FdQkPrep(cos_sin.data_ptr(), cos_sin.stride(0), position_ids.data_ptr(), int(position_ids.dtype == torch.int64),
               cos_sin.shape[0], position_ids.stride(0), position_ids.stride(1), q.data_ptr(), q.data_ptr(),
               *q.stride()[:3], *q.stride()[:3], None, None, 0.0, 0.0)
    p = FdParams(Hq, k.shape[2], D, k_cache.shape[1], 1, k_cache.shape[0], block_table.shape[1],
                 _DT[q.dtype], _DT[k_cache.dtype], FD_F32, FD_F32, 0.0, None, None, 0, 0)
    rc = _lib.fd_kv_append(torch.cuda.current_stream().cuda_stream, k.data_ptr(), v.data_ptr(), k_cache.data_ptr(),
                           v_cache.data_ptr(), block_table.data_ptr(), kv_offset.data_ptr(), kv_offset_out.data_ptr(),
                           None, B, T, *k.stride()[:3], *v.stride()[:3], k_cache.stride(1), k_cache.stride(2),
                           v_cache.stride(1), v_cache.stride(2), block_table.stride(0), byref(r), byref(p))
    if rc:
        raise RuntimeError(_lib.fd_last_error().decode())
