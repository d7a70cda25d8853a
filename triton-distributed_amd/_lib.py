"""ctypes binding of libflash_decode_gfx950.so (the C ABI declared in include/flash_decode.h).

The library is the only compute path of this package: if it is missing or a
call fails, a ``RuntimeError`` is raised.  There is no CPU or PyTorch fallback.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int32, c_int64, c_void_p

import torch

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libflash_decode_gfx950.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)

FD_ABI_VERSION = 3

# fd_dtype
FD_F32, FD_F16, FD_BF16, FD_FP8_E4M3 = 0, 1, 2, 3
# fd_path
FD_PATH_AUTO, FD_PATH_VALU, FD_PATH_MFMA = 0, 1, 2
# fd_combine_mode
FD_COMBINE_SPLIT, FD_COMBINE_SPLIT_LSE, FD_COMBINE_RANK = 0, 1, 2
FD_NOALLOC_SCRATCH_BYTES = 16 << 20   # static partial workspace of fd_decode_noalloc
# fd_step_flags
FD_STEP_EXACT_SPLITS, FD_STEP_SCHEDULE, FD_STEP_NO_ORDER, FD_STEP_FUSED, FD_STEP_LSE_TWICE = 1, 2, 4, 8, 16
FD_STEP_CALLER_PARTIALS, FD_STEP_ORDER_FROM_APPEND = 32, 64
# fd_order_kind
FD_ORDER_NONE, FD_ORDER_SEQUENCES, FD_ORDER_ITEMS = 0, 1, 2

EXPORTED_SYMBOLS = ("fd_split_kv", "fd_combine", "fd_decode", "fd_plan_decode", "fd_workspace_bytes", "fd_decode_planned", "fd_decode_noalloc", "fd_schedule", "fd_schedule_items", "fd_plan_splits", "fd_plan_min_splits",
                    "fd_kv_append",
                    "fd_last_error", "fd_abi_version", "fd_build_id")

_DTYPES = {torch.float32: FD_F32, torch.float16: FD_F16, torch.bfloat16: FD_BF16}
if hasattr(torch, "float8_e4m3fn"):
    _DTYPES[torch.float8_e4m3fn] = FD_FP8_E4M3


def fd_dtype_of(t: torch.Tensor, fp8_bytes: bool = False) -> int:
    """fd_dtype enum of a tensor; a uint8 tensor is taken as e4m3fn bit patterns when ``fp8_bytes``."""
    if fp8_bytes and t.dtype == torch.uint8:
        return FD_FP8_E4M3
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise RuntimeError(f"Unsupported data type: {t.dtype}") from None


class FdParams(Structure):
    """Mirror of ``struct fd_params``."""
    _fields_ = [
        ("q_heads", c_int32), ("kv_heads", c_int32), ("head_dim", c_int32), ("page_size", c_int32),
        ("num_splits", c_int32), ("num_pages", c_int32), ("max_pages_per_seq", c_int32),
        ("q_dtype", c_int32), ("kv_dtype", c_int32), ("mid_dtype", c_int32), ("out_dtype", c_int32),
        ("soft_cap", c_float), ("k_scale", c_void_p), ("v_scale", c_void_p),
        ("path", c_int32), ("waves_per_block", c_int32), ("seq_order_lens", c_void_p),
        ("split_align", c_int32),
        ("split_adapt", c_int32),
        ("max_kv_len", c_int32),
        ("seq_order_items", c_int32),
        ("v_head_dim", c_int32),
        ("rank_merge", c_void_p),
    ]


class FdRankMerge(Structure):
    """Mirror of ``struct fd_rank_merge``."""
    _fields_ = [
        ("rank_lens", c_void_p), ("this_rank", c_int32), ("local_dtype", c_int32), ("local_out", c_void_p),
        ("stride_lb", c_int64), ("stride_lh", c_int64),
    ]


class FdLaunchPlan(Structure):
    """Mirror of ``struct fd_launch_plan``."""
    _fields_ = [
        ("num_splits", c_int32), ("split_adapt", c_int32), ("split_align", c_int32), ("mid_dtype", c_int32),
        ("direct", c_int32), ("order_kind", c_int32), ("mfma", c_int32), ("tile", c_int32),
        ("waves_per_head", c_int32), ("members", c_int32), ("chunk", c_int32), ("head_block", c_int32),
        ("grid", c_int32 * 3), ("store_through", c_int32), ("max_kv_len", c_int32), ("reserved", c_int32),
        ("partial_bytes", c_int64), ("lse_bytes", c_int64), ("order_bytes", c_int64), ("workspace_bytes", c_int64),
    ]


class FdDecodeArgs(Structure):
    """Mirror of ``struct fd_decode_args``."""
    _fields_ = [
        ("q", c_void_p), ("k_cache", c_void_p), ("v_cache", c_void_p), ("workspace", c_void_p),
        ("workspace_bytes", c_int64), ("out", c_void_p), ("lse_out", c_void_p), ("block_table", c_void_p),
        ("kv_lens", c_void_p), ("seq_order", c_void_p), ("extra_out", c_void_p), ("extra_lse", c_void_p),
        ("stride_q_bs", c_int64), ("stride_q_h", c_int64), ("stride_k_tok", c_int64), ("stride_k_h", c_int64),
        ("stride_v_tok", c_int64), ("stride_v_h", c_int64), ("stride_table_bs", c_int64), ("stride_obs", c_int64),
        ("stride_oh", c_int64), ("sm_scale", c_float), ("batch", c_int32), ("combine_mode", c_int32),
        ("num_extra", c_int32), ("flags", c_int32), ("params", FdParams),
    ]


class FdQkPrep(Structure):
    """Mirror of ``struct fd_qk_prep``."""
    _fields_ = [
        ("cos_sin", c_void_p), ("stride_cos_sin", c_int64), ("position_ids", c_void_p),
        ("position_dtype", c_int32), ("max_positions", c_int32), ("stride_pos_b", c_int64), ("stride_pos_t", c_int64),
        ("q", c_void_p), ("q_out", c_void_p),
        ("stride_q_b", c_int64), ("stride_q_t", c_int64), ("stride_q_h", c_int64),
        ("stride_qo_b", c_int64), ("stride_qo_t", c_int64), ("stride_qo_h", c_int64),
        ("q_norm_weight", c_void_p), ("k_norm_weight", c_void_p), ("q_norm_eps", c_float), ("k_norm_eps", c_float),
    ]


_lib = None


def load_library(path: str = None) -> ctypes.CDLL:
    """Loads the shared library once and declares the argument types of every entry point.

    ``FD_LIBRARY_PATH`` in the environment names another build of the library (same ABI)."""
    global _lib
    if _lib is not None:
        return _lib
    if path is None:
        path = os.environ.get("FD_LIBRARY_PATH", LIB_PATH)
    if not os.path.exists(path):
        raise RuntimeError(
            f"{LIB_NAME} is not built ({path} missing). Build it with "
            f"`python {os.path.join(PKG_DIR, 'build.py')}`; this package has no fallback path.")
    lib = ctypes.CDLL(path)
    i64 = c_int64
    lib.fd_split_kv.restype = c_int32
    lib.fd_split_kv.argtypes = [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int32,
        i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, c_void_p, POINTER(FdParams)]
    lib.fd_combine.restype = c_int32
    lib.fd_combine.argtypes = [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32,
        i64, i64, i64, i64, i64, c_int32, c_void_p, c_void_p, c_int32, POINTER(FdParams)]
    lib.fd_decode.restype = c_int32
    lib.fd_decode.argtypes = [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p,
        c_int32, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, c_void_p, c_int32, c_void_p, c_void_p,
        c_int32, c_void_p, POINTER(FdParams)]
    lib.fd_plan_decode.restype = c_int32
    lib.fd_plan_decode.argtypes = [POINTER(FdParams), c_int32, c_int32, c_int32, POINTER(FdLaunchPlan)]
    lib.fd_workspace_bytes.restype = c_int64
    lib.fd_workspace_bytes.argtypes = [POINTER(FdParams), c_int32, c_int32, c_int32]
    lib.fd_decode_planned.restype = c_int32
    lib.fd_decode_planned.argtypes = [c_void_p, POINTER(FdDecodeArgs)]
    lib.fd_decode_noalloc.restype = c_int32
    lib.fd_decode_noalloc.argtypes = [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int32,
        i64, i64, i64, i64, i64, i64, i64, i64, i64, c_void_p, c_int32, c_void_p, c_void_p, c_int32, POINTER(FdParams)]
    lib.fd_schedule_items.restype = c_int32
    lib.fd_schedule_items.argtypes = [c_void_p, c_void_p, c_int32, c_void_p, POINTER(FdParams)]
    lib.fd_plan_splits.restype = c_int32
    lib.fd_plan_splits.argtypes = [POINTER(FdParams), c_int32]
    lib.fd_plan_min_splits.restype = c_int32
    lib.fd_plan_min_splits.argtypes = [POINTER(FdParams), c_int32]
    lib.fd_kv_append.restype = c_int32
    lib.fd_kv_append.argtypes = [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32,
        i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, POINTER(FdQkPrep), POINTER(FdParams)]
    lib.fd_schedule.restype = c_int32
    lib.fd_schedule.argtypes = [c_void_p, c_void_p, c_int32, c_void_p]
    lib.fd_last_error.restype = c_char_p
    lib.fd_last_error.argtypes = []
    lib.fd_abi_version.restype = c_int32
    lib.fd_abi_version.argtypes = []
    lib.fd_build_id.restype = c_char_p
    lib.fd_build_id.argtypes = []
    if lib.fd_abi_version() != FD_ABI_VERSION:
        raise RuntimeError(f"{path}: ABI version {lib.fd_abi_version()} != expected {FD_ABI_VERSION}; rebuild")
    _lib = lib
    return lib


def check(status: int) -> None:
    """Raises RuntimeError with the library's message for a non-zero status."""
    if status != 0:
        msg = _lib.fd_last_error().decode("utf-8", "replace") if _lib is not None else ""
        raise RuntimeError(f"flash_decode library error {status}: {msg}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_handle(stream=None, device_index=None) -> int:
    """hipStream_t of ``stream`` (a torch stream) or of the current torch stream of the device."""
    if stream is not None:
        return stream.cuda_stream
    if _raw_stream is not None:   # a direct lookup: torch.cuda.current_stream() costs several microseconds
        return _raw_stream(torch.cuda.current_device() if device_index is None else device_index)
    return torch.cuda.current_stream().cuda_stream
