"""fd_decode_noalloc (partials in the library's static device array) against fd_decode (partials in a caller
workspace), both through the C ABI: the same kernels on the same inputs, so outputs and LSEs must be bit-identical.
Two calls in a row share the static array, the second on a smaller input that leaves most of the first call's
partials in place."""
from ctypes import byref

import pytest
import torch

from helpers import DEV, assert_lse_close, assert_out_close, oracle_decode

pytestmark = pytest.mark.gpu


def _params(fd, g, num_splits, out, split_adapt=0, split_align=0):
    L = fd._lib
    p = L.FdParams()
    p.q_heads, p.kv_heads, p.head_dim = g.q.shape[1], g.k_cache.shape[2], g.q.shape[2]
    p.page_size, p.num_pages, p.max_pages_per_seq = g.k_cache.shape[1], g.k_cache.shape[0], g.block_table.shape[1]
    p.num_splits = num_splits
    p.q_dtype = L.fd_dtype_of(g.q)
    p.kv_dtype = L.fd_dtype_of(g.k_cache, fp8_bytes=g.k_scale is not None)
    p.mid_dtype = L.FD_F32
    p.out_dtype = L.fd_dtype_of(out)
    p.split_align, p.split_adapt = split_align, split_adapt
    if g.k_scale is not None:
        p.k_scale, p.v_scale = g.k_scale.data_ptr(), g.v_scale.data_ptr()
    return p


def _both(fd, wl, num_splits, mode=0, split_adapt=0, split_align=0):
    """(out, lse) of fd_decode_noalloc and of fd_decode on the same inputs; nothing is allocated between the
    set-up and the end of the no-alloc call."""
    L = fd._lib
    lib = fd.load_library()
    g = wl.to(DEV)
    B, Hq, D = g.q.shape
    cols = D + 1 if mode == L.FD_COMBINE_SPLIT_LSE else D
    out_a = torch.zeros(B, Hq, cols, dtype=g.q.dtype, device=DEV)
    out_b = torch.zeros_like(out_a)
    lse_a = torch.zeros(B, Hq, dtype=torch.float32, device=DEV)
    lse_b = torch.zeros_like(lse_a)
    mid = torch.empty(B * Hq * num_splits * (D + 1), dtype=torch.float32, device=DEV)
    p = _params(fd, g, num_splits, out_a, split_adapt, split_align)
    stream = torch.cuda.current_stream().cuda_stream
    lse_arg_a = None if mode == L.FD_COMBINE_SPLIT_LSE else lse_a.data_ptr()
    lse_arg_b = None if mode == L.FD_COMBINE_SPLIT_LSE else lse_b.data_ptr()
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(DEV)["allocation.all.allocated"]
    L.check(lib.fd_decode_noalloc(
        stream, g.q.data_ptr(), g.k_cache.data_ptr(), g.v_cache.data_ptr(), out_a.data_ptr(), lse_arg_a,
        float(g.scale), g.block_table.data_ptr(), g.kv_lens.data_ptr(), B, g.q.stride(0), g.q.stride(1),
        g.k_cache.stride(-3), g.k_cache.stride(-2), g.v_cache.stride(-3), g.v_cache.stride(-2),
        g.block_table.stride(0), out_a.stride(0), out_a.stride(1), None, mode, None, None, 0, byref(p)))
    assert torch.cuda.memory_stats(DEV)["allocation.all.allocated"] == before   # torch's allocator was not touched
    n_o = B * Hq * num_splits * D
    L.check(lib.fd_decode(
        stream, g.q.data_ptr(), g.k_cache.data_ptr(), g.v_cache.data_ptr(), mid.data_ptr(),
        mid.data_ptr() + 4 * n_o, out_b.data_ptr(), lse_arg_b, float(g.scale), g.block_table.data_ptr(),
        g.kv_lens.data_ptr(), B, g.q.stride(0), g.q.stride(1), g.k_cache.stride(-3), g.k_cache.stride(-2),
        g.v_cache.stride(-3), g.v_cache.stride(-2), Hq * num_splits * D, num_splits * D, D, g.block_table.stride(0),
        out_b.stride(0), out_b.stride(1), None, mode, None, None, 0, None, byref(p)))
    torch.cuda.synchronize()
    return (out_a.cpu(), lse_a.cpu()), (out_b.cpu(), lse_b.cpu())


def test_no_alloc_matches_fd_decode_twice_in_a_row(fd):
    # first call: 3 sequences, 8 splits; second call right after it: fewer, shorter sequences and fewer splits
    big = fd.utils.make_paged_workload("noalloc_big", [1320, 2049, 463], 32, 8, 128, 16, torch.bfloat16, 32, seed=41)
    small = fd.utils.make_paged_workload("noalloc_small", [70, 0], 32, 8, 128, 16, torch.bfloat16, 32, seed=42)
    for wl, splits in ((big, 8), (small, 4)):
        (out_a, lse_a), (out_b, lse_b) = _both(fd, wl, splits)
        assert torch.equal(out_a.view(torch.int16), out_b.view(torch.int16))
        assert torch.equal(lse_a.view(torch.int32), lse_b.view(torch.int32))
        ref, ref_lse = oracle_decode(wl)
        assert_out_close(out_a, ref)
        assert_lse_close(lse_a, ref_lse)


def test_no_alloc_other_kernels_and_modes(fd):
    L = fd._lib
    cases = [
        (fd.utils.make_paged_workload("noalloc_fp8", [777, 33, 2048, 5], 64, 8, 128, 16, torch.bfloat16, 32, seed=43,
                                      fp8_kv=True), 16, L.FD_COMBINE_SPLIT, 0, 0),
        # ranges by each sequence's own length, more than 16 splits: empty ranges write nothing
        (fd.utils.make_paged_workload("noalloc_adapt", [1320, 18, 9000], 32, 8, 128, 16, torch.float16, 32, seed=44),
         32, L.FD_COMBINE_SPLIT, 2, 64),
        (fd.utils.make_config(1), 4, L.FD_COMBINE_SPLIT, 0, 0),                      # fp32, VALU kernel
        (fd.utils.make_paged_workload("noalloc_lsecol", [300, 1], 16, 16, 256, 1, torch.float16, 32, seed=45), 4,
         L.FD_COMBINE_SPLIT_LSE, 0, 0),
        (fd.utils.make_paged_workload("noalloc_single", [300, 1], 32, 8, 128, 16, torch.bfloat16, 32, seed=46), 1,
         L.FD_COMBINE_SPLIT, 0, 0),                                                   # one split: no partials at all
    ]
    for wl, splits, mode, adapt, align in cases:
        (out_a, lse_a), (out_b, lse_b) = _both(fd, wl, splits, mode, adapt, align)
        assert torch.equal(out_a.float(), out_b.float()), wl.name
        assert torch.equal(lse_a, lse_b), wl.name
        ref, ref_lse = oracle_decode(wl)
        tol = 2e-4 if wl.q.dtype == torch.float32 else 2e-2
        assert_out_close(out_a[..., :ref.shape[-1]], ref, atol=tol)
        if mode == L.FD_COMBINE_SPLIT:
            assert_lse_close(lse_a, ref_lse, rtol=1e-5 if wl.q.dtype == torch.float32 else 1e-3)


def test_no_alloc_rejects_what_does_not_fit(fd):
    L = fd._lib
    lib = fd.load_library()
    wl = fd.utils.make_paged_workload("noalloc_too_big", [64] * 8, 32, 8, 128, 16, torch.bfloat16, 32, seed=47)
    g = wl.to(DEV)
    B, Hq, D = g.q.shape
    out = torch.zeros(B, Hq, D, dtype=g.q.dtype, device=DEV)
    splits = L.FD_NOALLOC_SCRATCH_BYTES // (B * Hq * (D + 1) * 4) + 1     # one split too many
    p = _params(fd, g, splits, out)
    rc = lib.fd_decode_noalloc(
        torch.cuda.current_stream().cuda_stream, g.q.data_ptr(), g.k_cache.data_ptr(), g.v_cache.data_ptr(),
        out.data_ptr(), None, float(g.scale), g.block_table.data_ptr(), g.kv_lens.data_ptr(), B, g.q.stride(0),
        g.q.stride(1), g.k_cache.stride(-3), g.k_cache.stride(-2), g.v_cache.stride(-3), g.v_cache.stride(-2),
        g.block_table.stride(0), out.stride(0), out.stride(1), None, 0, None, None, 0, byref(p))
    assert rc == -5   # FD_ERR_TOO_LARGE
    assert b"static workspace" in lib.fd_last_error()
    torch.cuda.synchronize()
    assert not out.any()   # nothing was launched
