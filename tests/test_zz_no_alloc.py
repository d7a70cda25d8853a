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
    def no_alloc_call():
        L.check(lib.fd_decode_noalloc(
            stream, g.q.data_ptr(), g.k_cache.data_ptr(), g.v_cache.data_ptr(), out_a.data_ptr(), lse_arg_a,
            float(g.scale), g.block_table.data_ptr(), g.kv_lens.data_ptr(), B, g.q.stride(0), g.q.stride(1),
            g.k_cache.stride(-3), g.k_cache.stride(-2), g.v_cache.stride(-3), g.v_cache.stride(-2),
            g.block_table.stride(0), out_a.stride(0), out_a.stride(1), None, mode, None, None, 0, byref(p)))

    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(DEV)["allocation.all.allocated"]
    no_alloc_call()
    assert torch.cuda.memory_stats(DEV)["allocation.all.allocated"] == before   # torch's allocator was not touched
    # ... and neither was the driver's: the device's free memory does not move over a call.  Checked on a repeat of
    # the call, because the runtime itself sets a kernel up the first time a process launches it (code object, kernel
    # argument pool), which has nothing to do with this entry point.
    torch.cuda.synchronize()
    out_a.zero_()
    lse_a.zero_()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(DEV)[0]
    no_alloc_call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(DEV)[0] == free_before
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


def test_no_alloc_keyword_of_the_python_wrappers(fd):
    """``no_alloc=True``: the wrappers plan the step as usual and keep the partials in the library's static array."""
    cases = [
        fd.utils.make_paged_workload("noalloc_kw_bf16", [1320, 2049, 463, 18], 32, 8, 128, 16, torch.bfloat16, 32, seed=51),
        fd.utils.make_paged_workload("noalloc_kw_fp8", [777, 33, 5000], 64, 8, 128, 16, torch.bfloat16, 32, seed=52,
                                     fp8_kv=True),
        fd.utils.make_paged_workload("noalloc_kw_d256", [300, 1, 900], 16, 8, 256, 1, torch.float16, 32, seed=53),
        fd.utils.make_paged_workload("noalloc_kw_direct", [200] * 70, 32, 8, 128, 16, torch.bfloat16, 32, seed=54),
    ]
    for wl in cases:
        g = wl.to(DEV)
        B, Hq, D = g.q.shape
        kw = dict(k_scale=g.k_scale, v_scale=g.v_scale) if g.k_scale is not None else {}
        ref, ref_lse = oracle_decode(wl)
        # plain wrapper with a separate fp32 LSE
        out = torch.zeros(B, Hq, D, dtype=g.q.dtype, device=DEV)
        lse = torch.zeros(B, Hq, dtype=torch.float32, device=DEV)
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats(DEV)["allocation.all.allocated"]
        same = fd.gqa_fwd_batch_decode(g.q, g.k_cache, g.v_cache, None, [1] * B, g.kv_lens, g.block_table, g.scale,
                                       output_combine=out, kv_split=g.kv_split, lse_out=lse, no_alloc=True, **kw)
        assert torch.cuda.memory_stats(DEV)["allocation.all.allocated"] == before
        torch.cuda.synchronize()
        assert same is out
        assert_out_close(out.cpu(), ref)
        assert_lse_close(lse.cpu(), ref_lse)
        # bit-identical to the same step with the partials in freshly allocated memory
        usual = fd.gqa_fwd_batch_decode(g.q, g.k_cache, g.v_cache, None, [1] * B, g.kv_lens, g.block_table, g.scale,
                                        kv_split=g.kv_split, auto_order=False, **kw)
        torch.cuda.synchronize()
        if fd.kernels.flash_decode.decode_plan(g.q, g.k_cache, g.block_table, g.kv_split, fp8=g.k_scale is not None
                                               ).mid_dtype == fd._lib.FD_F32:
            assert torch.equal(out.cpu().view(torch.int16), usual.cpu().view(torch.int16)), wl.name
        # intra-rank wrapper: merged LSE in the output's last column
        out1 = torch.zeros(B, Hq, D + 1, dtype=g.q.dtype, device=DEV)
        fd.gqa_fwd_batch_decode_intra_rank(g.q, g.k_cache, g.v_cache, None, [1] * B, g.kv_lens, g.block_table, g.scale,
                                           output_combine=out1, kv_split=g.kv_split, no_alloc=True, **kw)
        torch.cuda.synchronize()
        assert_out_close(out1[..., :D].cpu(), ref)
        assert_lse_close(out1[..., D].float().cpu(), ref_lse, rtol=1e-2)   # the column has the output's 16-bit type
    with pytest.raises(RuntimeError, match="output_combine"):
        g = cases[0].to(DEV)
        fd.gqa_fwd_batch_decode(g.q, g.k_cache, g.v_cache, None, None, g.kv_lens, g.block_table, g.scale, no_alloc=True)
    with pytest.raises(RuntimeError, match="output_split"):
        fd.gqa_fwd_batch_decode(g.q, g.k_cache, g.v_cache, None, None, g.kv_lens, g.block_table, g.scale, no_alloc=True,
                                output_combine=torch.empty(4, 32, 128, dtype=torch.bfloat16, device=DEV),
                                output_split=torch.empty(4, 32, 32, 129, dtype=torch.float32, device=DEV))


def test_no_alloc_step_in_a_hip_graph(fd):
    """What the entry point is for: a decode step captured into a HIP graph (no allocation may happen under capture)
    and replayed with other lengths.  One eager call on the device comes first -- it looks up the static array's
    address, which is module set-up and not for a capture -- and every replay is checked against the eager result,
    with the program's own eager work and synchronisations between the replays."""
    L = fd._lib
    lib = fd.load_library()
    wl = fd.utils.make_paged_workload("noalloc_graph", [1320, 2049, 463], 32, 8, 128, 16, torch.bfloat16, 32, seed=61)
    g = wl.to(DEV)
    B, Hq, D = g.q.shape
    S = 8
    out = torch.zeros(B, Hq, D, dtype=g.q.dtype, device=DEV)
    lse = torch.zeros(B, Hq, dtype=torch.float32, device=DEV)
    lens = g.kv_lens.clone()
    p = _params(fd, g, S, out, split_adapt=2, split_align=64)

    def launch(stream):
        L.check(lib.fd_decode_noalloc(
            stream, g.q.data_ptr(), g.k_cache.data_ptr(), g.v_cache.data_ptr(), out.data_ptr(), lse.data_ptr(),
            float(g.scale), g.block_table.data_ptr(), lens.data_ptr(), B, g.q.stride(0), g.q.stride(1),
            g.k_cache.stride(-3), g.k_cache.stride(-2), g.v_cache.stride(-3), g.v_cache.stride(-2),
            g.block_table.stride(0), out.stride(0), out.stride(1), None, 0, None, None, 0, byref(p)))

    def eager(new_lens):
        lens.copy_(torch.tensor(new_lens, dtype=torch.int32))
        launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        res = out.clone(), lse.clone()
        out.zero_()
        lse.zero_()
        return res

    eager(wl.kv_lens.tolist())   # the first call on the device, outside any capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for new_lens in ([1320, 2049, 463], [70, 0, 2049], [2049, 2049, 2049], [1, 17, 33], [1320, 2049, 463]):
        want_out, want_lse = eager(new_lens)          # eager work between the replays
        lens.copy_(torch.tensor(new_lens, dtype=torch.int32))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), want_out.view(torch.int16)), new_lens
        assert torch.equal(lse.view(torch.int32), want_lse.view(torch.int32)), new_lens
        w2 = fd.utils.make_paged_workload("noalloc_graph", [1320, 2049, 463], 32, 8, 128, 16, torch.bfloat16, 32, seed=61)
        w2.kv_lens = torch.tensor(new_lens, dtype=torch.int32)
        ref, ref_lse = oracle_decode(w2)
        assert_out_close(out.cpu(), ref)
        assert_lse_close(lse.cpu(), ref_lse)
        out.zero_()
        lse.zero_()
