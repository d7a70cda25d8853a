"""GPU tests of the sequence-parallel layer, the inter-rank combine and the raw C-ABI entry points.

The layer test follows test_sp_decode_attn.py:135-202: every "rank" holds a shard of the KV
sequence, the oracle runs on the concatenated cache with concatenated, offset block tables, and
the merged result must match at the reference's tolerance (atol 0.05, rtol 1e-2) and at the
north-star gate.  All ranks run on the one GPU; the partials of the other ranks are produced by
the same kernels and handed to the layer as ``remote_partials``.
"""
import ctypes

import pytest
import torch

import oracle
from helpers import DEV, assert_lse_close, assert_out_close

pytestmark = pytest.mark.gpu


def _sp_inputs(R, B, Hq, Hkv, D, P, kv_per_rank, dtype, seed, scale_kv=0.1):
    g = torch.Generator().manual_seed(seed)
    pages = -(-max(max(x) for x in kv_per_rank) // P) + 1
    q = torch.randn(B, Hq, D, generator=g).to(dtype)
    ks = [(torch.randn(pages, P, Hkv, D, generator=g) * scale_kv).to(dtype) for _ in range(R)]
    vs = [(torch.randn(pages, P, Hkv, D, generator=g) * scale_kv).to(dtype) for _ in range(R)]
    bts = [torch.randint(0, pages, (B, pages), generator=g, dtype=torch.int32) for _ in range(R)]
    lens = torch.tensor(kv_per_rank, dtype=torch.int32)          # [R, B]
    return q, ks, vs, bts, lens, pages


def _oracle_concat(q, ks, vs, bts, lens, pages, scale):
    """Oracle on the concatenated cache: rank r's pages are offset by r*pages (test_sp_decode_attn.py:174-186)."""
    R, B = lens.shape
    P = ks[0].shape[1]
    kcat, vcat = torch.cat(ks).float(), torch.cat(vs).float()
    outs, lses = [], []
    for b in range(B):
        entries, total = [], 0
        # the reference concatenates whole tables because every rank is full; with ragged shards the
        # token order inside the softmax does not matter, so gather rank by rank, token by token
        rows = []
        for r in range(R):
            n = int(lens[r, b])
            for t in range(n):
                rows.append((int(bts[r][b, t // P]) + r * pages) * P + t % P)
        rows = torch.tensor(rows, dtype=torch.long)
        k1 = kcat.reshape(-1, *kcat.shape[2:])[rows][:, None]
        v1 = vcat.reshape(-1, *vcat.shape[2:])[rows][:, None]
        n = rows.numel()
        o, L = oracle.ref_paged_attn_lse(q[b:b + 1].float(), k1, v1, [n], torch.arange(max(n, 1), dtype=torch.int32)[None],
                                         scale)
        outs.append(o[0])
        lses.append(L[0])
    return torch.stack(outs), torch.stack(lses)


@pytest.mark.parametrize("R,Hq,Hkv,P,dtype", [(4, 96, 12, 1, torch.float16), (8, 32, 8, 16, torch.bfloat16),
                                              (2, 16, 16, 16, torch.float16)])
def test_sp_layer_matches_oracle_on_concatenated_cache(fd, R, Hq, Hkv, P, dtype):
    B, D = 2, 128
    kv_per_rank = [[1536, 100 + 37 * r] for r in range(R)]
    kv_per_rank[1][1] = 0                               # one rank holds nothing of sequence 1
    q, ks, vs, bts, lens, pages = _sp_inputs(R, B, Hq, Hkv, D, P, kv_per_rank, dtype, seed=R)
    scale = D ** -0.5
    ref, ref_lse = _oracle_concat(q, ks, vs, bts, lens, pages, scale)
    gq, glens = q.to(DEV), lens.to(DEV)
    # every rank's local partial (out, lse), computed by the same kernels
    parts = []
    for r in range(R):
        oc = torch.empty(B, Hq, D + 1, dtype=torch.float32, device=DEV)
        fd.gqa_fwd_batch_decode_intra_rank(gq, ks[r].to(DEV), vs[r].to(DEV), None, [1] * B, glens[r].contiguous(),
                                           bts[r].to(DEV), scale, output_combine=oc, kv_split=32)
        parts.append(oc)
    # both forms of the forward: the other ranks' partials merged where they are (two launches), and the reference's
    # steps one by one through the staged slots
    for rank, staged in ((0, False), (R - 1, False), (0, True), (R - 1, True)):
        layer = fd.SpGQAFlashDecodeAttention(rank, 0, R, 1, Hq, Hkv, D, D, page_size=P, scale=scale, soft_cap=0,
                                             max_allowed_batch=B, stages=3, staged_exchange=staged)
        others = [r for r in range(R) if r != rank]
        r_out = torch.stack([parts[r][..., :D] for r in others]).to(dtype)
        r_lse = torch.stack([parts[r][..., D] for r in others]).contiguous()
        if rank != 1:
            # rank 1 holds nothing of sequence 1: what it sends for that sequence must not be looked at
            r_out[others.index(1), 1] = float("nan")
            r_lse[others.index(1), 1] = float("nan")
        for _ in range(4):                                # the staging ring rotates
            out = layer(gq, ks[rank].to(DEV), vs[rank].to(DEV), glens, bts[rank].to(DEV),
                        remote_partials=(r_out, r_lse))
        torch.cuda.synchronize()
        torch.testing.assert_close(out.float().cpu(), ref, atol=0.05, rtol=1e-2)
        assert_out_close(out, ref)
        # this rank's slot of the staged buffer holds its own merged partial (out, lse): what a push would send
        stage = layer.ag_buffer[(layer.signal_target - 1) % layer.stages][:R * B * Hq * (D + 1) * 4]
        slot = stage.view(torch.float32).view(R, B, Hq, D + 1)[rank].cpu()
        mine = parts[rank].cpu()
        assert_out_close(slot[..., :D], mine[..., :D], atol=1e-5, rel=False)
        assert_lse_close(slot[..., D], mine[..., D], rtol=1e-6)
        layer.finalize()


def test_sp_layer_at_the_reference_settings_200_iterations(fd):
    """The reference's own loop (test_sp_decode_attn.py:158-202): 96 / 12 heads, head_dim 128, page size 1, fp16,
    1536 tokens per rank, K/V ~ N(0,1)/10, fresh seeded inputs in each of 200 iterations, the oracle on the
    concatenated cache, atol 0.05 / rtol 1e-2 -- with the layer at the reference's settings: 32 splits, split
    partials the caller can see, and everything staged in the query's dtype (LSE included, :95-97), over a
    3-stage ring.  All "ranks" run on the one GPU; every rank's partial comes from the same call the layer makes."""
    R, B, Hq, Hkv, D, P, n, dtype = 4, 1, 96, 12, 128, 1, 128 * 12, torch.float16
    pages = n + 1
    scale = D ** -0.5
    rank = 1
    layer = fd.SpGQAFlashDecodeAttention(rank, 0, R, 1, Hq, Hkv, D, D, page_size=P, scale=scale, soft_cap=0,
                                         max_allowed_batch=1, thrink_buffer_threshold=500, stages=3,
                                         partial_dtype=None)
    layer.kv_split = 32
    gen = torch.Generator(device=DEV).manual_seed(2024)
    lens = torch.full((R, B), n, dtype=torch.int32, device=DEV)
    worst = 0.0
    for it in range(200):
        q = torch.randn(B, Hq, D, generator=gen, device=DEV, dtype=torch.float32).to(dtype)
        kv = (torch.randn(R, 2, pages, P, Hkv, D, generator=gen, device=DEV, dtype=torch.float32) / 10).to(dtype)
        bts = torch.randint(0, pages, (R, B, pages), generator=gen, device=DEV, dtype=torch.int32)
        parts = []
        for r in range(R):
            if r == rank:
                continue
            mid = torch.empty(B, Hq, 32, D + 1, dtype=dtype, device=DEV)
            oc = torch.empty(B, Hq, D + 1, dtype=dtype, device=DEV)
            fd.gqa_fwd_batch_decode_intra_rank(q, kv[r, 0], kv[r, 1], None, [1] * B, lens[r], bts[r], scale,
                                               output_split=mid, output_combine=oc, kv_split=32)
            parts.append(oc)
        r_out = torch.stack([p_[..., :D] for p_ in parts])
        r_lse = torch.stack([p_[..., D].float() for p_ in parts])
        output_split = torch.full((B, Hq, 32, D + 1), float("nan"), dtype=dtype, device=DEV)
        out = layer(q, kv[rank, 0], kv[rank, 1], lens, bts[rank], remote_partials=(r_out, r_lse),
                    output_split=output_split)
        torch.cuda.synchronize()
        assert not torch.isnan(output_split).any()        # all 32 partials of every head were written
        kv_c, bts_c = kv.cpu(), bts.cpu()
        ref, _ = _oracle_concat(q.cpu(), [kv_c[r, 0] for r in range(R)], [kv_c[r, 1] for r in range(R)],
                                [bts_c[r] for r in range(R)], lens.cpu(), pages, scale)
        torch.testing.assert_close(out.float().cpu(), ref, atol=0.05, rtol=1e-2)
        worst = max(worst, (out.float().cpu() - ref).abs().max().item())
    assert layer.signal_target == 200
    assert worst < 5e-3, worst      # far inside the reference's tolerance: fp16 partials and LSEs of values ~0.01
    layer.finalize()


def test_sp_layer_single_rank_and_reference_partial_dtype(fd):
    q, ks, vs, bts, lens, pages = _sp_inputs(1, 1, 32, 8, 128, 16, [[777]], torch.bfloat16, seed=9, scale_kv=1.0)
    ref, _ = _oracle_concat(q, ks, vs, bts, lens, pages, 0.09)
    for pdt in (torch.float32, None):                     # None: q.dtype partials, the reference's layout
        layer = fd.SpGQAFlashDecodeAttention(0, 0, 1, 1, 32, 8, 128, 128, page_size=16, scale=0.09,
                                             max_allowed_batch=1, partial_dtype=pdt)
        out = layer(q.to(DEV), ks[0].to(DEV), vs[0].to(DEV), lens.to(DEV), bts[0].to(DEV))
        torch.cuda.synchronize()
        assert_out_close(out, ref)
    with pytest.raises(AssertionError, match="Only support"):
        layer(q.repeat(2, 1, 1).to(DEV), ks[0].to(DEV), vs[0].to(DEV), lens.repeat(1, 2).to(DEV),
              bts[0].repeat(2, 1).to(DEV))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_inter_rank_combine_validity_rule(fd, dtype):
    g = torch.Generator().manual_seed(21)
    R, B, Hq, D = 8, 3, 16, 128
    outs = torch.randn(R, B, Hq, D, generator=g)
    lses = torch.rand(R, B, Hq, generator=g) * 10 + 5
    packed = torch.cat([outs, lses[..., None]], -1).to(dtype)
    lens = torch.randint(0, 3, (R, B), generator=g, dtype=torch.int32)
    lens[:, 2] = 0                                        # nothing valid for sequence 2
    poisoned = packed.clone()
    poisoned[lens == 0] = float("nan")                    # invalid slots may hold anything
    final = torch.empty(B, Hq, D, dtype=dtype, device=DEV)
    lse_out = torch.empty(B, Hq, dtype=torch.float32, device=DEV)
    fd.inter_rank_combine(poisoned.to(DEV), final, lens.to(DEV), lse_out=lse_out)
    torch.cuda.synchronize()
    ref_o, ref_l = oracle.model_combine(packed.float(), "rank", global_kv_lens=lens.tolist())
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert_out_close(final, ref_o, atol=tol)
    assert_lse_close(lse_out, ref_l, rtol=1e-5 if dtype == torch.float32 else 1e-3)
    assert torch.all(final[2] == 0) and torch.all(torch.isneginf(lse_out[2]))
    # the Triton-style launch syntax of the reference call site (sp_flash_decode_layer.py:173-183)
    final2 = torch.empty_like(final)
    g_packed, g_lens = poisoned.to(DEV), lens.to(DEV)
    fd.kernel_inter_rank_gqa_fwd_batch_decode_combine_kv[(B, Hq, 1)](
        g_packed, final2, g_lens, B, Hq, g_packed.stride(1), g_packed.stride(2), g_packed.stride(0),
        final2.stride(0), final2.stride(1), R, 512, D)
    torch.cuda.synchronize()
    assert torch.equal(final, final2)


def test_many_partials_and_extras(fd):
    """More partials than one LDS pass holds (> 1024) and extra partials, through fd_combine."""
    g = torch.Generator().manual_seed(22)
    R, B, Hq, D = 1500, 1, 4, 128
    outs = torch.randn(R, B, Hq, D, generator=g)
    lses = torch.randn(R, B, Hq, generator=g) * 4
    packed = torch.cat([outs, lses[..., None]], -1)
    final = torch.empty(B, Hq, D, dtype=torch.float32, device=DEV)
    lse_out = torch.empty(B, Hq, dtype=torch.float32, device=DEV)
    fd.inter_rank_combine(packed.to(DEV), final, torch.ones(R, B, dtype=torch.int32, device=DEV), lse_out=lse_out)
    torch.cuda.synchronize()
    wts = torch.softmax(lses.double(), 0)
    assert_out_close(final, (wts[..., None] * outs.double()).sum(0).float(), atol=1e-5)
    assert_lse_close(lse_out, torch.logsumexp(lses.double(), 0).float(), rtol=1e-5)


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("rows,R", [((1, 1), 17), ((1, 8), 40), ((1, 8), 256), ((2, 3), 200), ((1, 2), 1100),
                                    ((1, 96), 128), ((4, 64), 33)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_combine_over_every_workgroup_width(fd, D, rows, R, dtype):
    """Few output rows and many partials make the combine kernel split a row over several workgroups (down to 16
    columns each); every width must give the closed form sum_r softmax(lse)_r * out_r, with invalid ranks skipped."""
    B, Hq = rows
    g = torch.Generator().manual_seed(100 * R + D + B)
    outs = torch.randn(R, B, Hq, D, generator=g)
    lses = torch.randn(R, B, Hq, generator=g) * 3 + 7
    packed = torch.cat([outs, lses[..., None]], -1).to(dtype)
    lens = torch.ones(R, B, dtype=torch.int32)
    lens[torch.rand(R, B, generator=g) < 0.2] = 0
    lens[0] = 1
    poisoned = packed.clone()
    poisoned[lens == 0] = float("nan")
    final = torch.empty(B, Hq, D, dtype=dtype, device=DEV)
    lse_out = torch.empty(B, Hq, dtype=torch.float32, device=DEV)
    fd.inter_rank_combine(poisoned.to(DEV), final, lens.to(DEV), lse_out=lse_out)
    torch.cuda.synchronize()
    o64, l64 = packed[..., :D].double(), packed[..., D].double()
    l64 = l64.masked_fill((lens == 0)[:, :, None], float("-inf"))
    wts = torch.softmax(l64, 0)
    ref = (wts[..., None] * o64.masked_fill((lens == 0)[:, :, None, None], 0.0)).sum(0).float()
    f32 = dtype == torch.float32
    assert_out_close(final, ref, atol=1e-5 if f32 else 2e-2)
    assert_lse_close(lse_out, torch.logsumexp(l64, 0).float(), rtol=1e-5 if f32 else 1e-3)


def test_raw_c_abi_split_then_combine(fd):
    """fd_split_kv and fd_combine called directly through ctypes with the reference's packed layouts."""
    lib = fd.load_library()
    L = fd._lib
    wl = fd.utils.make_paged_workload("abi", [300, 45], 32, 8, 128, 16, torch.bfloat16, 8, seed=31)
    gq, gk, gv = wl.q.to(DEV), wl.k_cache.to(DEV), wl.v_cache.to(DEV)
    gbt, glen = wl.block_table.to(DEV), wl.kv_lens.to(DEV)
    B, Hq, D, S = 2, 32, 128, 8
    mid = torch.empty(B, Hq, S, D + 1, dtype=torch.float32, device=DEV)       # [B,Hq,S,Dv+1], LSE packed
    out = torch.empty(B, Hq, D + 1, dtype=torch.bfloat16, device=DEV)          # intra-rank layout
    lse = torch.empty(B, Hq, dtype=torch.float32, device=DEV)
    order = torch.empty(B, dtype=torch.int32, device=DEV)
    p = L.FdParams()
    p.q_heads, p.kv_heads, p.head_dim, p.page_size, p.num_splits = Hq, 8, D, 16, S
    p.num_pages, p.max_pages_per_seq = gk.shape[0], gbt.shape[1]
    p.q_dtype = p.kv_dtype = p.out_dtype = L.FD_BF16
    p.mid_dtype = L.FD_F32
    hs = torch.cuda.current_stream().cuda_stream
    assert lib.fd_schedule(hs, glen.data_ptr(), B, order.data_ptr()) == 0
    rc = lib.fd_split_kv(hs, gq.data_ptr(), gk.data_ptr(), gv.data_ptr(), mid.data_ptr(), None, float(wl.scale),
                         gbt.data_ptr(), glen.data_ptr(), B, gq.stride(0), gq.stride(1), gk.stride(1), gk.stride(2),
                         gv.stride(1), gv.stride(2), mid.stride(0), mid.stride(1), mid.stride(2), gbt.stride(0),
                         order.data_ptr(), ctypes.byref(p))
    assert rc == 0, lib.fd_last_error()
    rc = lib.fd_combine(hs, mid.data_ptr(), None, out.data_ptr(), lse.data_ptr(), glen.data_ptr(), B, Hq, S,
                        mid.stride(0), mid.stride(1), mid.stride(2), out.stride(0), out.stride(1),
                        L.FD_COMBINE_SPLIT_LSE, None, None, 0, ctypes.byref(p))
    assert rc == 0, lib.fd_last_error()
    torch.cuda.synchronize()
    assert order.tolist() == [0, 1]
    ref, ref_lse = oracle.ref_paged_attn_lse(wl.q.float(), wl.k_cache.float(), wl.v_cache.float(), wl.kv_lens.tolist(),
                                             wl.block_table, wl.scale)
    assert_out_close(out[..., :D], ref)
    assert_lse_close(lse, ref_lse)
    assert_lse_close(out[..., D], ref_lse, rtol=1e-2)             # the packed column is bf16
    model = oracle.model_split_kv(wl.q.float(), wl.k_cache.float(), wl.v_cache.float(), wl.kv_lens.tolist(),
                                  wl.block_table, wl.scale, S)
    assert_out_close(mid[..., :D], model[..., :D], atol=5e-3)
    assert_lse_close(mid[..., D], model[..., D])
