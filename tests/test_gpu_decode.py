"""GPU parity tests of the split-KV decode + combine path against the CPU oracle.

Every test calls the HIP kernels through the C ABI (ctypes) via the package's
reference-compatible wrappers and compares with ``oracle.ref_paged_attn_lse`` on
the same seeded inputs.  Tolerances: the reference's own (atol = rtol = 1e-2,
test_decode_attn.py:164) for its fp16 grid; the north-star gate (max-abs <= 2e-2 on
16-bit outputs, <= 1e-3 relative on LSE) everywhere.
"""
import math

import pytest
import torch

import oracle
from helpers import assert_out_rel, DEV, assert_lse_close, assert_out_close, oracle_decode, run_decode

pytestmark = pytest.mark.gpu

NUM_BLOCKS = 4096  # pool pages of the grid tests (the 2^31-offset case has its own test)


def _grid_workload(fd, kv_lens, num_heads, head_size, block_size, dtype, soft_cap, seed=0, num_blocks=NUM_BLOCKS):
    """Inputs built the way test_decode_attn.py:140-156 builds them: N(0,1) q/k/v, block table
    drawn with replacement, entries past ceil(kv_len/page) random as well."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    Hq, Hkv = num_heads
    B = len(kv_lens)
    q = torch.randn(B, Hq, head_size, generator=gen).to(dtype)
    kv = torch.randn(num_blocks + 1, 2, block_size, Hkv, head_size, generator=gen).to(dtype)
    k_cache = kv[:, 0].contiguous()
    v_cache = kv[:, 1].contiguous()
    max_blocks = (max(kv_lens) + block_size - 1) // block_size
    bt = torch.randint(0, num_blocks, (B, max_blocks), generator=gen, dtype=torch.int32)
    return fd.utils.DecodeWorkload(name="grid", q=q, k_cache=k_cache, v_cache=v_cache,
                                   kv_lens=torch.tensor(kv_lens, dtype=torch.int32), block_table=bt,
                                   scale=head_size ** -0.5, kv_split=32, soft_cap=float(soft_cap))


# ---- the reference's own parameter grid (test_decode_attn.py:126-131)
@pytest.mark.parametrize("kv_lens", [[1320, 18, 463], [1, 54, 293, 70]])
@pytest.mark.parametrize("num_heads", [(16, 16), (32, 8), (64, 8), (6, 1)])
@pytest.mark.parametrize("head_size", [128, 256])
@pytest.mark.parametrize("block_size", [1, 16])
@pytest.mark.parametrize("soft_cap", [0, 30, 50])
def test_reference_grid_fp16(fd, kv_lens, num_heads, head_size, block_size, soft_cap):
    wl = _grid_workload(fd, kv_lens, num_heads, head_size, block_size, torch.float16, soft_cap)
    out, lse = run_decode(fd, wl)
    ref, ref_lse = oracle_decode(wl)
    torch.testing.assert_close(out.float(), ref, atol=1e-2, rtol=1e-2)
    assert_out_close(out, ref)
    assert_lse_close(lse, ref_lse)


# ---- head_dim 64 (its own MFMA kernel)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("num_heads", [(32, 8), (64, 8), (6, 1), (16, 16), (28, 4), (32, 1)])
@pytest.mark.parametrize("block_size,soft_cap", [(1, 0), (16, 0), (16, 30), (7, 50)])
def test_head_dim_64(fd, dtype, num_heads, block_size, soft_cap):
    wl = _grid_workload(fd, [1320, 18, 463, 1, 0, 64, 65, 2500], num_heads, 64, block_size, dtype, soft_cap, seed=11)
    out, lse = run_decode(fd, wl)
    ref, ref_lse = oracle_decode(wl)
    assert_out_close(out, ref)
    assert_lse_close(lse, ref_lse)
    # both kernels exist for every shape here: each agrees with the oracle when forced
    out_v, lse_v = run_decode(fd, wl, path="valu")
    assert_out_close(out_v, ref)
    out_m, lse_m = run_decode(fd, wl, path="mfma", waves_per_block=2, plan_splits=False)
    assert_out_close(out_m, ref)
    assert_lse_close(lse_m, ref_lse)


# ---- V head dim != K head dim (flash_decode.py:765-774 takes v_head_dim from the V cache; K_DIM / V_DIM :162-163)
@pytest.mark.parametrize("dims", [(128, 64), (128, 256), (64, 128), (256, 64), (64, 256), (256, 128)])
@pytest.mark.parametrize("dtype,num_heads,block_size,soft_cap", [
    (torch.bfloat16, (32, 8), 16, 0), (torch.float16, (6, 1), 1, 30), (torch.float32, (16, 16), 7, 0),
    (torch.bfloat16, (20, 2), 16, 50)])
def test_v_head_dim_differs_from_k_head_dim(fd, dims, dtype, num_heads, block_size, soft_cap):
    Dk, Dv = dims
    wl = _grid_workload(fd, [1320, 18, 463, 1, 0, 70, 2500], num_heads, Dk, block_size, dtype, soft_cap, seed=Dk + Dv)
    gen = torch.Generator().manual_seed(Dk * 7 + Dv)
    wl.v_cache = torch.randn(*wl.k_cache.shape[:3], Dv, generator=gen).to(dtype)
    ref, ref_lse = oracle_decode(wl)
    assert ref.shape[-1] == Dv
    f32 = dtype == torch.float32
    tol = dict(atol=2e-4 if f32 else 2e-2)
    for kw in (dict(), dict(plan_splits=False), dict(fuse_combine=True), dict(variant="persistent"),
               dict(waves_per_block=2, plan_splits=False)):
        out, lse = run_decode(fd, wl, **kw)
        assert out.shape[-1] == Dv
        assert_out_close(out, ref, **tol)
        assert_lse_close(lse, ref_lse, rtol=1e-5 if f32 else 1e-3)
    # merged LSE at column Dv, and caller-visible partials [B, Hq, S, Dv + 1] against the per-split model
    res, _ = run_decode(fd, wl, variant="intra")
    assert res.shape[-1] == Dv + 1
    assert_out_close(res[..., :Dv], ref, **tol)
    assert_lse_close(res[..., Dv].float(), ref_lse, rtol=1e-5 if f32 else 1e-2)
    B, Hq = wl.q.shape[:2]
    mid = torch.full((B, Hq, 8, Dv + 1), float("nan"), dtype=torch.float32, device=DEV)
    wl.kv_split = 8
    out_v, _ = run_decode(fd, wl, output_split=mid)
    assert_out_close(out_v, ref, **tol)
    model = oracle.model_split_kv(wl.q.float(), wl.k_cache.float(), wl.v_cache.float(), wl.kv_lens.tolist(),
                                  wl.block_table, wl.scale, 8, soft_cap=wl.soft_cap)
    valid = torch.isfinite(model[..., Dv])
    got = mid.cpu()
    assert torch.allclose(got[..., :Dv][valid], model[..., :Dv][valid], atol=2e-5 if f32 else 5e-3)   # (bf16 P on the MFMA path)
    assert torch.allclose(got[..., Dv][valid], model[..., Dv][valid], atol=1e-3, rtol=1e-3)
    if not f32:
        G = num_heads[0] // num_heads[1]
        if Dk == 128 and G <= 16:
            # K head dim 128: the head_dim-128 MFMA kernel with its V side narrowed (64) or split into two members
            # per KV head (256); every launch shape, and the partials against the per-split model as above
            for kw in (dict(), dict(plan_splits=False), dict(waves_per_block=1, plan_splits=False),
                       dict(waves_per_block=4, plan_splits=False), dict(variant="persistent")):
                out_m, lse_m = run_decode(fd, wl, path="mfma", **kw)
                assert_out_close(out_m, ref, **tol)
                assert_lse_close(lse_m, ref_lse, rtol=1e-3)
            mid_m = torch.full((B, Hq, 8, Dv + 1), float("nan"), dtype=torch.float32, device=DEV)
            run_decode(fd, wl, output_split=mid_m, path="mfma")
            got_m = mid_m.cpu()
            assert not torch.isnan(got_m[..., :Dv][valid]).any()
            assert torch.allclose(got_m[..., :Dv][valid], model[..., :Dv][valid], atol=5e-3)
            assert torch.allclose(got_m[..., Dv][valid], model[..., Dv][valid], atol=1e-3, rtol=1e-3)
            with pytest.raises(RuntimeError, match="equal K and V head"):
                run_decode(fd, wl, path="mfma", fuse_combine=True)
        else:   # the other MFMA kernels need equal dims and say so
            with pytest.raises(RuntimeError, match="equal K and V head"):
                run_decode(fd, wl, path="mfma")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("num_heads", [(16, 16), (8, 4), (32, 8), (64, 8), (6, 1), (32, 2), (3, 1), (20, 1), (48, 2),
                                       (33, 1)])
@pytest.mark.parametrize("block_size", [1, 16, 7])
def test_other_dtypes_and_groups(fd, dtype, num_heads, block_size):
    wl = _grid_workload(fd, [1320, 18, 463, 1, 70], num_heads, 128, block_size, dtype, 0, seed=3)
    out, lse = run_decode(fd, wl)
    ref, ref_lse = oracle_decode(wl)
    assert_out_close(out, ref, atol=2e-2 if dtype != torch.float32 else 2e-4)
    assert_lse_close(lse, ref_lse, rtol=1e-3 if dtype != torch.float32 else 1e-5)


# ---- groups above 16 query heads: two 16-head blocks per wave (head_dim 128, 16-bit cache), further blocks as
# sibling waves; the last block may be partly or wholly padding
@pytest.mark.parametrize("dtype,soft_cap,fp8", [(torch.bfloat16, 0, False), (torch.float16, 30, False),
                                                (torch.bfloat16, 0, True), (torch.float16, 50, True)])
@pytest.mark.parametrize("num_heads", [(32, 1), (64, 2), (17, 1), (48, 1), (64, 1), (80, 1), (132, 1)])
@pytest.mark.parametrize("waves,fuse,plan", [(0, False, True), (1, False, False), (2, True, False), (4, False, False),
                                             (8, True, True)])
def test_two_head_blocks_per_wave(fd, dtype, soft_cap, fp8, num_heads, waves, fuse, plan):
    if fp8:
        wl = fd.utils.make_paged_workload("two_blocks_fp8", [1320, 18, 463, 2049, 33, 0, 1], num_heads[0], num_heads[1],
                                          128, 16, dtype, 32, seed=17, soft_cap=float(soft_cap), fp8_kv=True)
    else:
        wl = _grid_workload(fd, [1320, 18, 463, 2049, 33, 0, 1], num_heads, 128, 16, dtype, soft_cap, seed=17)
    out, lse = run_decode(fd, wl, path="mfma", waves_per_block=waves, fuse_combine=fuse, plan_splits=plan)
    ref, ref_lse = oracle_decode(wl)
    assert_out_close(out, ref)
    assert_lse_close(lse, ref_lse)


@pytest.mark.parametrize("path", ["valu", "mfma"])
@pytest.mark.parametrize("waves", [1, 2, 4, 8])
@pytest.mark.parametrize("fuse", [True, False])
def test_paths_and_waves_agree(fd, path, waves, fuse):
    wl = _grid_workload(fd, [1320, 18, 463, 2049, 33], (32, 8), 128, 16, torch.bfloat16, 0, seed=5)
    out, lse = run_decode(fd, wl, path=path, waves_per_block=waves, fuse_combine=fuse)
    ref, ref_lse = oracle_decode(wl)
    assert_out_close(out, ref)
    assert_lse_close(lse, ref_lse)


# ---- AOT (explicit stream) and persistent variants (test_decode_attn.py:168-251)
@pytest.mark.parametrize("kv_len", [32, 1320, 18, 463, 1, 54, 293, 70])
def test_aot_variant(fd, kv_len):
    wl = _grid_workload(fd, [kv_len], (96, 12), 128, 1, torch.float16, 0, seed=kv_len).to(DEV)
    stream = torch.cuda.current_stream()
    for _ in range(10):
        out = fd.gqa_fwd_batch_decode_aot(stream, wl.q, wl.k_cache, wl.v_cache, None, [1], wl.kv_lens,
                                          wl.block_table, wl.scale, 0)
    torch.cuda.synchronize()
    ref, _ = oracle_decode(wl.to("cpu"))
    torch.testing.assert_close(out.float().cpu(), ref, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("kv_len", [1320, 18, 463, 1, 54, 293, 70])
def test_persistent_variant(fd, kv_len):
    wl = _grid_workload(fd, [kv_len], (64, 8), 128, 1, torch.float16, 0, seed=kv_len + 7)
    out, lse = run_decode(fd, wl, variant="persistent")
    ref, ref_lse = oracle_decode(wl)
    torch.testing.assert_close(out.float(), ref, atol=1e-2, rtol=1e-2)
    assert_lse_close(lse, ref_lse)


def test_persistent_matches_plain_on_ragged_batch(fd):
    wl = _grid_workload(fd, [70, 4000, 1, 900, 2500, 17], (32, 8), 128, 16, torch.bfloat16, 0, seed=11)
    out_p, lse_p = run_decode(fd, wl, variant="persistent")
    out, lse = run_decode(fd, wl)
    assert torch.equal(out_p, out) and torch.equal(lse_p, lse)  # issue order must not change results


def test_fused_combine_leaves_tickets_clean_and_repeats(fd):
    """The fused combine's ticket counters must be back at zero after every launch: ten calls in a
    row on changing inputs all have to match the two-launch path."""
    for i in range(10):
        wl = _grid_workload(fd, [1320 - 97 * i, 18 + i, 463, 5 * i], (32, 8), 128, 16, torch.bfloat16, 0, seed=100 + i)
        out_f, lse_f = run_decode(fd, wl, fuse_combine=True)
        out_u, lse_u = run_decode(fd, wl, fuse_combine=False)
        assert_out_close(out_f, out_u.float(), atol=1e-2)
        assert_lse_close(lse_f, lse_u, rtol=1e-5)
    fk = __import__("importlib").import_module("triton-distributed_amd.kernels.flash_decode")
    for t in fk._TICKETS.values():
        assert int(t.abs().sum().item()) == 0


# ---- the benchmark configurations
@pytest.mark.parametrize("fuse", [True, False])
@pytest.mark.parametrize("idx,scale_down", [(1, 1), (2, 8), (3, 16), (4, 8), (5, 16)])
def test_configs_scaled(fd, idx, scale_down, fuse):
    wl = fd.utils.make_config(idx, scale_down=scale_down)
    kw = {"fuse_combine": fuse}
    if wl.extra_out is not None:
        kw["extra_partials"] = (wl.extra_out.to(DEV), wl.extra_lse.to(DEV))
    out, lse = run_decode(fd, wl, **kw)
    ref, ref_lse = oracle_decode(wl)
    if wl.extra_out is not None:
        ref, ref_lse = _merge_extra(ref, ref_lse, wl.extra_out, wl.extra_lse)
    fp32 = wl.q.dtype == torch.float32
    assert_out_close(out, ref, atol=2e-4 if fp32 else 2e-2)
    assert_out_rel(out, ref, rms_rtol=1e-5 if fp32 else 1e-2, max_rtol=1e-4 if fp32 else 2e-2)
    assert_lse_close(lse, ref_lse, rtol=1e-5 if fp32 else 1e-3)


def _merge_extra(out, lse, extra_out, extra_lse):
    """Closed form of the LSE merge: sum_r softmax(lse)_r * out_r, logsumexp(lse)."""
    all_o = torch.cat([out[None].double(), extra_out.double()], 0)
    all_l = torch.cat([lse[None].double(), extra_lse.double()], 0)
    w = torch.softmax(all_l, dim=0)
    return (w[..., None] * all_o).sum(0).float(), torch.logsumexp(all_l, 0).float()


def test_config2_full_size(fd):
    wl = fd.utils.make_config(2)
    assert wl.algorithmic_bytes() == 268_583_968
    out, lse = run_decode(fd, wl)
    ref, ref_lse = oracle_decode(wl)
    assert_out_close(out, ref)
    assert_out_rel(out, ref)
    assert_lse_close(lse, ref_lse)
    # the scale-aware gate has the power the absolute one lacks at this size: an output off by a factor (a halved V
    # scale, a dropped split) passes max-abs <= 2e-2 because the values themselves are that small, and must fail here
    assert_out_close(out.float() * 0.8, ref, rel=False)
    with pytest.raises(AssertionError):
        assert_out_rel(out.float() * 0.8, ref)
    with pytest.raises(AssertionError):
        assert_out_rel(out.float() * 0.5, ref)
    with pytest.raises(AssertionError):
        assert_out_rel(out.float() * 1.05, ref)
    # size-independent property: the result does not depend on the number of splits
    wl.kv_split = 8
    out8, lse8 = run_decode(fd, wl)
    assert_out_close(out8, out.float(), atol=1e-2)
    assert_out_rel(out8, ref)
    assert_lse_close(lse8, lse, rtol=1e-5)
    # exactly the 32 splits the configuration names (one workgroup walks several of them, 16-bit partials), and
    # with caller-visible partials in the reference's layout
    wl.kv_split = 32
    out32, lse32 = run_decode(fd, wl, plan_splits=False)
    assert_out_close(out32, ref)
    assert_out_rel(out32, ref)
    assert_lse_close(lse32, ref_lse)
    mid = torch.empty(8, 32, 32, 129, dtype=torch.float32, device=DEV)
    out_v, lse_v = run_decode(fd, wl, output_split=mid)
    assert_out_rel(out_v, ref)
    assert_lse_close(lse_v, ref_lse)


def test_config3_full_size_with_extra_partials(fd):
    wl = fd.utils.make_config(3)
    assert wl.algorithmic_bytes() == 536_978_436
    out, lse = run_decode(fd, wl, extra_partials=(wl.extra_out.to(DEV), wl.extra_lse.to(DEV)))
    ref_local, ref_lse_local = oracle_decode(wl)
    ref, ref_lse = _merge_extra(ref_local, ref_lse_local, wl.extra_out, wl.extra_lse)
    assert_out_close(out, ref)
    assert_out_rel(out, ref)
    assert_lse_close(lse, ref_lse)
    # the shard alone (the seven N(0,1) partials dominate the merged values): sharp on the decode itself
    out_l, lse_l = run_decode(fd, wl)
    assert_out_rel(out_l, ref_local)
    assert_lse_close(lse_l, ref_lse_local)


def _check_every_sequence(wl, out, lse):
    """The oracle on every sequence of a large batch, one at a time so that its fp32 copies stay small."""
    for b in range(wl.q.shape[0]):
        ref, ref_lse = oracle_decode(wl, rows=[b])
        assert_out_close(out[b:b + 1], ref)
        assert_out_rel(out[b:b + 1], ref)
        assert_lse_close(lse[b:b + 1], ref_lse)


def test_config4_full_size_every_sequence(fd):
    wl = fd.utils.make_config(4)
    out, lse = run_decode(fd, wl, variant="persistent")
    _check_every_sequence(wl, out, lse)
    out2, lse2 = run_decode(fd, wl)   # unscheduled launch: identical bits
    assert torch.equal(out, out2) and torch.equal(lse, lse2)


def test_config5_full_size_every_sequence(fd):
    wl = fd.utils.make_config(5)
    out, lse = run_decode(fd, wl)
    _check_every_sequence(wl, out, lse)
    # exactly 64 splits (chunked work items, 16-bit partials written through): same values within output rounding
    out64, lse64 = run_decode(fd, wl, plan_splits=False)
    assert_out_rel(out64, out.float(), rms_rtol=5e-3, max_rtol=1e-2)
    assert_lse_close(lse64, lse, rtol=1e-5)
    # the reference's own partial buffers, [B, Hq, 64, D + 1] in the query's dtype (flash_decode.py:763-766) and in
    # fp32: rows that start on odd element offsets, large enough (34 / 68 MB) to be written through
    B, Hq, D = wl.q.shape
    for mdt in (wl.q.dtype, torch.float32):
        mid = torch.full((B, Hq, 64, D + 1), float("nan"), dtype=mdt, device=DEV)
        outv, lsev = run_decode(fd, wl, output_split=mid)
        assert not torch.isnan(mid).any(), "a partial slot was not written"
        # a bf16 row holds its LSE in bf16 as well (8 bits of mantissa on a value near 10): the weights of the merge
        # carry that rounding, which the layout fixes, not the kernel
        loose = mdt != torch.float32
        assert_out_rel(outv, out.float(), rms_rtol=2e-2 if loose else 5e-3, max_rtol=5e-2 if loose else 1e-2)
        assert_lse_close(lsev, lse, rtol=1e-2 if loose else 1e-5)


# ---- edge cases
def test_empty_and_short_sequences(fd):
    """kv_len 0 (defined: out 0, lse -inf), kv_len < S (empty splits), kv_len == 1."""
    wl = _grid_workload(fd, [0, 1, 5, 31, 32, 33, 64, 100], (32, 8), 128, 16, torch.bfloat16, 0, seed=21)
    for variant in ("plain", "persistent"):
        out, lse = run_decode(fd, wl, variant=variant)
        ref, ref_lse = oracle_decode(wl)
        assert torch.all(out[0] == 0) and torch.all(torch.isneginf(lse[0]))
        assert_out_close(out, ref)
        assert_lse_close(lse, ref_lse)


def test_poisoned_pool_and_garbage_table(fd):
    """Unreferenced pages hold NaN and table entries past ceil(kv_len/P) are out of range:
    neither may influence the result (the reference leaves such entries random, test_decode_attn.py:156)."""
    wl = _grid_workload(fd, [100, 37, 513], (32, 8), 128, 16, torch.bfloat16, 0, seed=23, num_blocks=256)
    ref, ref_lse = oracle_decode(wl)
    used = set()
    for b, n in enumerate(wl.kv_lens.tolist()):
        npg = -(-n // 16)
        used.update(wl.block_table[b, :npg].tolist())
        wl.block_table[b, npg:] = 2 ** 30  # far outside the pool
    poison = torch.ones(wl.k_cache.shape[0], dtype=torch.bool)
    poison[list(used)] = False
    wl.k_cache[poison] = float("nan")
    wl.v_cache[poison] = float("nan")
    # the unused tail of the last page of every sequence is poisoned as well
    for b, n in enumerate(wl.kv_lens.tolist()):
        if n % 16:
            page = int(wl.block_table[b, n // 16])
            if sum(1 for bb, nn in enumerate(wl.kv_lens.tolist())
                   if page in wl.block_table[bb, :-(-nn // 16)].tolist()) == 1:
                wl.k_cache[page, n % 16:] = float("nan")
                wl.v_cache[page, n % 16:] = float("nan")
    for path in ("mfma", "valu"):
        out, lse = run_decode(fd, wl, path=path)
        assert_out_close(out, ref)
        assert_lse_close(lse, ref_lse)


def test_block_table_indexing_is_bit_exact(fd):
    """Permuting the pool pages together with the table, and duplicating pages, leaves the output bits unchanged."""
    wl = _grid_workload(fd, [777, 130], (32, 8), 128, 16, torch.bfloat16, 0, seed=25, num_blocks=128)
    out, lse = run_decode(fd, wl)
    gen = torch.Generator(device="cpu").manual_seed(99)
    perm = torch.randperm(wl.k_cache.shape[0], generator=gen)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(perm.numel())
    wl2 = fd.utils.DecodeWorkload(**{**wl.__dict__})
    wl2.k_cache = wl.k_cache[perm].contiguous()
    wl2.v_cache = wl.v_cache[perm].contiguous()
    wl2.block_table = inv[wl.block_table.long()].to(torch.int32)
    out2, lse2 = run_decode(fd, wl2)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)


def test_offsets_beyond_2_31_bytes(fd):
    """A pool whose byte offsets exceed 2^31 (the reference computes them in int32, flash_decode.py:205-206)."""
    Hkv, D, P = 8, 128, 16
    pages = (2 ** 31) // (P * Hkv * D * 2) + 600       # > 2 GiB per cache
    gen = torch.Generator(device="cpu").manual_seed(31)
    k_cache = torch.empty(pages, P, Hkv, D, dtype=torch.bfloat16, device=DEV).normal_()
    v_cache = torch.empty(pages, P, Hkv, D, dtype=torch.bfloat16, device=DEV).normal_()
    kv_lens = [300, 129]
    maxp = -(-max(kv_lens) // P)
    bt = torch.randint(pages - 500, pages, (2, maxp), generator=gen, dtype=torch.int32)  # all in the high region
    q = torch.randn(2, 32, D, generator=gen).to(torch.bfloat16)
    lse = torch.empty(2, 32, dtype=torch.float32, device=DEV)
    out = fd.gqa_fwd_batch_decode(q.to(DEV), k_cache, v_cache, None, [1, 1],
                                  torch.tensor(kv_lens, dtype=torch.int32, device=DEV), bt.to(DEV), D ** -0.5,
                                  lse_out=lse)
    torch.cuda.synchronize()
    # oracle on the referenced pages only, with the table remapped into the compact copy
    used = torch.unique(bt.long())
    remap = torch.zeros(pages, dtype=torch.long)
    remap[used] = torch.arange(used.numel())
    kc = k_cache[used.to(DEV)].cpu().float()
    vc = v_cache[used.to(DEV)].cpu().float()
    ref, ref_lse = oracle.ref_paged_attn_lse(q.float(), kc, vc, kv_lens, remap[bt.long()].to(torch.int32), D ** -0.5)
    assert_out_close(out, ref)
    assert_lse_close(lse, ref_lse)


def test_strided_inputs(fd):
    """K and V as head-slices of one fused [pages, P, 2*Hkv, D] tensor and q as a slice of a wider
    tensor: token / head / batch strides are honoured, nothing is copied."""
    gen = torch.Generator(device="cpu").manual_seed(41)
    fused = torch.randn(300, 16, 16, 128, generator=gen).to(torch.bfloat16)
    qw = torch.randn(3, 32, 256, generator=gen).to(torch.bfloat16)
    kv_lens = [500, 16, 1000]
    bt = torch.randint(0, 300, (3, 63), generator=gen, dtype=torch.int32)
    g_fused, g_q = fused.to(DEV), qw.to(DEV)
    k, v = g_fused[:, :, :8], g_fused[:, :, 8:]
    assert not k.is_contiguous() and not v.is_contiguous()
    lse = torch.empty(3, 32, dtype=torch.float32, device=DEV)
    out = fd.gqa_fwd_batch_decode(g_q[:, :, 128:], k, v, None, [1] * 3,
                                  torch.tensor(kv_lens, dtype=torch.int32, device=DEV), bt.to(DEV), 128 ** -0.5,
                                  lse_out=lse)
    torch.cuda.synchronize()
    ref, ref_lse = oracle.ref_paged_attn_lse(qw[:, :, 128:].float(), fused[:, :, :8].float(), fused[:, :, 8:].float(),
                                             kv_lens, bt, 128 ** -0.5)
    assert_out_close(out, ref)
    assert_lse_close(lse, ref_lse)


@pytest.mark.parametrize("layout", ["fused_kv", "padded_heads"])
def test_strided_fp8_head_dim_64(fd, layout):
    """fp8 caches of 64-byte rows as views: K and V as head-slices of one fused tensor (rows of two adjacent KV heads
    still side by side: a wave may serve both), and as the first 64 bytes of 128-byte head slots (they are not)."""
    gen = torch.Generator(device="cpu").manual_seed(43)
    Hkv, G, D = 4, 6, 64
    raw = torch.randint(0, 256, (200, 16, 2 * Hkv, 2 * D), generator=gen, dtype=torch.uint8)
    raw[(raw & 0x7f) == 0x7f] = 0x11          # no NaN patterns
    raw[(raw & 0x78) == 0x78] &= 0xb7         # keep magnitudes moderate
    if layout == "fused_kv":
        big = raw[..., :D].contiguous()                      # [pages, P, 2*Hkv, 64]
        k, v = big[:, :, :Hkv], big[:, :, Hkv:]
    else:
        k, v = raw[:, :, :Hkv, :D], raw[:, :, Hkv:, :D]      # head stride 128
    assert not k.is_contiguous() and k.stride(-2) == (D if layout == "fused_kv" else 2 * D)
    q = torch.randn(3, Hkv * G, D, generator=gen).to(torch.float16)
    kv_lens = [700, 1, 2049]
    bt = torch.randint(0, 200, (3, 129), generator=gen, dtype=torch.int32)
    k_scale = torch.tensor([0.02, 0.01, 0.03, 0.015])
    v_scale = torch.tensor([0.5, 1.0, 0.25, 2.0])
    tab = torch.from_numpy(oracle.fp8_e4m3fn_decode_table())
    ref, ref_lse = oracle.ref_paged_attn_lse(q.float(), tab[k.long()] * k_scale[None, None, :, None],
                                             tab[v.long()] * v_scale[None, None, :, None], kv_lens, bt, D ** -0.5)
    if layout == "fused_kv":
        gbig = big.to(DEV)
        gk, gv = gbig[:, :, :Hkv], gbig[:, :, Hkv:]
    else:
        graw = raw.to(DEV)
        gk, gv = graw[:, :, :Hkv, :D], graw[:, :, Hkv:, :D]
    for path in ("auto", "valu"):
        lse = torch.empty(3, Hkv * G, dtype=torch.float32, device=DEV)
        out = fd.gqa_fwd_batch_decode(q.to(DEV), gk, gv, None, [1] * 3, torch.tensor(kv_lens, dtype=torch.int32, device=DEV),
                                      bt.to(DEV), D ** -0.5, lse_out=lse, k_scale=k_scale.to(DEV), v_scale=v_scale.to(DEV),
                                      path=path)
        torch.cuda.synchronize()
        assert_out_close(out.cpu(), ref)
        assert_lse_close(lse.cpu(), ref_lse)


@pytest.mark.parametrize("D,dtype", [(128, torch.bfloat16), (64, torch.float16), (256, torch.bfloat16)])
@pytest.mark.parametrize("shape", ["ramp", "steps", "falling"])
def test_scores_that_keep_growing(fd, D, dtype, shape):
    """The kernels rescale their accumulators only when the running maximum has grown by more than 2^8 since the last
    rescale.  Scores that creep up by a fraction of that per tile (ramp), jump far beyond it (steps) or only fall
    must all give the oracle's output and LSE."""
    gen = torch.Generator(device="cpu").manual_seed(77)
    Hq, Hkv, P, n = 8, 2, 16, 3000
    pages = -(-n // P)
    pos = torch.arange(pages * P, dtype=torch.float32)
    level = {"ramp": pos / n * 60.0, "steps": (pos // 700) * 25.0, "falling": (n - pos) / n * 60.0}[shape]
    # q = 1/sqrt(D) in every dim and k[token] = level / sqrt(D) + noise: score = scale * (level + noise . q)
    q = torch.full((1, Hq, D), D ** -0.5).to(dtype)
    k = (level.view(pages, P, 1, 1) * D ** -0.5 + 0.05 * torch.randn(pages, P, Hkv, D, generator=gen)).to(dtype)
    v = torch.randn(pages, P, Hkv, D, generator=gen).to(dtype)
    bt = torch.arange(pages, dtype=torch.int32).view(1, pages)
    ref, ref_lse = oracle.ref_paged_attn_lse(q.float(), k.float(), v.float(), [n], bt, 1.0)
    for kv_split in (1, 4, -1):
        lse = torch.empty(1, Hq, dtype=torch.float32, device=DEV)
        out = fd.gqa_fwd_batch_decode(q.to(DEV), k.to(DEV), v.to(DEV), None, [1], torch.tensor([n], dtype=torch.int32, device=DEV),
                                      bt.to(DEV), 1.0, kv_split=kv_split, lse_out=lse)
        torch.cuda.synchronize()
        assert_out_close(out.cpu(), ref)
        assert_lse_close(lse.cpu(), ref_lse)


# ---- caller-supplied partial buffers in the reference layout [B, Hq, S, Dv+1]
@pytest.mark.parametrize("mid_dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("num_heads", [(32, 8), (4, 4)])
def test_output_split_layout(fd, mid_dtype, num_heads):
    wl = _grid_workload(fd, [1320, 18, 463], num_heads, 128, 16, torch.float16, 0, seed=51)
    g = wl.to(DEV)
    B, Hq, D = g.q.shape
    S = 16
    mid = torch.full((B, Hq, S, D + 1), 7.0, dtype=mid_dtype, device=DEV)
    outc = torch.empty(B, Hq, D, dtype=torch.float16, device=DEV)
    ret = fd.gqa_fwd_batch_decode(g.q, g.k_cache, g.v_cache, None, [1] * B, g.kv_lens, g.block_table, g.scale, 0.0,
                                  output_split=mid, output_combine=outc, kv_split=S)
    torch.cuda.synchronize()
    assert ret is outc                                   # the same object is returned (flash_decode.py:844)
    model = oracle.model_split_kv(wl.q.float(), wl.k_cache.float(), wl.v_cache.float(), wl.kv_lens.tolist(),
                                  wl.block_table, wl.scale, S)
    got = mid.float().cpu()
    loose = mid_dtype != torch.float32
    # empty splits: out 0, lse -inf; others match the per-split model
    assert torch.equal(torch.isneginf(got[..., D]), torch.isneginf(model[..., D]))
    fin = ~torch.isneginf(model[..., D])
    assert_out_close(got[..., :D][fin], model[..., :D][fin], atol=2e-2 if loose else 5e-3)
    assert_lse_close(got[..., D][fin], model[..., D][fin], rtol=1e-2 if loose else 1e-3)
    assert torch.all(got[..., :D][~fin] == 0)
    ref, _ = oracle_decode(wl)
    assert_out_close(outc, ref)


# ---- exactly the caller's splits on the chunked path (one workgroup walks consecutive splits, every wave stores one
# partial per split): every partial against the per-split model (flash_decode.py:193-239), odd split counts that the
# chunk does not divide, sequences shorter than the split count, empty ones, two head blocks per wave, fp8
@pytest.mark.parametrize("kind", ["bf16", "fp16_g32", "fp8", "bf16_mha", "bf16_d256", "fp16_d64", "fp16_d256_g16"])
@pytest.mark.parametrize("S,mid_dtype", [(32, torch.float32), (24, torch.bfloat16), (7, torch.float16), (64, torch.float32),
                                         (3, torch.float32)])
@pytest.mark.parametrize("soft_cap", [0, 30])
def test_exact_splits_on_chunked_work_items(fd, kind, S, mid_dtype, soft_cap):
    Hq, Hkv, dtype, fp8, D = {"bf16": (32, 8, torch.bfloat16, False, 128), "fp16_g32": (128, 4, torch.float16, False, 128),
                              "fp8": (64, 8, torch.bfloat16, True, 128), "bf16_mha": (8, 8, torch.bfloat16, False, 128),
                              "bf16_d256": (32, 8, torch.bfloat16, False, 256), "fp16_d64": (32, 8, torch.float16, False, 64),
                              "fp16_d256_g16": (64, 4, torch.float16, False, 256)}[kind]
    lens = [4099, 18, 0, 1, 2049, 777, 64, 33]
    wl = fd.utils.make_paged_workload("chunked_" + kind, lens, Hq, Hkv, D, 16, dtype, S, seed=61 + S,
                                      soft_cap=float(soft_cap), fp8_kv=fp8)
    # the launch must actually be chunked for this to test anything: the library's own plan has fewer splits
    L = fd._lib
    from ctypes import byref
    p = L.FdParams()
    p.q_heads, p.kv_heads, p.head_dim, p.page_size, p.num_splits = Hq, Hkv, D, 16, S
    p.num_pages, p.max_pages_per_seq = wl.k_cache.shape[0], wl.block_table.shape[1]
    p.q_dtype, p.kv_dtype = L.fd_dtype_of(wl.q), (L.FD_FP8_E4M3 if fp8 else L.fd_dtype_of(wl.k_cache))
    planned = fd.load_library().fd_plan_splits(byref(p), len(lens))
    g = wl.to(DEV)
    B = len(lens)
    mid = torch.full((B, Hq, S, D + 1), float("nan"), dtype=mid_dtype, device=DEV)
    out, lse = run_decode(fd, wl, output_split=mid)
    kc, vc = wl.k_cache, wl.v_cache
    if fp8:
        kc = oracle.dequant_fp8_cache(kc.view(torch.uint8), wl.k_scale)
        vc = oracle.dequant_fp8_cache(vc.view(torch.uint8), wl.v_scale)
    model = oracle.model_split_kv(wl.q.float(), kc.float(), vc.float(), lens, wl.block_table, wl.scale, S,
                                  soft_cap=wl.soft_cap)
    got = mid.float().cpu()
    assert not torch.isnan(got).any(), "a partial slot was not written"
    assert torch.equal(torch.isneginf(got[..., D]), torch.isneginf(model[..., D]))
    fin = ~torch.isneginf(model[..., D])
    loose = mid_dtype != torch.float32
    # fp32 partials: the probabilities enter P.V rounded to the cache's 16-bit type (flash_decode.py:230), i.e. an error
    # of up to 2^-9 (bf16) / 2^-12 (fp16) of the largest value row, which is about 4.5 for N(0,1) data
    exact_atol = 1e-2 if dtype == torch.bfloat16 else 5e-3
    assert_out_close(got[..., :D][fin], model[..., :D][fin], atol=2e-2 if loose else exact_atol, rel=False)
    assert_lse_close(got[..., D][fin], model[..., D][fin], rtol=1e-2 if loose else 1e-3)
    assert torch.all(got[..., :D][~fin] == 0)
    ref, ref_lse = oracle_decode(wl)
    assert_out_close(out, ref)
    # a 16-bit caller buffer holds the partial LSEs in 16 bits too (the reference's layout, flash_decode.py:239)
    assert_lse_close(lse, ref_lse, rtol=1e-2 if loose else 1e-3)
    # internal partials with exactly S splits (16-bit, separate LSE buffer) and the library's own plan agree
    out_x, lse_x = run_decode(fd, wl, plan_splits=False)
    assert_out_close(out_x, ref)
    assert_lse_close(lse_x, ref_lse)
    if S >= 24:
        assert 0 < planned < S
        fk = __import__("importlib").import_module("triton-distributed_amd.kernels.flash_decode")
        plan = fk.decode_plan(g.q, g.k_cache, g.block_table, S, flags=L.FD_STEP_CALLER_PARTIALS,
                              mid_dtype=L.fd_dtype_of(mid), fp8=fp8)
        if S // planned >= 2 and D == 128:   # (the head_dim 64 / 256 kernels launch one workgroup per split)
            assert plan.launch["chunk"] > 1, plan.launch


# ---- the library's own partial layout on the chunked path: rows [B, Hq, S, D] on multiples of four elements and the
# LSEs in their own fp32 buffer.  A wave then parks finished (normalised, mid-dtype) partials and walks up to four splits;
# every partial against the per-split model, through the C ABI's split entry point
@pytest.mark.parametrize("kind", ["bf16", "fp16_g32", "fp8", "bf16_g8", "fp16_d256", "bf16_d64"])
@pytest.mark.parametrize("S,mid_dtype", [(64, torch.bfloat16), (32, torch.float32), (27, torch.float16), (5, torch.bfloat16)])
def test_exact_splits_internal_layout_every_partial(fd, kind, S, mid_dtype):
    from ctypes import byref
    fk = __import__("importlib").import_module("triton-distributed_amd.kernels.flash_decode")
    Hq, Hkv, dtype, fp8, D = {"bf16": (32, 8, torch.bfloat16, False, 128), "fp16_g32": (128, 4, torch.float16, False, 128),
                              "fp8": (64, 8, torch.bfloat16, True, 128), "bf16_g8": (64, 8, torch.bfloat16, False, 128),
                              "fp16_d256": (32, 8, torch.float16, False, 256), "bf16_d64": (64, 8, torch.bfloat16, False, 64)}[kind]
    lens = [8200, 18, 0, 1, 4097, 777, 64, 2500]
    wl = fd.utils.make_paged_workload("internal_" + kind, lens, Hq, Hkv, D, 16, dtype, S, seed=71 + S, fp8_kv=fp8)
    g = wl.to(DEV)
    B = len(lens)
    L = fd._lib
    lib = fd.load_library()
    p = fk._make_params(g.q, g.k_cache, g.block_table, S, 0.0, L.fd_dtype_of(torch.empty(0, dtype=mid_dtype)),
                        L.fd_dtype_of(g.q), g.k_scale, g.v_scale, "auto", 0)
    mid = torch.full((B, Hq, S, D), float("nan"), dtype=mid_dtype, device=DEV)
    lse = torch.full((B, Hq, S), float("nan"), dtype=torch.float32, device=DEV)
    L.check(lib.fd_split_kv(
        torch.cuda.current_stream().cuda_stream, g.q.data_ptr(), g.k_cache.data_ptr(), g.v_cache.data_ptr(),
        mid.data_ptr(), lse.data_ptr(), float(g.scale), g.block_table.data_ptr(), g.kv_lens.data_ptr(), B,
        g.q.stride(0), g.q.stride(1), g.k_cache.stride(-3), g.k_cache.stride(-2), g.v_cache.stride(-3),
        g.v_cache.stride(-2), mid.stride(0), mid.stride(1), mid.stride(2), g.block_table.stride(0), None, byref(p)))
    torch.cuda.synchronize()
    kc, vc = wl.k_cache, wl.v_cache
    if fp8:
        kc = oracle.dequant_fp8_cache(kc.view(torch.uint8), wl.k_scale)
        vc = oracle.dequant_fp8_cache(vc.view(torch.uint8), wl.v_scale)
    model = oracle.model_split_kv(wl.q.float(), kc.float(), vc.float(), lens, wl.block_table, wl.scale, S)
    got, got_lse = mid.float().cpu(), lse.cpu()
    assert not torch.isnan(got).any() and not torch.isnan(got_lse).any(), "a partial slot was not written"
    assert torch.equal(torch.isneginf(got_lse), torch.isneginf(model[..., D]))
    fin = ~torch.isneginf(model[..., D])
    exact_atol = 1e-2 if dtype == torch.bfloat16 else 5e-3   # P enters P.V rounded to the cache's 16-bit type
    assert_out_close(got[fin], model[..., :D][fin], atol=2e-2 if mid_dtype != torch.float32 else exact_atol, rel=False)
    assert_lse_close(got_lse[fin], model[..., D][fin], rtol=1e-3)
    assert torch.all(got[~fin] == 0)


@pytest.mark.parametrize("mid_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_partial_buffer_one_element_off_alignment(fd, mid_dtype, D):
    """A caller's [B, Hq, S, D + 1] partial buffer that starts one element past an aligned address holds the same bits
    as an aligned one, and the elements on either side of it stay untouched."""
    lens = [700, 0, 45, 2100]
    S = 12
    wl = fd.utils.make_paged_workload("offset_mid", lens, 16, 4, D, 16, torch.bfloat16, S, seed=67)
    B, Hq = len(lens), 16
    n = B * Hq * S * (D + 1)
    flat = torch.full((n + 2,), 7.0, dtype=mid_dtype, device=DEV)
    mid_off = flat[1:n + 1].view(B, Hq, S, D + 1)
    mid = torch.full((B, Hq, S, D + 1), float("nan"), dtype=mid_dtype, device=DEV)
    out_a, lse_a = run_decode(fd, wl, output_split=mid)
    out_b, lse_b = run_decode(fd, wl, output_split=mid_off)
    assert flat[0].item() == 7.0 and flat[n + 1].item() == 7.0
    assert torch.equal(mid.view(torch.uint8 if mid_dtype != torch.float32 else torch.int32),
                       mid_off.contiguous().view(torch.uint8 if mid_dtype != torch.float32 else torch.int32))
    assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)
    ref, ref_lse = oracle_decode(wl)
    assert_out_close(out_a, ref)
    assert_lse_close(lse_a, ref_lse, rtol=1e-3 if mid_dtype == torch.float32 else 1e-2)


def test_intra_rank_packs_lse_column(fd):
    wl = _grid_workload(fd, [1320, 18, 463], (32, 8), 128, 16, torch.bfloat16, 0, seed=53)
    g = wl.to(DEV)
    outc = torch.empty(3, 32, 129, dtype=torch.float32, device=DEV)
    fd.gqa_fwd_batch_decode_intra_rank(g.q, g.k_cache, g.v_cache, None, [1] * 3, g.kv_lens, g.block_table, g.scale,
                                       output_combine=outc)
    torch.cuda.synchronize()
    ref, ref_lse = oracle_decode(wl)
    assert_out_close(outc[..., :128], ref)
    assert_lse_close(outc[..., 128], ref_lse)


# ---- fp8
def test_fp8_dequant_table_through_the_kernel(fd):
    """kv_len == 1 makes out == dequantised V[0]: all 256 byte patterns (NaN patterns excluded)
    must come back as table[byte] * v_scale."""
    tab = torch.from_numpy(oracle.fp8_e4m3fn_decode_table())
    bytes_ = torch.arange(256, dtype=torch.uint8)
    bytes_[0x7f] = 0
    bytes_[0xff] = 0x80
    Hkv, D = 2, 128
    v = torch.zeros(2, 1, Hkv, D, dtype=torch.uint8)
    v[0, 0, 0] = bytes_[:128]
    v[0, 0, 1] = bytes_[128:]
    v[1, 0, 0] = bytes_[128:]
    v[1, 0, 1] = bytes_[:128]
    k = torch.full_like(v, 0x38)  # 1.0
    k_scale = torch.tensor([0.5, 2.0])
    v_scale = torch.tensor([0.25, 3.0])
    q = torch.ones(2, 8, D, dtype=torch.bfloat16)
    bt = torch.tensor([[0], [1]], dtype=torch.int32)
    for path in ("valu", "auto"):
        lse = torch.empty(2, 8, dtype=torch.float32, device=DEV)
        out = fd.gqa_fwd_batch_decode(q.to(DEV), k.to(DEV), v.to(DEV), None, [1, 1],
                                      torch.tensor([1, 1], dtype=torch.int32, device=DEV), bt.to(DEV), 0.125,
                                      output_combine=torch.empty(2, 8, D, dtype=torch.float32, device=DEV),
                                      lse_out=lse, k_scale=k_scale.to(DEV), v_scale=v_scale.to(DEV), path=path)
        torch.cuda.synchronize()
        out = out.cpu()
        for b in range(2):
            for h in range(8):
                kvh = h // 4
                expect = tab[v[b, 0, kvh].long()] * v_scale[kvh]
                assert torch.equal(out[b, h], expect), (path, b, h)
                # one key: lse = scale * q.k = 0.125 * 128 * k_scale
                assert math.isclose(lse[b, h].item(), 0.125 * 128 * k_scale[kvh].item(), rel_tol=1e-6)


@pytest.mark.parametrize("num_heads", [(64, 8), (16, 4), (8, 8)])
@pytest.mark.parametrize("D", [128, 256, 64])
def test_fp8_decode_matches_oracle_on_dequantised_cache(fd, num_heads, D):
    wl = fd.utils.make_paged_workload("fp8", [1000, 17, 4097, 0, 33], num_heads[0], num_heads[1], D, 16, torch.bfloat16,
                                      16, seed=61, fp8_kv=True)
    out, lse = run_decode(fd, wl)
    ref, ref_lse = oracle_decode(wl)
    assert_out_close(out, ref)
    assert_lse_close(lse, ref_lse)
    for path, extra in (("valu", {}), ("mfma", dict(waves_per_block=4, plan_splits=False))):   # force each kernel
        out_p, lse_p = run_decode(fd, wl, path=path, **extra)
        assert_out_close(out_p, ref)
        assert_lse_close(lse_p, ref_lse)


def test_fp8_d64_dequant_table_and_soft_cap(fd):
    """All byte patterns through the head_dim-64 fp8 kernels (kv_len == 1: out == dequantised V[0], exact), and the
    soft cap with a 40-head group over ragged lengths."""
    tab = torch.from_numpy(oracle.fp8_e4m3fn_decode_table())
    bytes_ = torch.arange(256, dtype=torch.uint8)
    bytes_[0x7f] = 0
    bytes_[0xff] = 0x80
    Hkv, D = 4, 64
    v = bytes_.view(1, 1, Hkv, D).clone()
    k = torch.full_like(v, 0x38)  # 1.0
    k_scale = torch.tensor([0.5, 2.0, 1.0, 0.25])
    v_scale = torch.tensor([0.25, 3.0, 1.0, 0.5])
    q = torch.ones(1, 8, D, dtype=torch.float16)
    bt = torch.tensor([[0]], dtype=torch.int32)
    for path in ("valu", "mfma"):
        lse = torch.empty(1, 8, dtype=torch.float32, device=DEV)
        out = fd.gqa_fwd_batch_decode(q.to(DEV), k.to(DEV), v.to(DEV), None, [1],
                                      torch.tensor([1], dtype=torch.int32, device=DEV), bt.to(DEV), 0.125,
                                      output_combine=torch.empty(1, 8, D, dtype=torch.float32, device=DEV),
                                      lse_out=lse, k_scale=k_scale.to(DEV), v_scale=v_scale.to(DEV), path=path)
        torch.cuda.synchronize()
        out = out.cpu()
        for h in range(8):
            kvh = h // 2
            assert torch.equal(out[0, h], tab[v[0, 0, kvh].long()] * v_scale[kvh]), (path, h)
            assert math.isclose(lse[0, h].item(), 0.125 * 64 * k_scale[kvh].item(), rel_tol=1e-6)
    wl = fd.utils.make_paged_workload("fp8_d64_cap", [700, 129, 31, 2050], 80, 2, 64, 1, torch.float16, 32, seed=63,
                                      soft_cap=30.0, fp8_kv=True)
    ref, ref_lse = oracle_decode(wl)
    for kw in (dict(), dict(path="mfma", waves_per_block=8, plan_splits=False), dict(fuse_combine=True)):
        out, lse = run_decode(fd, wl, **kw)
        assert_out_close(out, ref)
        assert_lse_close(lse, ref_lse)


def test_fp8_d256_dequant_table_and_soft_cap(fd):
    """All byte patterns through the head_dim-256 fp8 kernel (kv_len == 1: out == dequantised V[0], exact),
    then a soft-capped, fp16-query run against the oracle."""
    tab = torch.from_numpy(oracle.fp8_e4m3fn_decode_table())
    bytes_ = torch.arange(256, dtype=torch.uint8)
    bytes_[0x7f] = 0
    bytes_[0xff] = 0x80
    v = bytes_.view(1, 1, 1, 256).clone()
    k = torch.full_like(v, 0x38)
    q = torch.ones(1, 4, 256, dtype=torch.bfloat16)
    out = fd.gqa_fwd_batch_decode(q.to(DEV), k.to(DEV), v.to(DEV), None, [1], torch.tensor([1], dtype=torch.int32, device=DEV),
                                  torch.zeros(1, 1, dtype=torch.int32, device=DEV), 0.0625,
                                  output_combine=torch.empty(1, 4, 256, dtype=torch.float32, device=DEV),
                                  k_scale=torch.tensor([0.5], device=DEV), v_scale=torch.tensor([3.0], device=DEV), path="mfma")
    torch.cuda.synchronize()
    for h in range(4):
        assert torch.equal(out[0, h].cpu(), tab[v[0, 0, 0].long()] * 3.0)
    wl = fd.utils.make_paged_workload("fp8_d256_cap", [700, 129, 31], 24, 2, 256, 1, torch.float16, 32, seed=62,
                                      soft_cap=30.0, fp8_kv=True)
    out, lse = run_decode(fd, wl, path="mfma")
    ref, ref_lse = oracle_decode(wl)
    assert_out_close(out, ref)
    assert_lse_close(lse, ref_lse)


# ---- scheduler
def test_schedule_orders_longest_first(fd):
    gen = torch.Generator(device="cpu").manual_seed(71)
    # (2048 lengths go through LDS at a time; 64 lanes share a sequence up to 2048 of them, fewer beyond)
    for B in (1, 2, 3, 64, 300, 1025, 2047, 2048, 2049, 5000, 20000, 65535):
        lens = torch.randint(-3 if B == 300 else 0, 50, (B,), generator=gen, dtype=torch.int32)
        order = fd.schedule_sequences(lens.to(DEV)).cpu()
        expect = torch.argsort(lens, descending=True, stable=True).to(torch.int32)
        assert torch.equal(order, expect)


# ---- error behaviour of the boundary
def test_errors_are_reported_not_fatal(fd):
    wl = _grid_workload(fd, [100], (32, 8), 128, 16, torch.float16, 0).to(DEV)
    with pytest.raises(AssertionError):   # head-dim mismatch: the reference asserts too (flash_decode.py:767)
        fd.gqa_fwd_batch_decode(wl.q[:, :, :64], wl.k_cache, wl.v_cache, None, [1], wl.kv_lens, wl.block_table, 1.0)
    with pytest.raises(RuntimeError, match="MFMA path"):
        fd.gqa_fwd_batch_decode(wl.q.float(), wl.k_cache, wl.v_cache, None, [1], wl.kv_lens, wl.block_table, 1.0,
                                path="mfma")   # an fp32 query cannot take the MFMA path
    with pytest.raises(RuntimeError, match="Unsupported data type"):
        fd.gqa_fwd_batch_decode(wl.q.double(), wl.k_cache, wl.v_cache, None, [1], wl.kv_lens, wl.block_table, 1.0)
    # and the library still works afterwards
    out = fd.gqa_fwd_batch_decode(wl.q, wl.k_cache, wl.v_cache, None, [1], wl.kv_lens, wl.block_table, wl.scale)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()


# ---- HIP graph capture: the whole step (scheduler + split + combine) replays from a graph
@pytest.mark.parametrize("variant", ["plain", "persistent", "persistent_items"])
def test_graph_capture_and_replay(fd, variant):
    wl = _grid_workload(fd, [1320, 463, 2049, 77], (32, 8), 128, 16, torch.bfloat16, 0, seed=81).to(DEV)
    B = 4
    out = torch.empty(B, 32, 128, dtype=torch.bfloat16, device=DEV)
    lse = torch.empty(B, 32, dtype=torch.float32, device=DEV)
    ws = torch.empty(B * 32 * 32 * 129, dtype=torch.float32, device=DEV)
    order = torch.empty(B, dtype=torch.int32, device=DEV)
    fn = fd.gqa_fwd_batch_decode if variant == "plain" else fd.gqa_fwd_batch_decode_persistent

    def step():
        kw = {}   # persistent_items: the wrapper schedules (sequence, range) items itself
        if variant == "persistent":
            fd.schedule_sequences(wl.kv_lens, out=order)
            kw["seq_order"] = order
        fn(wl.q, wl.k_cache, wl.v_cache, ws, [1] * B, wl.kv_lens, wl.block_table, wl.scale, 0.0,
           output_combine=out, kv_split=32, lse_out=lse, **kw)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    gen = torch.Generator(device="cpu").manual_seed(5)
    for it in range(4):
        # new query and new lengths, written in place (the graph holds the addresses)
        wl.q.copy_(torch.randn(wl.q.shape, generator=gen).to(torch.bfloat16))
        wl.kv_lens.copy_(torch.tensor([1320 - 100 * it, 463 + it, 2049 - 500 * it, 77 + 9 * it], dtype=torch.int32))
        graph.replay()
        torch.cuda.synchronize()
        got_out, got_lse = out.clone(), lse.clone()
        out.zero_()
        lse.zero_()
        step()                                   # the program's own eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(got_out, out) and torch.equal(got_lse, lse), f"replay {it} differs from eager"
    ref, ref_lse = oracle_decode(wl.to("cpu"))
    assert_out_close(out, ref)
    assert_lse_close(lse, ref_lse)


# ---- block tables sized for the longest context: the split count follows each sequence's own length
@pytest.mark.parametrize("capacity", [8192, 131072, 1048576])
@pytest.mark.parametrize("kind", ["bf16", "fp16_d256", "fp8", "fp32_valu", "bf16_d64", "g32"])
@pytest.mark.parametrize("batch", [5, 70])
def test_short_sequences_in_a_block_table_sized_for_long_contexts(fd, capacity, kind, batch):
    import random
    rng = random.Random(capacity + batch)
    lens = [rng.choice([0, 1, 37, 64, 1000, 4096, 4097, 5000, 8192]) for _ in range(batch)]
    lens[0], lens[1] = 5000, 0
    Hq, Hkv, D, dtype, fp8 = {"bf16": (32, 8, 128, torch.bfloat16, False), "fp16_d256": (16, 4, 256, torch.float16, False),
                              "fp8": (64, 8, 128, torch.bfloat16, True), "fp32_valu": (8, 4, 128, torch.float32, False),
                              "bf16_d64": (32, 8, 64, torch.bfloat16, False), "g32": (32, 1, 128, torch.bfloat16, False)}[kind]
    P = 16
    wl = fd.utils.make_paged_workload("wide_table", lens, Hq, Hkv, D, P, dtype, -1, seed=29, fp8_kv=fp8)
    # widen the table: entries beyond a sequence's pages are garbage, as in a serving engine's preallocated table
    gen = torch.Generator().manual_seed(3)
    wide = torch.randint(-5, 1 << 30, (batch, capacity // P), generator=gen, dtype=torch.int32)
    for b, n in enumerate(lens):
        used = -(-n // P)
        wide[b, :used] = wl.block_table[b, :used]
    wl.block_table = wide
    ref, ref_lse = oracle_decode(wl)
    f32 = dtype == torch.float32
    for kv_split in (-1, 32, 8):
        wl.kv_split = kv_split
        out, lse = run_decode(fd, wl)
        assert_out_close(out, ref, atol=2e-4 if f32 else 2e-2)
        assert_lse_close(lse, ref_lse, rtol=1e-5 if f32 else 1e-3)
    # a host-side length hint only changes the launch shape: exact, too small (longer sequences are still decoded in
    # full) or beyond the capacity
    wl.kv_split = -1
    for hint in (max(lens), 100, 10 * capacity):
        for variant in ("plain", "persistent"):
            out, lse = run_decode(fd, wl, variant=variant, max_kv_len=hint)
            assert_out_close(out, ref, atol=2e-4 if f32 else 2e-2)
            assert_lse_close(lse, ref_lse, rtol=1e-5 if f32 else 1e-3)
    # the merged LSE column and extra partials go through the same ranges
    res, _ = run_decode(fd, wl, variant="intra")
    assert_out_close(res[..., :D], ref, atol=2e-4 if f32 else 2e-2)
    assert_lse_close(res[..., D].float(), ref_lse, rtol=1e-5 if f32 else 1e-2)


def test_lengths_above_the_table_capacity_are_clamped_alike_by_split_and_combine(fd):
    """kv_lens beyond max_pages * page_size are documented as clamped to the capacity.  With more than 16 splits and
    ranges by each sequence's own length the empty ranges write nothing and the combine derives the valid slots from
    kv_lens: it has to clamp the way the split kernels do, or it would merge slots that nobody wrote."""
    P, cap_pages = 16, 512          # capacity 8192 tokens
    lens_real = [8192, 8192, 3000]
    wl = fd.utils.make_paged_workload("over_capacity", lens_real, 32, 8, 128, P, torch.bfloat16, 32, seed=37)
    assert wl.block_table.shape[1] == cap_pages
    ref, ref_lse = oracle_decode(wl)
    wl.kv_lens = torch.tensor([100000, 8193, 3000], dtype=torch.int32)   # two of them above the capacity
    g = wl.to(DEV)
    B, Hq, D = g.q.shape
    for kv_split, adapt in ((32, 2), (64, 1), (32, 0)):
        lse = torch.empty(B, Hq, dtype=torch.float32, device=DEV)
        out = torch.empty(B, Hq, D, dtype=g.q.dtype, device=DEV)
        # poison the partial workspace: a slot that is read without having been written shows
        ws = torch.full((B * Hq * kv_split * (D + 1),), float("nan"), dtype=torch.float32, device=DEV)
        L = fd._lib
        lib = fd.load_library()
        p = L.FdParams()
        p.q_heads, p.kv_heads, p.head_dim, p.page_size = Hq, 8, D, P
        p.num_splits, p.num_pages, p.max_pages_per_seq = kv_split, g.k_cache.shape[0], cap_pages
        p.q_dtype = p.kv_dtype = p.out_dtype = L.FD_BF16
        p.mid_dtype = L.FD_F32
        p.split_align, p.split_adapt = (64, adapt) if adapt else (0, 0)
        from ctypes import byref
        n_o = B * Hq * kv_split * D
        L.check(lib.fd_decode(
            torch.cuda.current_stream().cuda_stream, g.q.data_ptr(), g.k_cache.data_ptr(), g.v_cache.data_ptr(),
            ws.data_ptr(), ws.data_ptr() + 4 * n_o, out.data_ptr(), lse.data_ptr(), float(g.scale),
            g.block_table.data_ptr(), g.kv_lens.data_ptr(), B, g.q.stride(0), g.q.stride(1), g.k_cache.stride(-3),
            g.k_cache.stride(-2), g.v_cache.stride(-3), g.v_cache.stride(-2), Hq * kv_split * D, kv_split * D, D,
            g.block_table.stride(0), out.stride(0), out.stride(1), None, 0, None, None, 0, None, byref(p)))
        torch.cuda.synchronize()
        assert_out_close(out.cpu(), ref)
        assert_lse_close(lse.cpu(), ref_lse)


# ---- scheduled issue order by (sequence, range) items: the scheduling launch, the append-fused one, the raw ABI
@pytest.mark.parametrize("capacity", [4096, 65536])
@pytest.mark.parametrize("kind", ["bf16", "fp8", "fp32_valu"])
@pytest.mark.parametrize("batch", [3, 40, 300])
def test_item_schedule_matches_oracle_and_is_a_permutation(fd, capacity, kind, batch):
    import random
    from ctypes import byref
    rng = random.Random(7 * capacity + batch)
    lens = [rng.choice([0, 1, 63, 64, 65, 700, 1024, 1025, 2500, 4096]) for _ in range(batch)]
    lens[0] = 4096
    Hq, Hkv, D, dtype, fp8 = {"bf16": (32, 8, 128, torch.bfloat16, False), "fp8": (64, 8, 128, torch.bfloat16, True),
                              "fp32_valu": (8, 4, 128, torch.float32, False)}[kind]
    P = 16
    wl = fd.utils.make_paged_workload("items", lens, Hq, Hkv, D, P, dtype, -1, seed=31, fp8_kv=fp8)
    wide = torch.zeros((batch, capacity // P), dtype=torch.int32)
    wide[:, :wl.block_table.shape[1]] = wl.block_table
    wl.block_table = wide
    ref, ref_lse = oracle_decode(wl)
    f32 = dtype == torch.float32
    out, lse = run_decode(fd, wl, variant="persistent")
    assert_out_close(out, ref, atol=2e-4 if f32 else 2e-2)
    assert_lse_close(lse, ref_lse, rtol=1e-5 if f32 else 1e-3)
    # the raw scheduler: a permutation of all (sequence, range) pairs, non-empty ranges first and largest first
    fk = __import__("importlib").import_module("triton-distributed_amd.kernels.flash_decode")
    g = wl.to(DEV)
    plan = fk.decode_plan(g.q, g.k_cache, g.block_table, -1, fp8=g.k_scale is not None)
    S, adapt, align = plan.num_splits, plan.split_adapt, plan.split_align
    if S == 1 or adapt == 0:
        return
    p = fk._make_params(g.q, g.k_cache, g.block_table, S, 0.0, 0, 0, g.k_scale, g.v_scale, "auto", 0, None,
                        align, adapt)
    items = fk.item_order_buffer(batch, S, DEV)
    fd._lib.check(fd.load_library().fd_schedule_items(None, g.kv_lens.data_ptr(), batch, items.data_ptr(), byref(p)))
    torch.cuda.synchronize()
    it = items.cpu().view(2, batch * S)
    seq, rng_ = (it[0] & 0xFFFF).tolist(), ((it[0] >> 16) & 0xFFFF).tolist()
    assert sorted(zip(seq, rng_)) == [(b, s) for b in range(batch) for s in range(S)]
    assert it[1].tolist() == [lens[b] for b in seq]

    def per(n):   # the library's range rule (include/flash_decode.h, fd_params.split_adapt)
        v = max(-(-n // S), min(-(-n // adapt), min(max(-(-n // 8), 1024), 4096)))
        return -(-v // align) * align
    busy = [per(lens[b]) * s < lens[b] for b, s in zip(seq, rng_)]
    n_busy = sum(busy)
    assert all(busy[:n_busy]) and not any(busy[n_busy:])
    sizes = [per(lens[b]) for b in seq[:n_busy]]
    assert sizes == sorted(sizes, reverse=True)


# ---- single-split steps: the split kernel writes the output itself, no combine launch
@pytest.mark.parametrize("kind", ["bf16", "fp16_d256", "fp8", "fp32_valu", "mha"])
@pytest.mark.parametrize("variant", ["plain", "intra"])
def test_large_batch_single_split_direct_output(fd, kind, variant):
    import random
    rng = random.Random(17)
    B = 160
    lens = [rng.randint(1, 300) for _ in range(B)]
    lens[3] = 0
    lens[77] = 0
    Hq, Hkv, D, dtype, fp8 = {"bf16": (32, 8, 128, torch.bfloat16, False), "fp16_d256": (16, 4, 256, torch.float16, False),
                              "fp8": (64, 8, 128, torch.bfloat16, True), "fp32_valu": (16, 8, 128, torch.float32, False),
                              "mha": (8, 8, 128, torch.bfloat16, False)}[kind]
    wl = fd.utils.make_paged_workload("direct", lens, Hq, Hkv, D, 16, dtype, 32, seed=23, fp8_kv=fp8)
    # the plan for this shape is one split (enough (sequence, KV head) pairs to fill the chip)
    from ctypes import byref
    fk = __import__("importlib").import_module("triton-distributed_amd.kernels.flash_decode")
    g = wl.to(DEV)
    p = fk._make_params(g.q, g.k_cache, g.block_table, 32, 0.0, 0, 0, g.k_scale, g.v_scale, "auto", 0)
    assert fd.load_library().fd_plan_splits(byref(p), B) == 1
    out, lse = run_decode(fd, wl, variant=variant) if variant == "plain" else (None, None)
    ref, ref_lse = oracle_decode(wl)
    atol = 2e-4 if dtype == torch.float32 else 2e-2
    if variant == "plain":
        assert_out_close(out, ref, atol=atol)
        assert_lse_close(lse, ref_lse, rtol=1e-5 if dtype == torch.float32 else 1e-3)
        # without an LSE request nothing is written beyond the [B, Hq, D] rows
        canary = torch.full((B, Hq, D + 8), 7.0, dtype=g.q.dtype, device=DEV)
        kw = dict(k_scale=g.k_scale, v_scale=g.v_scale) if fp8 else {}
        fd.gqa_fwd_batch_decode(g.q, g.k_cache, g.v_cache, None, None, g.kv_lens, g.block_table, g.scale,
                                output_combine=canary[..., :D], kv_split=32, **kw)
        torch.cuda.synchronize()
        assert_out_close(canary[..., :D].cpu(), ref, atol=atol)
        assert (canary[..., D:] == 7.0).all()
    else:
        kw = dict(k_scale=g.k_scale, v_scale=g.v_scale) if fp8 else {}
        res = fd.gqa_fwd_batch_decode_intra_rank(g.q, g.k_cache, g.v_cache, None, None, g.kv_lens, g.block_table, g.scale,
                                                 kv_split=32, **kw)
        torch.cuda.synchronize()
        assert res.shape == (B, Hq, D + 1)
        assert_out_close(res[..., :D].cpu(), ref, atol=atol)
        # the LSE column has the output's dtype
        assert_lse_close(res[..., D].float().cpu(), ref_lse, rtol=1e-5 if dtype == torch.float32 else 1e-2)
    # two launches on the same inputs (exactly one split into a caller buffer, then the combine): same bits, given
    # the same waves per range (the planner's own choice differs between a planned and a literal split count)
    if not fp8:
        two = fd.gqa_fwd_batch_decode(g.q, g.k_cache, g.v_cache, None, None, g.kv_lens, g.block_table, g.scale,
                                      kv_split=1, output_split=torch.empty(B, Hq, 1, D + 1, dtype=torch.float32,
                                                                           device=DEV), waves_per_block=1)
        one = fd.gqa_fwd_batch_decode(g.q, g.k_cache, g.v_cache, None, None, g.kv_lens, g.block_table, g.scale,
                                      kv_split=32, waves_per_block=1)
        torch.cuda.synchronize()
        assert torch.equal(one.cpu().view(torch.uint8), two.cpu().view(torch.uint8))


def test_direct_output_c_abi_rules(fd):
    from ctypes import byref
    lib = fd.load_library()
    fk = __import__("importlib").import_module("triton-distributed_amd.kernels.flash_decode")
    wl = fd.utils.make_paged_workload("direct_abi", [40, 9], 8, 2, 128, 16, torch.bfloat16, 32, seed=5).to(DEV)
    out = torch.empty(2, 8, 128, dtype=torch.bfloat16, device=DEV)
    lse = torch.empty(2, 8, dtype=torch.float32, device=DEV)

    def call(S, mode, lse_ptr, n_extra=0):
        p = fk._make_params(wl.q, wl.k_cache, wl.block_table, S, 0.0, fd._lib.FD_F32, fd._lib.FD_BF16, None, None, "auto", 0)
        return lib.fd_decode(None, wl.q.data_ptr(), wl.k_cache.data_ptr(), wl.v_cache.data_ptr(), None, None,
                             out.data_ptr(), lse_ptr, float(wl.scale), wl.block_table.data_ptr(), wl.kv_lens.data_ptr(), 2,
                             wl.q.stride(0), wl.q.stride(1), wl.k_cache.stride(-3), wl.k_cache.stride(-2),
                             wl.v_cache.stride(-3), wl.v_cache.stride(-2), 0, 0, 0, wl.block_table.stride(0),
                             out.stride(0), out.stride(1), None, mode, out.data_ptr() if n_extra else None,
                             lse.data_ptr() if n_extra else None, n_extra, None, byref(p))

    assert call(2, fd._lib.FD_COMBINE_SPLIT, lse.data_ptr()) < 0 and b"out_split may be NULL only" in lib.fd_last_error()
    assert call(1, fd._lib.FD_COMBINE_SPLIT, lse.data_ptr(), n_extra=1) < 0
    assert call(1, fd._lib.FD_COMBINE_SPLIT_LSE, lse.data_ptr()) < 0 and b"not both" in lib.fd_last_error()
    assert call(1, fd._lib.FD_COMBINE_SPLIT, lse.data_ptr()) == 0
    torch.cuda.synchronize()
    ref, ref_lse = oracle_decode(wl.to("cpu"))
    assert_out_close(out.cpu(), ref)
    assert_lse_close(lse.cpu(), ref_lse)


def test_prepared_decode_step(fd):
    """PreparedDecode: arguments marshalled once, launched many times -- the same bits as the wrappers, with new
    contents in the same buffers, with rebound pools of the same geometry, and replayed from a HIP graph."""
    wl = fd.utils.make_paged_workload("prepared", [1320, 18, 463, 2049, 0, 777], 32, 8, 128, 16, torch.bfloat16, 32, seed=71)
    g = wl.to(DEV)
    B, Hq, D = g.q.shape
    ref, ref_lse = oracle_decode(wl)
    for variant, fn in (("plain", fd.gqa_fwd_batch_decode), ("intra_rank", fd.gqa_fwd_batch_decode_intra_rank),
                        ("persistent", fd.gqa_fwd_batch_decode_persistent)):
        lse = torch.zeros(B, Hq, dtype=torch.float32, device=DEV)
        kw = {} if variant == "intra_rank" else {"lse_out": lse}
        step = fd.PreparedDecode(g.q, g.k_cache, g.v_cache, g.kv_lens, g.block_table, g.scale, variant=variant,
                                 kv_split=g.kv_split, **kw)
        out = step()
        torch.cuda.synchronize()
        want = fn(g.q, g.k_cache, g.v_cache, None, [1] * B, g.kv_lens, g.block_table, g.scale, kv_split=g.kv_split)
        torch.cuda.synchronize()
        assert out is step.output and torch.equal(out.view(torch.int16), want.view(torch.int16)), variant
        assert_out_close(out[..., :D].cpu(), ref)
        if variant != "intra_rank":
            assert_lse_close(lse.cpu(), ref_lse)
    # new contents in the same buffers, then other pools of the same geometry
    lse = torch.zeros(B, Hq, dtype=torch.float32, device=DEV)
    q, kc, vc, lens = g.q.clone(), g.k_cache.clone(), g.v_cache.clone(), g.kv_lens.clone()
    step = fd.PreparedDecode(q, kc, vc, lens, g.block_table, g.scale, kv_split=-1, lse_out=lse)
    import dataclasses
    gen = torch.Generator().manual_seed(72)
    wl2 = dataclasses.replace(
        wl, q=torch.randn(wl.q.shape, generator=gen).to(torch.bfloat16),
        k_cache=torch.randn(wl.k_cache.shape, generator=gen).to(torch.bfloat16),
        v_cache=torch.randn(wl.v_cache.shape, generator=gen).to(torch.bfloat16),
        block_table=torch.randint(0, wl.k_cache.shape[0], wl.block_table.shape, generator=gen, dtype=torch.int32),
        kv_lens=torch.tensor([5, 2049, 1000, 64, 333, 0], dtype=torch.int32))
    g2 = wl2.to(DEV)
    q.copy_(g2.q)
    lens.copy_(g2.kv_lens)
    out = step(k_cache=g2.k_cache, v_cache=g2.v_cache, block_table=g2.block_table)
    torch.cuda.synchronize()
    ref2, ref2_lse = oracle_decode(wl2)
    assert_out_close(out.cpu(), ref2)
    assert_lse_close(lse.cpu(), ref2_lse)
    with pytest.raises(RuntimeError, match="must keep shape"):
        step(k_cache=g2.k_cache[:-1])
    with pytest.raises(RuntimeError, match="planned step"):
        fd.PreparedDecode(q, kc, vc, lens, g.block_table, g.scale, fuse_combine=True)
    # in a HIP graph: replays follow the contents of the buffers
    step = fd.PreparedDecode(q, g2.k_cache, g2.v_cache, lens, g2.block_table, g.scale, lse_out=lse)
    step()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step()
    torch.cuda.synchronize()
    for new_lens in ([5, 2049, 1000, 64, 333, 0], [2049, 1, 0, 700, 2049, 31]):
        lens.copy_(torch.tensor(new_lens, dtype=torch.int32))
        step.output.zero_()
        graph.replay()
        torch.cuda.synchronize()
        wl2.kv_lens = torch.tensor(new_lens, dtype=torch.int32)
        r3, r3_lse = oracle_decode(wl2)
        assert_out_close(step.output.cpu(), r3)
        assert_lse_close(lse.cpu(), r3_lse)
