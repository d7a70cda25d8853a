"""KV pools far beyond 4 GiB: a 288 GB part holds pools of tens of GiB, so every kernel's row addressing must be 64-bit.

One 2 x 12 GiB allocation is viewed as the K and V pool of each case; only the pages a case references are ever written
(at the far end of the pool, around the 4 GiB and 8 GiB byte offsets, and at the start).  The oracle runs on
the compact CPU copy of those pages with the table mapped back."""
import pytest
import torch

import oracle
from helpers import DEV, assert_lse_close, assert_out_close, oracle_decode

pytestmark = pytest.mark.gpu

POOL_BYTES = 12 << 30


@pytest.fixture(scope="module")
def raw_pools():
    free, _ = torch.cuda.mem_get_info()
    if free < 2 * POOL_BYTES + (8 << 30):
        pytest.skip("needs 32 GiB of free device memory")
    raw = torch.empty(2, POOL_BYTES, dtype=torch.uint8, device=DEV)
    yield raw
    del raw
    torch.cuda.empty_cache()


def _far_pages(num_big, n_used, page_bytes, gen):
    """n_used distinct page ids of a pool of num_big pages: its last pages, pages on both sides of the 4 / 8 GiB
    byte offsets, and its first pages."""
    ids = set(range(num_big - 1, num_big - 1 - n_used // 2, -1))
    for gib in (4, 8):
        mid = (gib << 30) // page_bytes
        ids.update(range(mid - 2, mid + 2))
    ids.update(range(0, 4))
    ids = sorted(i for i in ids if 0 <= i < num_big)
    extra = num_big // 2
    while len(ids) < n_used:
        if extra not in ids:
            ids.append(extra)
        extra += 7
    ids = torch.tensor(ids[:n_used], dtype=torch.int64)
    return ids[torch.randperm(n_used, generator=gen)]


def _big_view(raw_half, like, P, Hkv, D):
    page_bytes = P * Hkv * D * like.element_size()
    num_big = POOL_BYTES // page_bytes
    return raw_half[:num_big * page_bytes].view(like.dtype).view(num_big, P, Hkv, D), num_big, page_bytes


CASES = [  # name, Hq, Hkv, D, P, dtype, fp8, path
    ("mfma_bf16_d128", 32, 8, 128, 16, torch.bfloat16, False, "auto"),
    ("mfma_fp16_d128_two_blocks", 64, 2, 128, 16, torch.float16, False, "auto"),
    ("mfma_fp8_d128", 64, 8, 128, 16, torch.bfloat16, True, "auto"),
    ("mfma_fp8_d128_two_blocks", 64, 2, 128, 16, torch.float16, True, "auto"),
    ("mfma_bf16_d256", 16, 4, 256, 16, torch.bfloat16, False, "auto"),
    ("mfma_fp8_d256", 16, 4, 256, 16, torch.bfloat16, True, "auto"),
    ("mfma_bf16_d64", 32, 8, 64, 16, torch.bfloat16, False, "auto"),
    ("valu_bf16_d128", 32, 8, 128, 16, torch.bfloat16, False, "valu"),
    ("valu_fp32_d128_page1", 8, 2, 128, 1, torch.float32, False, "auto"),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_decode_from_the_far_end_of_a_12_gib_pool(fd, raw_pools, case):
    name, Hq, Hkv, D, P, dtype, fp8, path = case
    wl = fd.utils.make_paged_workload(name, [1320, 18, 463, 2049], Hq, Hkv, D, P, dtype, 8, seed=41, fp8_kv=fp8)
    gen = torch.Generator().manual_seed(5)
    n_used = wl.k_cache.shape[0]
    big_k, num_big, page_bytes = _big_view(raw_pools[0], wl.k_cache, P, Hkv, D)
    big_v, _, _ = _big_view(raw_pools[1], wl.v_cache, P, Hkv, D)
    assert num_big * page_bytes > 8 << 30
    ids = _far_pages(num_big, n_used, page_bytes, gen)
    ids_dev = ids.to(DEV)
    if fp8:   # index_put is not implemented for float8: move the bytes
        big_k.view(torch.uint8)[ids_dev] = wl.k_cache.view(torch.uint8).to(DEV)
        big_v.view(torch.uint8)[ids_dev] = wl.v_cache.view(torch.uint8).to(DEV)
    else:
        big_k[ids_dev] = wl.k_cache.to(DEV)
        big_v[ids_dev] = wl.v_cache.to(DEV)
    table = ids[wl.block_table.long()].to(torch.int32).to(DEV)
    B = wl.q.shape[0]
    lse = torch.empty(B, Hq, dtype=torch.float32, device=DEV)
    kw = dict(k_scale=wl.k_scale.to(DEV), v_scale=wl.v_scale.to(DEV)) if fp8 else {}
    out = fd.gqa_fwd_batch_decode(wl.q.to(DEV), big_k, big_v, None, None, wl.kv_lens.to(DEV), table, wl.scale,
                                  kv_split=wl.kv_split, lse_out=lse, path=path, **kw)
    torch.cuda.synchronize()
    ref, ref_lse = oracle_decode(wl)
    f32 = dtype == torch.float32
    assert_out_close(out.cpu(), ref, atol=2e-4 if f32 else 2e-2)
    assert_lse_close(lse.cpu(), ref_lse, rtol=1e-5 if f32 else 1e-3)


@pytest.mark.parametrize("cache_dtype", [torch.bfloat16, torch.float8_e4m3fn])
def test_append_into_the_far_end_of_a_12_gib_pool(fd, raw_pools, cache_dtype):
    gen = torch.Generator().manual_seed(9)
    B, T, Hq, Hkv, D, P = 3, 5, 8, 2, 128, 16
    fp8 = cache_dtype == torch.float8_e4m3fn
    n_used = 12
    lens = torch.tensor([5, 16, 27], dtype=torch.int32)
    k = torch.randn(B, T, Hkv, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(B, T, Hkv, D, generator=gen).to(torch.bfloat16)
    compact_k = torch.randn(n_used, P, Hkv, D, generator=gen).to(torch.bfloat16)
    compact_v = torch.randn(n_used, P, Hkv, D, generator=gen).to(torch.bfloat16)
    k_scale = v_scale = None
    if fp8:
        k_scale, v_scale = torch.tensor([0.02, 0.015]), torch.tensor([0.01, 0.03])
        compact_k = oracle.ref_quantize_fp8(compact_k.float(), k_scale)
        compact_v = oracle.ref_quantize_fp8(compact_v.float(), v_scale)
    big_k, num_big, page_bytes = _big_view(raw_pools[0], compact_k, P, Hkv, D)
    big_v, _, _ = _big_view(raw_pools[1], compact_v, P, Hkv, D)
    ids = _far_pages(num_big, n_used, page_bytes, gen)
    ids_dev = ids.to(DEV)
    big_k.view(torch.uint8)[ids_dev] = compact_k.view(torch.uint8).to(DEV)
    big_v.view(torch.uint8)[ids_dev] = compact_v.view(torch.uint8).to(DEV)
    bt = torch.randperm(n_used, generator=gen).to(torch.int32)[:9].view(B, 3)
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    tab = oracle.ref_set_cos_sin_cache(inv_freq, 64)
    pos = lens[:, None].long() + torch.arange(T)[None, :]
    oracle.ref_kv_append(oracle.ref_rope(k, tab, pos), v, compact_k, compact_v, bt, lens, k_scale=k_scale, v_scale=v_scale)
    kw = dict(k_scale=k_scale.to(DEV), v_scale=v_scale.to(DEV)) if fp8 else {}
    fd.rope_kv_append(k.to(DEV), v.to(DEV), big_k, big_v, ids[bt.long()].to(torch.int32).to(DEV), lens.to(DEV),
                      cos_sin=tab.to(DEV), position_ids=pos.to(DEV), **kw)
    torch.cuda.synchronize()
    assert torch.equal(big_k.view(torch.uint8)[ids_dev].cpu(), compact_k.view(torch.uint8))
    assert torch.equal(big_v.view(torch.uint8)[ids_dev].cpu(), compact_v.view(torch.uint8))
