"""Properties of the decode path that hold at any size, checked on the GPU at the full sizes of the benchmark
configurations and without the CPU oracle: a closed form (all keys equal -> the output is the mean of V and
lse = score + ln n), exact scaling in V, every token twice (same output, lse + ln 2), and independence of where
the pages lie in the pool.  Each would catch a dropped or doubled range, a wrong split weight or a wrong page."""
import math

import pytest
import torch

from helpers import DEV, assert_lse_close, assert_out_rel

pytestmark = pytest.mark.gpu


def _run(fd, g, **kw):
    B, Hq, _ = g.q.shape
    lse = torch.empty(B, Hq, dtype=torch.float32, device=DEV)
    if g.k_scale is not None:
        kw.update(k_scale=g.k_scale, v_scale=g.v_scale)
    out = fd.gqa_fwd_batch_decode(g.q, g.k_cache, g.v_cache, None, None, g.kv_lens, g.block_table, g.scale, g.soft_cap,
                                  kv_split=g.kv_split, lse_out=lse, **kw)
    torch.cuda.synchronize()
    return out, lse


def _values(g, cache, scale):
    """fp32 values of a pool (an fp8 pool dequantised with its per-head scales)."""
    if scale is None:
        return cache.float()
    return cache.view(torch.float8_e4m3fn).float() * scale[:, None]


@pytest.mark.parametrize("idx", [2, 4, 5])
@pytest.mark.parametrize("exact", [False, True])
def test_doubling_v_doubles_the_output_bit_for_bit(fd, idx, exact):
    """Multiplying by two commutes with every rounding on the way (products, sums, 16-bit partials, the output), so
    out(2 V) == 2 out(V) exactly and the LSEs do not move; with the library's split plan and with exactly the
    configuration's split count."""
    g = fd.utils.make_config(idx).to(DEV)
    kw = dict(plan_splits=not exact)
    out, lse = _run(fd, g, **kw)
    assert torch.isfinite(out.float()).all() and out.float().abs().max() > 0
    if g.v_scale is not None:
        g.v_scale = g.v_scale * 2
    else:
        g.v_cache.mul_(2)
    out2, lse2 = _run(fd, g, **kw)
    assert torch.equal(out2.float(), out.float() * 2)
    assert torch.equal(lse2, lse)


@pytest.mark.parametrize("idx", [2, 5])
def test_all_keys_equal_gives_the_mean_of_v(fd, idx):
    """One key vector per KV head in every slot of the pool: all scores of a query head are the same number, so the
    softmax is uniform -- out = mean of the sequence's V rows, lse = scale * q.k + ln(kv_len)."""
    g = fd.utils.make_config(idx).to(DEV)
    B, Hq, D = g.q.shape
    _, P, Hkv, _ = g.k_cache.shape
    G = Hq // Hkv
    gen = torch.Generator().manual_seed(77 + idx)
    kvec = torch.randn(Hkv, D, generator=gen).to(DEV)
    if g.k_scale is not None:
        kvec = (kvec / g.k_scale[:, None]).clamp(-448, 448).to(torch.float8_e4m3fn)
        g.k_cache.view(torch.float8_e4m3fn).copy_(kvec.expand_as(g.k_cache))
    else:
        kvec = kvec.to(g.k_cache.dtype)
        g.k_cache.copy_(kvec.expand_as(g.k_cache))
    out, lse = _run(fd, g)
    kval = _values(g, kvec, g.k_scale)                                        # [Hkv, D] as the kernel sees them
    score = (g.q.float() * kval.repeat_interleave(G, dim=0)[None]).sum(-1) * g.scale   # [B, Hq]
    lens = g.kv_lens.tolist()
    ref = torch.empty(B, Hq, D, dtype=torch.float32, device=DEV)
    for b, n in enumerate(lens):
        pages = g.block_table[b, :-(-n // P)].long()
        v = _values(g, g.v_cache[pages], g.v_scale).view(-1, Hkv, D)[:n]      # the sequence's V rows in order
        ref[b] = v.double().mean(0).float().repeat_interleave(G, dim=0)
    ref_lse = score + torch.tensor([math.log(n) for n in lens], device=DEV)[:, None]
    # the output is rounded to bf16 once: 2^-9 of each value
    assert_out_rel(out, ref, rms_rtol=3e-3, max_rtol=4e-3)
    assert_lse_close(lse, ref_lse, rtol=1e-5)


@pytest.mark.parametrize("idx", [2, 5])
def test_every_token_twice_keeps_the_output_and_adds_ln2(fd, idx):
    """The block table lists every page of a sequence twice and the length doubles (the sequences of these
    configurations fill their pages): softmax over each token twice is the same distribution, lse grows by ln 2."""
    g = fd.utils.make_config(idx).to(DEV)
    P = g.k_cache.shape[1]
    assert all(n % P == 0 for n in g.kv_lens.tolist())
    out, lse = _run(fd, g)
    g.block_table = torch.cat([g.block_table, g.block_table], dim=1).contiguous()
    g.kv_lens = g.kv_lens * 2
    out2, lse2 = _run(fd, g)
    # two roundings to bf16 of nearly the same fp32 values (the split plan differs): one ulp, 2^-8, at most
    assert_out_rel(out2, out.float(), rms_rtol=3e-3, max_rtol=8e-3)
    assert_lse_close(lse2, lse + math.log(2.0), rtol=1e-5)


def test_moving_the_pages_in_the_pool_changes_no_bit(fd):
    """Config 2 with its pages permuted inside the pool and the block table following them."""
    g = fd.utils.make_config(2).to(DEV)
    out, lse = _run(fd, g)
    pages = g.k_cache.shape[0]
    perm = torch.randperm(pages, generator=torch.Generator().manual_seed(5)).to(DEV)   # page i moves to perm[i]
    k2, v2 = torch.empty_like(g.k_cache), torch.empty_like(g.v_cache)
    k2[perm] = g.k_cache
    v2[perm] = g.v_cache
    g.k_cache, g.v_cache = k2, v2
    g.block_table = perm[g.block_table.long()].to(torch.int32)
    out2, lse2 = _run(fd, g)
    assert torch.equal(out2, out) and torch.equal(lse2, lse)
