"""GPU tests of the decode block (projection -> rotary + cache append -> split-KV decode -> projection) against
the CPU oracle run on the same projected activations."""
import pytest
import torch

import oracle
from helpers import DEV

pytestmark = pytest.mark.gpu


class _Norm:
    def __init__(self, w, eps):
        self.weight, self.variance_epsilon = w, eps


class _Proj:
    def __init__(self, w):
        self.weight = w


class _HFAttn:
    """Stand-in for a HF attention module: just the attributes TP_Attn._init_parameters reads."""

    def __init__(self, wq, wk, wv, wo, qn=None, kn=None):
        self.q_proj, self.k_proj, self.v_proj, self.o_proj = _Proj(wq), _Proj(wk), _Proj(wv), _Proj(wo)
        if qn is not None:
            self.q_norm, self.k_norm = _Norm(qn, 1e-6), _Norm(kn, 1e-6)


@pytest.mark.parametrize("cache_kind", ["dense", "paged", "paged_fp8"])
@pytest.mark.parametrize("qk_norm", [False, True])
def test_decode_block_steps(fd, cache_kind, qk_norm):
    gen = torch.Generator().manual_seed(5 + qk_norm)
    B, hidden, Hq, Hkv, D, L, prefill, steps = 3, 256, 8, 2, 128, 128, 37, 3
    dt = torch.bfloat16
    wq = (torch.randn(Hq * D, hidden, generator=gen) * 0.06).to(dt)
    wk = (torch.randn(Hkv * D, hidden, generator=gen) * 0.06).to(dt)
    wv = (torch.randn(Hkv * D, hidden, generator=gen) * 0.06).to(dt)
    wo = (torch.randn(hidden, Hq * D, generator=gen) * 0.03).to(dt)
    qn = (1 + 0.1 * torch.randn(D, generator=gen)).to(dt) if qk_norm else None
    kn = (1 + 0.1 * torch.randn(D, generator=gen)).to(dt) if qk_norm else None
    attn = fd.layers.TP_Attn(rank=0, world_size=1)
    attn._init_parameters(_HFAttn(wq, wk, wv, wo, qn, kn))
    attn._init_ctx()
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    tab = fd.layers._set_cos_sin_cache(inv_freq.to(DEV), L)
    assert torch.allclose(tab.cpu(), oracle.ref_set_cos_sin_cache(inv_freq, L), atol=1e-6)
    tab = oracle.ref_set_cos_sin_cache(inv_freq, L).to(DEV)       # same bits on both sides

    if cache_kind == "dense":
        cache = fd.layers.KV_Cache(num_layers=2, batch_size=B, max_length=L, kv_heads=Hkv, head_dim=D, dtype=dt,
                                   world_size=1)
        P = L
        bt_cpu = torch.arange(B, dtype=torch.int32).view(B, 1)
    else:
        cache = fd.layers.PagedKV_Cache(num_layers=2, batch_size=B, max_length=L, kv_heads=Hkv, head_dim=D, dtype=dt,
                                        page_size=16, fp8=cache_kind == "paged_fp8", seed=3)
        P = 16
        bt_cpu = cache.block_table.cpu()
    layer = 1
    fp8 = cache_kind == "paged_fp8"
    ks = cache.update_kv_cache(None, None, layer) and cache.k_scale
    vs = cache.v_scale
    ks_cpu, vs_cpu = (ks.cpu(), vs.cpu()) if fp8 else (None, None)

    # fill the cache with a "prompt" through the same append kernel (rotated K), mirrored on the CPU
    pk = torch.randn(B, prefill, Hkv, D, generator=gen).to(dt)
    pv = torch.randn(B, prefill, Hkv, D, generator=gen).to(dt)
    ppos = torch.arange(prefill).repeat(B, 1)
    kc, vc, off = cache.update_kv_cache(None, None, layer)
    bt_g = cache.block_table if cache.block_table is not None else bt_cpu.to(DEV)
    new_off = torch.empty_like(off)
    fd.rope_kv_append(pk.to(DEV), pv.to(DEV), kc, vc, bt_g, off, kv_lens_out=new_off, k_scale=ks, v_scale=vs,
                      cos_sin=tab, position_ids=ppos.to(DEV))
    cache.kv_offset.copy_(new_off)
    ref_kc = torch.zeros(kc.shape, dtype=kc.dtype)
    ref_vc = torch.zeros(vc.shape, dtype=vc.dtype)
    ref_off = oracle.ref_kv_append(oracle.ref_rope(pk, tab.cpu(), ppos), pv, ref_kc, ref_vc, bt_cpu,
                                   torch.zeros(B, dtype=torch.int32), ks_cpu, vs_cpu)

    for step in range(steps):
        x = torch.randn(B, 1, hidden, generator=gen).to(dt)
        pos = cache.get_kv_len().cpu()[:, None].long()
        y = attn.fwd(x.to(DEV), pos.to(DEV), tab, cache, layer)
        cache.inc_offset()
        torch.cuda.synchronize()

        # oracle from the projected activations (the projections themselves are library GEMMs on both sides)
        qkv = torch.nn.functional.linear(x.to(DEV), attn.wqkv)
        q, k, v = [t.view(B, 1, -1, D) for t in qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)]
        q, k, v = q.cpu(), k.cpu(), v.cpu()
        if qk_norm:
            q, k = oracle.ref_rms_norm(q, qn, 1e-6), oracle.ref_rms_norm(k, kn, 1e-6)
        q_r, k_r = oracle.ref_rope(q, tab.cpu(), pos), oracle.ref_rope(k, tab.cpu(), pos)
        ref_off = oracle.ref_kv_append(k_r, v, ref_kc, ref_vc, bt_cpu, ref_off, ks_cpu, vs_cpu)
        kf = oracle.dequant_fp8_cache(ref_kc, ks_cpu) if fp8 else ref_kc.float()
        vf = oracle.dequant_fp8_cache(ref_vc, vs_cpu) if fp8 else ref_vc.float()
        o, _ = oracle.ref_paged_attn_lse(q_r[:, 0].float(), kf, vf, ref_off.tolist(), bt_cpu, D ** -0.5)
        ref_y = torch.nn.functional.linear(o.view(B, 1, -1), wo.float())

        assert torch.equal(cache.get_kv_len().cpu(), ref_off)
        if qk_norm:
            # the fused norm sums in another order than the float64 oracle: K agrees to rounding, not bit for bit
            got_k = oracle.dequant_fp8_cache(kc.cpu(), ks_cpu) if fp8 else kc.cpu().float()
            assert (got_k - kf).abs().max().item() <= (0.13 if fp8 else 0.04), f"K cache differs at step {step}"
            ref_kc.copy_(kc.cpu())   # continue from the same cache on both sides
        else:
            assert torch.equal(kc.cpu().view(torch.uint8), ref_kc.view(torch.uint8)), f"K cache differs at step {step}"
        assert torch.equal(vc.cpu().view(torch.uint8), ref_vc.view(torch.uint8))
        err = (y.float().cpu() - ref_y).abs().max().item()
        assert err <= 3e-2, f"step {step}: max abs err {err}"
    # the other layer's cache was never touched
    assert int(cache.k_cache[0].view(torch.uint8).max()) == 0


def test_refusals(fd):
    with pytest.raises(NotImplementedError):
        fd.layers.TP_Attn(rank=0, world_size=8)
    attn = fd.layers.TP_Attn()
    w = torch.zeros(128, 64, dtype=torch.bfloat16)
    attn.init_from_weights(w, w, w, torch.zeros(64, 128, dtype=torch.bfloat16))
    with pytest.raises(NotImplementedError):
        attn.fwd(torch.zeros(1, 2, 64, dtype=torch.bfloat16, device=DEV), None, None, None, 0)


@pytest.mark.parametrize("cache_kind", ["dense", "paged_fp8"])
def test_decode_block_in_a_hip_graph(fd, cache_kind):
    """The reference's engine captures its decode step in a graph and replays it with static input tensors
    (models/engine.py:75-105).  The whole block -- projections, norm + rotary + append, split, combine -- is
    captured once here and replayed while the cache grows; every replay is checked against the same step run
    eagerly on a twin cache."""
    gen = torch.Generator().manual_seed(12)
    B, hidden, Hq, Hkv, D, L, prefill, steps = 20, 256, 8, 2, 128, 256, 150, 4
    dt = torch.bfloat16
    mk = lambda *s, sc=0.06: (torch.randn(*s, generator=gen) * sc).to(dt)  # noqa: E731
    attn = fd.layers.TP_Attn()
    attn._init_parameters(_HFAttn(mk(Hq * D, hidden), mk(Hkv * D, hidden), mk(Hkv * D, hidden), mk(hidden, Hq * D, sc=0.03),
                                  (1 + mk(D, sc=0.1)).to(dt), (1 + mk(D, sc=0.1)).to(dt)))
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    tab = fd.layers._set_cos_sin_cache(inv_freq.to(DEV), L)

    def new_cache():
        if cache_kind == "dense":
            return fd.layers.KV_Cache(num_layers=1, batch_size=B, max_length=L, kv_heads=Hkv, head_dim=D, dtype=dt,
                                      world_size=1)
        return fd.layers.PagedKV_Cache(num_layers=1, batch_size=B, max_length=L, kv_heads=Hkv, head_dim=D, dtype=dt,
                                       page_size=16, fp8=True, seed=1)
    caches = [new_cache(), new_cache()]
    start = torch.randint(1, prefill, (B,), generator=gen, dtype=torch.int32)     # ragged: the append also schedules
    pk, pv = mk(B, prefill, Hkv, D, sc=1.0), mk(B, prefill, Hkv, D, sc=1.0)
    for c in caches:
        kc, vc, off = c.update_kv_cache(None, None, 0)
        bt = c.block_table if c.block_table is not None else torch.arange(B, dtype=torch.int32, device=DEV).view(B, 1)
        fd.rope_kv_append(pk.to(DEV), pv.to(DEV), kc, vc, bt, off, k_scale=c.k_scale, v_scale=c.v_scale)
        c.kv_offset.copy_(start)       # only the first start[b] prompt tokens count

    x = torch.zeros(B, 1, hidden, dtype=dt, device=DEV)
    pos = torch.zeros(B, 1, dtype=torch.long, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        attn.fwd(x, pos, tab, caches[0], 0)         # warm-up outside the capture (library handles, allocator)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    caches[0].kv_offset.copy_(start)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_graph = attn.fwd(x, pos, tab, caches[0], 0)
    caches[0].kv_offset.copy_(start)
    # the capture ran no kernel, but the warm-up wrote one token at position start[b]: the replays overwrite it

    for step in range(steps):
        x.copy_(torch.randn(B, 1, hidden, generator=gen).to(dt))
        pos.copy_(caches[0].get_kv_len()[:, None].long())
        graph.replay()
        caches[0].inc_offset()
        torch.cuda.synchronize()
        got = y_graph.clone()
        y_eager = attn.fwd(x, pos, tab, caches[1], 0)          # eager twin, its own cache
        caches[1].inc_offset()
        torch.cuda.synchronize()
        assert torch.equal(got, y_eager), f"replay {step} differs from the eager step"
        assert torch.equal(caches[0].k_cache.view(torch.uint8), caches[1].k_cache.view(torch.uint8))
        assert torch.equal(caches[0].kv_offset, caches[1].kv_offset)
    assert torch.isfinite(y_eager.float()).all() and float(y_eager.float().abs().max()) > 0
