"""GPU parity tests of the write side: rotary embedding + KV-cache append (+ fp8 quantisation), and the
decode call on top of it, against the CPU oracle on the same bits.

The append and the fp8 rounding are byte work: bit-exact.  The rotation is floating point with every
operation rounded as in the oracle, so it is compared bit-exactly too.  The attention that follows is held
to the decode path's tolerances.
"""
import numpy as np
import pytest
import torch

import oracle
from helpers import DEV, assert_lse_close, assert_out_close

pytestmark = pytest.mark.gpu


def _tables(B, lens_after, P, num_pages, gen):
    """Disjoint page lists per sequence drawn from one shuffled pool; unused entries hold garbage."""
    maxp = max(1, max(-(-n // P) for n in lens_after))
    perm = torch.randperm(num_pages, generator=gen)
    bt = torch.randint(0, num_pages, (B, maxp + 1), generator=gen, dtype=torch.int32)
    used = 0
    for b, n in enumerate(lens_after):
        need = -(-n // P)
        bt[b, :need] = perm[used:used + need].to(torch.int32)
        used += need
    assert used <= num_pages
    return bt


def _cos_sin(D, max_pos=4096):
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    return oracle.ref_set_cos_sin_cache(inv_freq, max_pos)


@pytest.mark.parametrize("src_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("kv_dtype", ["same", torch.bfloat16, torch.float32, "fp8"])
@pytest.mark.parametrize("D,P,T", [(128, 16, 1), (64, 1, 3), (256, 7, 5)])
def test_append_bit_exact(fd, src_dtype, kv_dtype, D, P, T):
    gen = torch.Generator().manual_seed(1000 * D + 10 * P + T + src_dtype.itemsize)
    B, Hkv, num_pages = 4, 4, 128
    lens = [0, 5, 16, 33]
    bt = _tables(B, [n + T for n in lens], P, num_pages, gen)
    fp8 = kv_dtype == "fp8"
    cdt = torch.uint8 if fp8 else (src_dtype if kv_dtype == "same" else kv_dtype)
    k_new = torch.randn(B, T, Hkv, D, generator=gen).to(src_dtype)
    v_new = (torch.randn(B, T, Hkv, D, generator=gen) * 3).to(src_dtype)
    kc = torch.randint(0, 100, (num_pages, P, Hkv, D), generator=gen).to(cdt)
    vc = torch.randint(0, 100, (num_pages, P, Hkv, D), generator=gen).to(cdt)
    ks = vs = None
    if fp8:
        ks = (k_new.float().abs().amax(dim=(0, 1, 3)) / 448.0).contiguous()
        vs = (v_new.float().abs().amax(dim=(0, 1, 3)) / 300.0).contiguous()     # some values saturate
    kv_lens = torch.tensor(lens, dtype=torch.int32)

    ref_k, ref_v = kc.clone(), vc.clone()
    ref_lens = oracle.ref_kv_append(k_new, v_new, ref_k, ref_v, bt, kv_lens, ks, vs)

    g = lambda t: t.to(DEV) if t is not None else None  # noqa: E731
    kc_g, vc_g, out_lens = g(kc), g(vc), torch.zeros(B, dtype=torch.int32, device=DEV)
    fd.paged_kv_append(g(k_new), g(v_new), kc_g, vc_g, g(bt), g(kv_lens), kv_lens_out=out_lens, k_scale=g(ks),
                       v_scale=g(vs))
    torch.cuda.synchronize()
    assert torch.equal(out_lens.cpu(), ref_lens)
    assert torch.equal(kc_g.cpu().view(torch.uint8), ref_k.view(torch.uint8))    # whole pool: nothing else touched
    assert torch.equal(vc_g.cpu().view(torch.uint8), ref_v.view(torch.uint8))


def test_fp8_rounding_exhaustive_points(fd):
    """Every tie point of the format, its float32 neighbours, all representable values and the subnormal
    range go through the kernel's quantiser and must match torch's conversion byte for byte."""
    tab = oracle.fp8_e4m3fn_decode_table()
    finite = np.sort(tab[~np.isnan(tab)].astype(np.float64))
    mids = ((finite[1:] + finite[:-1]) / 2).astype(np.float32)
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        finite.astype(np.float32), mids, np.nextafter(mids, np.float32(1e9)), np.nextafter(mids, np.float32(-1e9)),
        rng.uniform(-2 ** -5, 2 ** -5, 4096).astype(np.float32), rng.uniform(-500, 500, 4096).astype(np.float32),
        (rng.normal(size=8192) * 20).astype(np.float32),
    ])
    D = 128
    n = -(-vals.size // D)
    x = np.zeros(n * D, dtype=np.float32)
    x[:vals.size] = vals
    k_new = torch.from_numpy(x).view(1, n, 1, D)
    scale = torch.tensor([1.0])
    bt = torch.arange(n, dtype=torch.int32).view(1, n)
    kc = torch.zeros(n, 1, 1, D, dtype=torch.uint8, device=DEV)
    vc = torch.zeros_like(kc)
    for s in (1.0, 0.37):
        scale = torch.tensor([s])
        fd.paged_kv_append(k_new.to(DEV), (k_new * 0.5).to(DEV), kc, vc, bt.to(DEV),
                           torch.zeros(1, dtype=torch.int32, device=DEV), k_scale=scale.to(DEV), v_scale=scale.to(DEV))
        torch.cuda.synchronize()
        assert torch.equal(kc.cpu().view(n, 1, D), oracle.ref_quantize_fp8(k_new[0], scale))
        assert torch.equal(vc.cpu().view(n, 1, D), oracle.ref_quantize_fp8(k_new[0] * 0.5, scale))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("pos_dtype", [torch.int64, torch.int32])
def test_apply_rotary_pos_emb_bit_exact(fd, dtype, D, pos_dtype):
    gen = torch.Generator().manual_seed(D + pos_dtype.itemsize)
    B, T, H = 3, 4, 5
    x = torch.randn(B, T, H, D, generator=gen).to(dtype)
    tab = _cos_sin(D, 512)
    pos = torch.randint(0, 512, (B, T), generator=gen).to(pos_dtype)
    pos[0, 0] = 100000      # clamped to the last row
    got = fd.apply_rotary_pos_emb(x.to(DEV), tab.to(DEV), pos.to(DEV))
    torch.cuda.synchronize()
    ref = oracle.ref_rope(x, tab, pos)
    assert got.dtype == dtype and torch.equal(got.cpu().view(torch.uint8), ref.view(torch.uint8))


def test_rope_append_fused_strided_inputs(fd):
    """q, k, v as column slices of one qkv projection output (the layout the attention block produces),
    rotated q written in place, K rotated then quantised to fp8."""
    gen = torch.Generator().manual_seed(77)
    B, T, Hq, Hkv, D, P, num_pages = 5, 2, 8, 2, 128, 16, 32
    lens = [3, 15, 16, 40, 0]
    qkv = torch.randn(B, T, (Hq + 2 * Hkv) * D, generator=gen).to(torch.bfloat16)
    bt = _tables(B, [n + T for n in lens], P, num_pages, gen)
    kv_lens = torch.tensor(lens, dtype=torch.int32)
    tab = _cos_sin(D)
    pos = (kv_lens[:, None] + torch.arange(T)).long()
    ks, vs = torch.tensor([0.011, 0.009]), torch.tensor([0.01, 0.012])
    kc = torch.zeros(num_pages, P, Hkv, D, dtype=torch.uint8)
    vc = torch.zeros_like(kc)

    q, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
    q4, k4, v4 = q.view(B, T, Hq, D), k.view(B, T, Hkv, D), v.view(B, T, Hkv, D)
    ref_q = oracle.ref_rope(q4, tab, pos)
    ref_k, ref_v = kc.clone(), vc.clone()
    oracle.ref_kv_append(oracle.ref_rope(k4, tab, pos), v4, ref_k, ref_v, bt, kv_lens, ks, vs)

    qkv_g = qkv.to(DEV)
    qg, kg, vg = qkv_g.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
    qg4 = qg.view(B, T, Hq, D)
    kc_g, vc_g = kc.to(DEV), vc.to(DEV)
    ret = fd.rope_kv_append(kg.view(B, T, Hkv, D), vg.view(B, T, Hkv, D), kc_g, vc_g, bt.to(DEV), kv_lens.to(DEV),
                            k_scale=ks.to(DEV), v_scale=vs.to(DEV), cos_sin=tab.to(DEV), position_ids=pos.to(DEV),
                            q=qg4, q_out=qg4)
    torch.cuda.synchronize()
    assert ret.data_ptr() == qg4.data_ptr()
    assert torch.equal(qg4.cpu().view(torch.int16), ref_q.view(torch.int16))
    assert torch.equal(kc_g.cpu(), ref_k) and torch.equal(vc_g.cpu(), ref_v)
    # k and v columns of the projection output are left as they were
    assert torch.equal(kg.cpu(), k) and torch.equal(vg.cpu(), v)


def test_capacity_clamp_and_empty_calls(fd):
    P, Hkv, D = 4, 1, 64
    bt = torch.tensor([[2, 0]], dtype=torch.int32)
    kc = torch.zeros(3, P, Hkv, D, dtype=torch.float16)
    vc = torch.zeros_like(kc)
    k = torch.randn(1, 5, Hkv, D).half()
    v = torch.randn(1, 5, Hkv, D).half()
    lens = torch.tensor([6], dtype=torch.int32)
    ref_k, ref_v = kc.clone(), vc.clone()
    ref_lens = oracle.ref_kv_append(k, v, ref_k, ref_v, bt, lens)
    kc_g, vc_g, out = kc.to(DEV), vc.to(DEV), torch.zeros(1, dtype=torch.int32, device=DEV)
    fd.paged_kv_append(k.to(DEV), v.to(DEV), kc_g, vc_g, bt.to(DEV), lens.to(DEV), kv_lens_out=out)
    # zero new tokens and an empty batch are no-ops
    fd.paged_kv_append(k[:, :0].to(DEV), v[:, :0].to(DEV), kc_g, vc_g, bt.to(DEV), lens.to(DEV))
    fd.paged_kv_append(k[:0].to(DEV), v[:0].to(DEV), kc_g, vc_g, bt[:0].to(DEV), lens[:0].to(DEV))
    torch.cuda.synchronize()
    assert int(out[0]) == 8 == int(ref_lens[0])
    assert torch.equal(kc_g.cpu(), ref_k) and torch.equal(vc_g.cpu(), ref_v)


def test_error_paths(fd):
    B, T, Hkv, D, P = 2, 1, 2, 128, 16
    k = torch.zeros(B, T, Hkv, D, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(8, P, Hkv, D, dtype=torch.bfloat16, device=DEV)
    bt = torch.zeros(B, 2, dtype=torch.int32, device=DEV)
    lens = torch.zeros(B, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="kv_lens_out must not be kv_lens"):
        fd.paged_kv_append(k, k, kc, kc, bt, lens, kv_lens_out=lens)
    with pytest.raises(RuntimeError, match="fp8 KV cache needs"):
        lib = fd.load_library()
        from ctypes import byref
        p = fd._lib.FdParams()
        p.q_heads, p.kv_heads, p.head_dim, p.page_size, p.num_pages, p.max_pages_per_seq = 1, Hkv, D, P, 8, 2
        p.q_dtype, p.kv_dtype = fd._lib.FD_BF16, fd._lib.FD_FP8_E4M3
        fd._lib.check(lib.fd_kv_append(None, k.data_ptr(), k.data_ptr(), kc.data_ptr(), kc.data_ptr(), bt.data_ptr(),
                                       lens.data_ptr(), None, None, B, T, *k.stride()[:3], *k.stride()[:3], kc.stride(1),
                                       kc.stride(2), kc.stride(1), kc.stride(2), bt.stride(0), None, byref(p)))
    with pytest.raises(RuntimeError, match="16-byte aligned"):
        kk = torch.zeros(B, T, Hkv, D + 1, dtype=torch.bfloat16, device=DEV)[..., 1:]
        fd.paged_kv_append(kk, kk, kc, kc, bt, lens)
    with pytest.raises(NotImplementedError):
        fd.flash_attn_with_kvcache(torch.zeros(B, 2, 4, D, dtype=torch.bfloat16, device=DEV), kc, kc, cache_seqlens=lens)
    torch.cuda.synchronize()


def test_token_by_token_build_equals_direct_cache(fd):
    """A cache filled one token per step through the append kernel is the cache the decode tests build
    directly, byte for byte; the decode over it then agrees with the oracle."""
    gen = torch.Generator().manual_seed(9)
    B, Hq, Hkv, D, P, num_pages, steps = 3, 8, 2, 128, 4, 64, 21
    bt = _tables(B, [steps] * B, P, num_pages, gen)
    seq_k = torch.randn(B, steps, Hkv, D, generator=gen).to(torch.bfloat16)
    seq_v = torch.randn(B, steps, Hkv, D, generator=gen).to(torch.bfloat16)
    kc = torch.zeros(num_pages, P, Hkv, D, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    lens_a = torch.zeros(B, dtype=torch.int32, device=DEV)
    lens_b = torch.zeros_like(lens_a)
    bt_g, k_g, v_g = bt.to(DEV), seq_k.to(DEV), seq_v.to(DEV)
    for t in range(steps):
        fd.paged_kv_append(k_g[:, t:t + 1], v_g[:, t:t + 1], kc, vc, bt_g, lens_a, kv_lens_out=lens_b)
        lens_a, lens_b = lens_b, lens_a
    torch.cuda.synchronize()
    assert lens_a.tolist() == [steps] * B
    ref_k = torch.zeros(num_pages, P, Hkv, D, dtype=torch.bfloat16)
    ref_v = torch.zeros_like(ref_k)
    for b in range(B):
        for n in range(steps):
            ref_k[bt[b, n // P], n % P] = seq_k[b, n]
            ref_v[bt[b, n // P], n % P] = seq_v[b, n]
    assert torch.equal(kc.cpu().view(torch.int16), ref_k.view(torch.int16))
    assert torch.equal(vc.cpu().view(torch.int16), ref_v.view(torch.int16))


@pytest.mark.parametrize("layout", ["paged", "dense"])
@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("rope", [False, True])
def test_flash_attn_with_kvcache_decode_step(fd, layout, fp8, rope):
    gen = torch.Generator().manual_seed(31 + 2 * fp8 + rope)
    B, Hq, Hkv, D = 4, 32, 8, 128
    lens = [700, 1, 0, 255]
    if layout == "paged":
        P, num_pages = 16, 128
        bt = _tables(B, [n + 1 for n in lens], P, num_pages, gen)
    else:
        P, num_pages = 1024, B      # KV_Cache layout: one "page" of max_length tokens per sequence
        bt = None
    dtype = torch.bfloat16
    src_k = torch.randn(num_pages, P, Hkv, D, generator=gen).to(dtype)
    src_v = torch.randn(num_pages, P, Hkv, D, generator=gen).to(dtype)
    ks = vs = None
    if fp8:
        ks = torch.full((Hkv,), 5.0 / 448.0)
        vs = torch.full((Hkv,), 5.0 / 448.0)
        kc, vc = oracle.ref_quantize_fp8(src_k, ks), oracle.ref_quantize_fp8(src_v, vs)
    else:
        kc, vc = src_k, src_v
    q = torch.randn(B, 1, Hq, D, generator=gen).to(dtype)
    k = torch.randn(B, 1, Hkv, D, generator=gen).to(dtype)
    v = torch.randn(B, 1, Hkv, D, generator=gen).to(dtype)
    seqlens = torch.tensor(lens, dtype=torch.int32)
    tab = _cos_sin(D, 2048) if rope else None
    pos = seqlens[:, None].long() if rope else None

    # oracle: rotate, append, then attention over cache_seqlens + 1 tokens
    bt_ref = bt if bt is not None else torch.arange(B, dtype=torch.int32).view(B, 1)
    ref_kc, ref_vc = kc.clone(), vc.clone()
    q_r = oracle.ref_rope(q, tab, pos) if rope else q
    k_r = oracle.ref_rope(k, tab, pos) if rope else k
    new_lens = oracle.ref_kv_append(k_r, v, ref_kc, ref_vc, bt_ref, seqlens, ks, vs)
    kf = oracle.dequant_fp8_cache(ref_kc, ks) if fp8 else ref_kc.float()
    vf = oracle.dequant_fp8_cache(ref_vc, vs) if fp8 else ref_vc.float()
    ref, ref_lse = oracle.ref_paged_attn_lse(q_r[:, 0].float(), kf, vf, new_lens.tolist(), bt_ref, D ** -0.5)

    g = lambda t: t.to(DEV) if t is not None else None  # noqa: E731
    kc_g, vc_g, seq_g = g(kc), g(vc), g(seqlens)
    out, lse = fd.flash_attn_with_kvcache(g(q), kc_g, vc_g, k=g(k), v=g(v), cache_seqlens=seq_g, block_table=g(bt),
                                          causal=True, return_softmax_lse=True, cos_sin_cache=g(tab),
                                          position_ids=g(pos), k_scale=g(ks), v_scale=g(vs))
    torch.cuda.synchronize()
    assert out.shape == (B, 1, Hq, D) and lse.shape == (B, Hq, 1)
    assert torch.equal(seq_g.cpu(), seqlens)                       # flash-attn leaves cache_seqlens alone
    assert torch.equal(kc_g.cpu().view(torch.uint8), ref_kc.view(torch.uint8))
    assert torch.equal(vc_g.cpu().view(torch.uint8), ref_vc.view(torch.uint8))
    assert_out_close(out[:, 0], ref)
    assert_lse_close(lse[..., 0], ref_lse)


def test_append_also_ranks_sequences(fd):
    """seq_order_out of the append launch == the stand-alone scheduler on the grown lengths (ties by index,
    lengths capped at the table's capacity), and flash_attn_with_kvcache uses it for batches of 16 and more."""
    gen = torch.Generator().manual_seed(4)
    B, Hq, Hkv, D, P = 300, 8, 2, 128, 16
    lens = torch.randint(0, 48, (B,), generator=gen, dtype=torch.int32)
    lens[5] = lens[9] = lens[200] = 47          # ties, and 47 + 2 new tokens exceeds the capacity of 48
    bt = torch.randperm(B * 3, generator=gen).to(torch.int32).view(B, 3).to(DEV)
    k = torch.randn(B, 2, Hkv, D, generator=gen).to(torch.bfloat16).to(DEV)
    kc = torch.zeros(B * 3, P, Hkv, D, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    grown = torch.empty(B, dtype=torch.int32, device=DEV)
    order = torch.full((2, B), -1, dtype=torch.int32, device=DEV)
    fd.paged_kv_append(k, k, kc, vc, bt, lens.to(DEV), kv_lens_out=grown, seq_order_out=order)
    want = fd.schedule_sequences(grown)
    torch.cuda.synchronize()
    assert torch.equal(grown.cpu(), (lens + 2).clamp(max=48))
    assert torch.equal(order[0].cpu(), want.cpu())
    ref = sorted(range(B), key=lambda i: (-int(grown[i]), i))
    assert order[0].cpu().tolist() == ref
    assert torch.equal(order[1].cpu(), grown.cpu()[order[0].cpu().long()])      # the lengths in issue order

    # the decode-step call: ragged batch of 24 sequences, oracle on the CPU
    B = 24
    lens = torch.randint(0, 600, (B,), generator=gen, dtype=torch.int32)
    pages = 40
    bt = torch.randperm(B * pages, generator=gen).to(torch.int32).view(B, pages)
    kc = torch.randn(B * pages, P, Hkv, D, generator=gen).to(torch.bfloat16)
    vc = torch.randn(B * pages, P, Hkv, D, generator=gen).to(torch.bfloat16)
    q = torch.randn(B, 1, Hq, D, generator=gen).to(torch.bfloat16)
    k = torch.randn(B, 1, Hkv, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(B, 1, Hkv, D, generator=gen).to(torch.bfloat16)
    ref_k, ref_v = kc.clone(), vc.clone()
    new_lens = oracle.ref_kv_append(k, v, ref_k, ref_v, bt, lens)
    ref, _ = oracle.ref_paged_attn_lse(q[:, 0].float(), ref_k.float(), ref_v.float(), new_lens.tolist(), bt, D ** -0.5)
    seen = {}
    real = fd.kernels.kv_append._decode

    def spy(*a, **kw):
        seen["order"], seen["lens"], seen["items"] = kw.get("seq_order"), kw.get("seq_order_lens"), kw.get("item_order")
        return real(*a, **kw)
    fd.kernels.kv_append._decode = spy
    try:
        out = fd.flash_attn_with_kvcache(q.to(DEV), kc.to(DEV), vc.to(DEV), k=k.to(DEV), v=v.to(DEV),
                                         cache_seqlens=lens.to(DEV), block_table=bt.to(DEV), causal=True)
    finally:
        fd.kernels.kv_append._decode = real
    torch.cuda.synchronize()
    if seen["items"] is not None:
        # the append launch computed the decode's (sequence, range) issue order: every pair once, with the grown
        # length of its sequence beside it
        it = seen["items"].cpu().view(2, -1)
        S = it.shape[1] // B
        seqs, ranges = (it[0] & 0xFFFF).tolist(), ((it[0] >> 16) & 0xFFFF).tolist()
        assert sorted(zip(seqs, ranges)) == [(b, r) for b in range(B) for r in range(S)]
        assert it[1].tolist() == [int(new_lens[b]) for b in seqs]
    else:
        assert seen["order"] is not None
        assert seen["order"].cpu().tolist() == sorted(range(B), key=lambda i: (-int(new_lens[i]), i))
        assert seen["lens"].cpu().tolist() == sorted(new_lens.tolist(), reverse=True)
    assert_out_close(out[:, 0], ref)


@pytest.mark.parametrize("fp8", [False, True])
def test_serving_loop_ragged_batch_wide_block_table(fd, fp8):
    """Several decode steps of a ragged batch of 40 sequences through the drop-in call: each step appends one token
    per sequence, lets the append launch order the decode's (sequence, range) items, and decodes -- in a block table
    sized for 8192 tokens whose unused entries are garbage.  Oracle on the CPU after every step."""
    gen = torch.Generator().manual_seed(77)
    B, Hq, Hkv, D, P, cap_pages = 40, 16, 4, 128, 16, 512
    lens = torch.randint(0, 1500, (B,), generator=gen, dtype=torch.int32)
    lens[0], lens[1], lens[2] = 0, 15, 4095
    need = [-(-(int(n) + 4) // P) for n in lens]
    pool = sum(need) + 1
    perm = torch.randperm(pool, generator=gen).to(torch.int32)
    bt = torch.randint(-3, 1 << 20, (B, cap_pages), generator=gen, dtype=torch.int32)
    o = 0
    for b, u in enumerate(need):
        bt[b, :u] = perm[o:o + u]
        o += u
    kc = torch.randn(pool, P, Hkv, D, generator=gen).to(torch.bfloat16)
    vc = torch.randn(pool, P, Hkv, D, generator=gen).to(torch.bfloat16)
    k_scale = v_scale = None
    ref_k, ref_v = kc.clone(), vc.clone()
    if fp8:
        k_scale, v_scale = torch.full((Hkv,), 0.02), torch.full((Hkv,), 0.015)
        ref_k, ref_v = oracle.ref_quantize_fp8(kc.float(), k_scale), oracle.ref_quantize_fp8(vc.float(), v_scale)
    kc_g, vc_g = ref_k.to(DEV), ref_v.to(DEV)
    kw = dict(k_scale=k_scale.to(DEV), v_scale=v_scale.to(DEV)) if fp8 else {}
    lens_g, bt_g = lens.to(DEV), bt.to(DEV)
    for step in range(4):
        q = torch.randn(B, 1, Hq, D, generator=gen).to(torch.bfloat16)
        k = torch.randn(B, 1, Hkv, D, generator=gen).to(torch.bfloat16)
        v = torch.randn(B, 1, Hkv, D, generator=gen).to(torch.bfloat16)
        new_lens = oracle.ref_kv_append(k, v, ref_k, ref_v, bt, lens, k_scale=k_scale, v_scale=v_scale)
        kf = oracle.dequant_fp8_cache(ref_k, k_scale) if fp8 else ref_k.float()
        vf = oracle.dequant_fp8_cache(ref_v, v_scale) if fp8 else ref_v.float()
        ref, _ = oracle.ref_paged_attn_lse(q[:, 0].float(), kf, vf, new_lens.tolist(), bt, D ** -0.5)
        grown = torch.empty_like(lens_g)
        hint = dict(max_kv_len=int(new_lens.max())) if step % 2 else {}   # every other step with the host-side hint
        out = fd.flash_attn_with_kvcache(q.to(DEV), kc_g, vc_g, k=k.to(DEV), v=v.to(DEV), cache_seqlens=lens_g,
                                         block_table=bt_g, causal=True, kv_lens_out=grown, **hint, **kw)
        torch.cuda.synchronize()
        assert torch.equal(grown.cpu(), new_lens), step
        assert_out_close(out[:, 0], ref)
        lens, lens_g = new_lens, grown
    assert torch.equal(kc_g.cpu().view(torch.uint8), ref_k.view(torch.uint8))


def _assert_within_ulps(got, ref, mant_bits, ulps, what):
    got, ref = got.double(), ref.double()
    tol = ref.abs() * (2.0 ** -mant_bits) * ulps + 1e-30
    bad = (got - ref).abs() > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} elements beyond {ulps} ulp, worst {(got - ref).abs().max().item():.3e}"


@pytest.mark.parametrize("dtype,mant,ulps", [(torch.bfloat16, 7, 1), (torch.float16, 10, 1), (torch.float32, 23, 8)])
@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("rope", [True, False])
def test_fused_qk_norm(fd, dtype, mant, ulps, D, rope):
    """RMS norm of q and k inside the append launch against the float64 oracle: within rounding of the activation
    dtype (a different summation order cannot be bit-exact), V untouched by the norm, bit-exact."""
    gen = torch.Generator().manual_seed(D + mant)
    B, T, Hq, Hkv, P, num_pages = 3, 2, 6, 2, 8, 16
    lens = [0, 7, 11]
    q = (torch.randn(B, T, Hq, D, generator=gen) * 3).to(dtype)
    k = (torch.randn(B, T, Hkv, D, generator=gen) * 0.2).to(dtype)
    v = torch.randn(B, T, Hkv, D, generator=gen).to(dtype)
    qw = (1 + 0.3 * torch.randn(D, generator=gen)).to(dtype)
    kw = (1 + 0.3 * torch.randn(D, generator=gen)).to(dtype)
    bt = _tables(B, [n + T for n in lens], P, num_pages, gen)
    kv_lens = torch.tensor(lens, dtype=torch.int32)
    tab = _cos_sin(D, 64) if rope else None
    pos = (kv_lens[:, None] + torch.arange(T)).long() if rope else None
    kc = torch.zeros(num_pages, P, Hkv, D, dtype=dtype)
    vc = torch.zeros_like(kc)

    q_ref = oracle.ref_rms_norm(q, qw, 1e-6)
    k_ref = oracle.ref_rms_norm(k, kw, 1e-5)
    if rope:
        q_ref, k_ref = oracle.ref_rope(q_ref, tab, pos), oracle.ref_rope(k_ref, tab, pos)
    ref_k, ref_v = kc.clone(), vc.clone()
    oracle.ref_kv_append(k_ref, v, ref_k, ref_v, bt, kv_lens)

    g = lambda t: t.to(DEV) if t is not None else None  # noqa: E731
    kc_g, vc_g = g(kc), g(vc)
    q_out = fd.rope_kv_append(g(k), g(v), kc_g, vc_g, g(bt), g(kv_lens), cos_sin=g(tab), position_ids=g(pos), q=g(q),
                              q_norm=(g(qw), 1e-6), k_norm=(g(kw), 1e-5))
    torch.cuda.synchronize()
    if rope:
        # each output mixes two normalised values (each off by up to `ulps`) and is rounded once more: bound the
        # error by the larger partner of the rotated pair
        def close(got, ref):
            got, ref = got.double().reshape(-1, D), ref.double().reshape(-1, D)
            pair = torch.maximum(ref[:, :D // 2].abs(), ref[:, D // 2:].abs()).repeat(1, 2)
            return ((got - ref).abs() <= pair * (2.0 ** -mant) * (3 * ulps + 1) + 1e-30).all()
        assert close(q_out.cpu(), q_ref), "q"
        assert close(kc_g.cpu(), ref_k), "K cache"
    else:
        _assert_within_ulps(q_out.cpu(), q_ref, mant, ulps, "q")
        _assert_within_ulps(kc_g.cpu(), ref_k, mant, ulps, "K cache")
    assert torch.equal(vc_g.cpu().view(torch.uint8), ref_v.view(torch.uint8))
    # q-only call (no append): the same rows
    q_only = fd.rope_kv_append(None, None, None, None, None, None, cos_sin=g(tab), position_ids=g(pos), q=g(q),
                               q_norm=(g(qw), 1e-6))
    torch.cuda.synchronize()
    assert torch.equal(q_only.cpu().view(torch.uint8), q_out.cpu().view(torch.uint8))
