"""Pins the CPU oracle (oracle/) without importing the reference.

The reference holds no golden vectors for this path (its tests are random-vs-PyTorch), so
every function of the oracle is checked against what the mathematics fixes: closed forms,
a library routine (torch SDPA) on the gathered cache, an independent pure-Python float64
brute force, and invariants chosen so that a dropped term, a wrong sign/index or a
transposed operand fails at least one of them.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle.split_combine_model import split_range

torch.manual_seed(0)


def _rand_paged(B, Hq, Hkv, D, P, kv_lens, num_pages, seed=0, dtype=torch.float64, with_replacement=False):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, D, generator=g, dtype=dtype)
    k = torch.randn(num_pages, P, Hkv, D, generator=g, dtype=dtype)
    v = torch.randn(num_pages, P, Hkv, D, generator=g, dtype=dtype)
    maxp = max(1, max(-(-n // P) for n in kv_lens))
    if with_replacement:
        bt = torch.randint(0, num_pages, (B, maxp), generator=g, dtype=torch.int32)
    else:
        bt = torch.stack([torch.randperm(num_pages, generator=g)[:maxp] for _ in range(B)]).to(torch.int32)
    return q, k, v, bt


def _brute_force(q, k, v, kv_lens, bt, scale, soft_cap=0.0):
    """Independent scalar float64 loops: no einsum, no torch softmax, explicit paging arithmetic."""
    B, Hq, D = q.shape
    _, P, Hkv, Dv = v.shape
    G = Hq // Hkv
    out = [[[0.0] * Dv for _ in range(Hq)] for _ in range(B)]
    lse = [[0.0] * Hq for _ in range(B)]
    for b in range(B):
        for h in range(Hq):
            hk = h // G
            scores = []
            for n in range(kv_lens[b]):
                page = int(bt[b][n // P])
                slot = n % P
                s = 0.0
                for d in range(D):
                    s += float(q[b, h, d]) * float(k[page, slot, hk, d])
                s *= scale
                if soft_cap > 0:
                    s = soft_cap * math.tanh(s / soft_cap)
                scores.append(s)
            mx = max(scores)
            ws = [math.exp(s - mx) for s in scores]
            tot = sum(ws)
            lse[b][h] = mx + math.log(tot)
            for n, wgt in enumerate(ws):
                page = int(bt[b][n // P])
                slot = n % P
                for d in range(Dv):
                    out[b][h][d] += wgt / tot * float(v[page, slot, hk, d])
    return torch.tensor(out, dtype=torch.float64), torch.tensor(lse, dtype=torch.float64)


# ------------------------------------------------------------------ decode output and LSE

def test_against_scalar_brute_force():
    kv_lens = [7, 1, 12]
    q, k, v, bt = _rand_paged(3, 6, 2, 8, 4, kv_lens, num_pages=9, seed=1)
    for cap in (0.0, 3.0):
        o, L = oracle.ref_paged_attn_lse(q, k, v, kv_lens, bt, 0.37, soft_cap=cap, compute_dtype=torch.float64)
        ob, Lb = _brute_force(q, k, v, kv_lens, bt, 0.37, soft_cap=cap)
        assert torch.allclose(o, ob, atol=1e-12, rtol=1e-12)
        assert torch.allclose(L, Lb, atol=1e-12, rtol=1e-12)


@pytest.mark.parametrize("Hq,Hkv", [(8, 8), (8, 2), (6, 1)])
def test_against_torch_sdpa_on_gathered_cache(Hq, Hkv):
    """Library cross-check: scaled_dot_product_attention on the contiguous, head-repeated K/V."""
    kv_lens = [33, 5]
    D, P = 16, 4
    q, k, v, bt = _rand_paged(2, Hq, Hkv, D, P, kv_lens, num_pages=20, seed=2)
    scale = 0.21
    o, L = oracle.ref_paged_attn_lse(q, k, v, kv_lens, bt, scale, compute_dtype=torch.float64)
    G = Hq // Hkv
    for b, n in enumerate(kv_lens):
        pages = bt[b, :-(-n // P)].long()
        kk = k[pages].reshape(-1, Hkv, D)[:n]                       # [n, Hkv, D]
        vv = v[pages].reshape(-1, Hkv, D)[:n]
        kk = kk.repeat_interleave(G, dim=1).permute(1, 0, 2)[None]  # [1, Hq, n, D]
        vv = vv.repeat_interleave(G, dim=1).permute(1, 0, 2)[None]
        ref = torch.nn.functional.scaled_dot_product_attention(q[b][None, :, None, :], kk, vv, scale=scale)
        assert torch.allclose(o[b], ref[0, :, 0, :], atol=1e-12)
        sc = torch.einsum("hd,hnd->hn", q[b] * scale, kk[0])
        assert torch.allclose(L[b], torch.logsumexp(sc, -1), atol=1e-12)


def test_closed_forms():
    B, Hq, Hkv, D, P = 1, 4, 2, 8, 4
    g = torch.Generator().manual_seed(3)
    q = torch.randn(B, Hq, D, generator=g, dtype=torch.float64)
    v = torch.randn(6, P, Hkv, D, generator=g, dtype=torch.float64)
    bt = torch.tensor([[4, 1, 5, 0]], dtype=torch.int32)
    n = 14
    # all keys equal -> uniform softmax: out = mean(V), lse = s + ln(n)
    kvec = torch.randn(Hkv, D, generator=g, dtype=torch.float64)
    k = kvec[None, None].expand(6, P, Hkv, D).contiguous()
    o, L = oracle.ref_paged_attn_lse(q, k, v, [n], bt, 0.5, compute_dtype=torch.float64)
    rows = v[bt[0].long()].reshape(-1, Hkv, D)[:n]
    for h in range(Hq):
        hk = h // 2
        assert torch.allclose(o[0, h], rows[:, hk].mean(0), atol=1e-13)
        s = 0.5 * float(q[0, h] @ kvec[hk])
        assert abs(float(L[0, h]) - (s + math.log(n))) < 1e-12
    # kv_len == 1 -> out = V[0], lse = scale * q.k0
    k1 = torch.randn(6, P, Hkv, D, generator=g, dtype=torch.float64)
    o, L = oracle.ref_paged_attn_lse(q, k1, v, [1], bt, 0.5, compute_dtype=torch.float64)
    for h in range(Hq):
        hk = h // 2
        assert torch.allclose(o[0, h], v[4, 0, hk], atol=1e-14)
        assert abs(float(L[0, h]) - 0.5 * float(q[0, h] @ k1[4, 0, hk])) < 1e-12
    # one dominant key -> out -> V[k*]
    kd = torch.zeros(6, P, Hkv, D, dtype=torch.float64)
    kd[1, 2] = 1000.0 * torch.sign(q[0, ::2])        # token 6 (page index 1 of the table -> page 1, slot 2)
    qq = q.clone()
    qq[0, 1] = qq[0, 0]
    qq[0, 3] = qq[0, 2]
    o, _ = oracle.ref_paged_attn_lse(qq, kd, v, [n], bt, 1.0, compute_dtype=torch.float64)
    for h in range(Hq):
        assert torch.allclose(o[0, h], v[1, 2, h // 2], atol=1e-9)


def test_shift_and_scale_invariance():
    kv_lens = [19]
    q, k, v, bt = _rand_paged(1, 4, 2, 8, 4, kv_lens, num_pages=8, seed=4)
    o, L = oracle.ref_paged_attn_lse(q, k, v, kv_lens, bt, 0.3, compute_dtype=torch.float64)
    # adding a vector u to every key adds the constant scale*q.u to every score of a head:
    # the output is unchanged and lse moves by exactly that constant
    u = torch.randn(2, 8, dtype=torch.float64)
    o2, L2 = oracle.ref_paged_attn_lse(q, k + u[None, None], v, kv_lens, bt, 0.3, compute_dtype=torch.float64)
    assert torch.allclose(o, o2, atol=1e-12)
    shift = torch.stack([0.3 * (q[0, h] @ u[h // 2]) for h in range(4)])
    assert torch.allclose(L2[0] - L[0], shift, atol=1e-12)
    # scale folds into q
    o3, L3 = oracle.ref_paged_attn_lse(q * 0.3, k, v, kv_lens, bt, 1.0, compute_dtype=torch.float64)
    assert torch.allclose(o, o3, atol=1e-13) and torch.allclose(L, L3, atol=1e-13)


def test_gqa_head_mapping_is_consecutive():
    """Query heads h*G .. h*G+G-1 share KV head h (repeat_interleave, not tile)."""
    kv_lens = [9]
    q, k, v, bt = _rand_paged(1, 6, 3, 4, 2, kv_lens, num_pages=6, seed=5)
    o, _ = oracle.ref_paged_attn_lse(q, k, v, kv_lens, bt, 1.0, compute_dtype=torch.float64)
    v2 = v.clone()
    v2[:, :, 1] += 100.0       # touch KV head 1 only: query heads 2, 3 change, the others do not
    o2, _ = oracle.ref_paged_attn_lse(q, k, v2, kv_lens, bt, 1.0, compute_dtype=torch.float64)
    changed = (o2 - o).abs().amax(-1)[0] > 1.0
    assert changed.tolist() == [False, False, True, True, False, False]


def test_soft_cap_identity():
    x = torch.linspace(-40, 40, 401, dtype=torch.float64)
    for cap in (30.0, 50.0):
        ref = cap * torch.tanh(x / cap)
        alt = cap * (2 * torch.sigmoid(2 * x / cap) - 1)   # flash_decode.py:64-67
        assert torch.allclose(ref, alt, atol=1e-12)


def test_signature_compatible_wrapper_does_not_mutate_query():
    kv_lens = [5, 3]
    q, k, v, bt = _rand_paged(2, 4, 2, 8, 2, kv_lens, num_pages=6, seed=6, dtype=torch.float32)
    q0 = q.clone()
    out = oracle.ref_paged_attn(q, k, v, [1, 1], kv_lens, bt, 0.5, soft_cap=0.0)
    assert torch.equal(q, q0)
    o, _ = oracle.ref_paged_attn_lse(q, k, v, kv_lens, bt, 0.5)
    assert torch.equal(out, o)


# ------------------------------------------------------------------ paging: bit-exact indexing

def test_paged_equals_contiguous_bit_exact():
    kv_lens = [37, 8, 21]
    q, k, v, bt = _rand_paged(3, 8, 2, 16, 4, kv_lens, num_pages=40, seed=7, dtype=torch.float32,
                              with_replacement=True)          # duplicate pages allowed
    o, L = oracle.ref_paged_attn_lse(q, k, v, kv_lens, bt, 0.25)
    # contiguous copy: sequence b occupies pages b*10 ..., identity table
    P = 4
    kc = torch.zeros(30, P, 2, 16)
    vc = torch.zeros(30, P, 2, 16)
    btc = torch.zeros(3, 10, dtype=torch.int32)
    for b, n in enumerate(kv_lens):
        for j in range(-(-n // P)):
            kc[b * 10 + j] = k[bt[b, j]]
            vc[b * 10 + j] = v[bt[b, j]]
            btc[b, j] = b * 10 + j
    oc, Lc = oracle.ref_paged_attn_lse(q, kc, vc, kv_lens, btc, 0.25)
    assert torch.equal(o, oc) and torch.equal(L, Lc)


def test_pool_permutation_poison_and_garbage_entries():
    kv_lens = [13, 6]
    q, k, v, bt = _rand_paged(2, 4, 2, 8, 4, kv_lens, num_pages=12, seed=8, dtype=torch.float32)
    o, L = oracle.ref_paged_attn_lse(q, k, v, kv_lens, bt, 0.4)
    perm = torch.randperm(12, generator=torch.Generator().manual_seed(1))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(12)
    k2, v2 = k[perm].clone(), v[perm].clone()
    bt2 = inv[bt.long()].to(torch.int32)
    used = set()
    for b, n in enumerate(kv_lens):
        used.update(bt2[b, :-(-n // 4)].tolist())
        bt2[b, -(-n // 4):] = 10 ** 6                 # garbage past ceil(kv_len / P) must never be read
    for pg in range(12):
        if pg not in used:
            k2[pg] = float("nan")
            v2[pg] = float("nan")
    o2, L2 = oracle.ref_paged_attn_lse(q, k2, v2, kv_lens, bt2, 0.4)
    assert torch.equal(o, o2) and torch.equal(L, L2)


def test_empty_sequence_is_defined():
    q, k, v, bt = _rand_paged(2, 4, 2, 8, 4, [0, 3], num_pages=4, seed=9, dtype=torch.float32)
    o, L = oracle.ref_paged_attn_lse(q, k, v, [0, 3], bt, 1.0)
    assert torch.all(o[0] == 0) and torch.all(torch.isneginf(L[0])) and torch.isfinite(o[1]).all()


# ------------------------------------------------------------------ split ranges

def test_split_ranges_partition_by_brute_force():
    for S in (1, 4, 8, 16, 32, 64):
        for kv_len in list(range(0, 300)) + [1023, 1024, 1025, 4095, 4096]:
            per = -(-kv_len // S)
            covered = []
            for s in range(S):
                st, en = split_range(kv_len, S, s)
                assert (en <= st) == (per * s >= kv_len)          # empty iff per*s >= kv_len
                if en > st:
                    assert st == per * s and en - st <= per
                    covered.extend(range(st, en))
            assert covered == list(range(kv_len))
    assert [split_range(1, 32, s)[1] > split_range(1, 32, s)[0] for s in range(32)] == [True] + [False] * 31
    assert sum(split_range(18, 32, s)[1] > split_range(18, 32, s)[0] for s in range(32)) == 18


# ------------------------------------------------------------------ split + combine recurrences

@pytest.mark.parametrize("S", [1, 4, 32])
@pytest.mark.parametrize("P", [1, 16])
def test_split_combine_equals_attention_over_union(S, P):
    kv_lens = [70, 1, 18, 0, 293]
    q, k, v, bt = _rand_paged(5, 8, 2, 16, P, kv_lens, num_pages=-(-300 // P) + 3, seed=10)
    ref_o, ref_L = oracle.ref_paged_attn_lse(q, k, v, kv_lens, bt, 0.3, soft_cap=0.0, compute_dtype=torch.float64)
    o, L, mid = oracle.model_gqa_fwd_batch_decode(q, k, v, kv_lens, bt, 0.3, kv_split=S, compute_dtype=torch.float64)
    assert torch.allclose(o, ref_o, atol=1e-12) and torch.allclose(L, ref_L, atol=1e-12)
    # each non-empty split, on its own, is attention over that token range
    b = 4
    for s in range(S):
        st, en = split_range(kv_lens[b], S, s)
        if en <= st:
            assert torch.all(mid[b, :, s, :16] == 0) and torch.all(torch.isneginf(mid[b, :, s, 16]))
            continue
        pages_needed = -(-en // P)
        # attention over tokens [st, en): shift the table so the range starts at token 0 (needs st % P == 0)
        if st % P == 0:
            sub_bt = bt[b:b + 1, st // P:pages_needed]
            so, sL = oracle.ref_paged_attn_lse(q[b:b + 1], k, v, [en - st], sub_bt, 0.3, compute_dtype=torch.float64)
            assert torch.allclose(mid[b, :, s, :16], so[0], atol=1e-12)
            assert torch.allclose(mid[b, :, s, 16], sL[0], atol=1e-12)


def test_split_model_soft_cap_and_p_rounding():
    kv_lens = [130]
    q, k, v, bt = _rand_paged(1, 4, 1, 16, 4, kv_lens, num_pages=40, seed=11, dtype=torch.float32)
    ref_o, ref_L = oracle.ref_paged_attn_lse(q, k, v, kv_lens, bt, 0.5, soft_cap=30.0)
    o, L, _ = oracle.model_gqa_fwd_batch_decode(q, k, v, kv_lens, bt, 0.5, soft_cap=30.0, kv_split=8)
    assert torch.allclose(o, ref_o, atol=1e-5) and torch.allclose(L, ref_L, atol=1e-5)
    # rounding P to fp16 before P.V (flash_decode.py:230) moves the result by at most fp16 resolution
    o16, _, _ = oracle.model_gqa_fwd_batch_decode(q, k, v, kv_lens, bt, 0.5, kv_split=8, round_p_to=torch.float16)
    o32, _, _ = oracle.model_gqa_fwd_batch_decode(q, k, v, kv_lens, bt, 0.5, kv_split=8)
    assert 0 < (o16 - o32).abs().max() < 5e-3


def test_combine_closed_form_permutation_and_validity():
    g = torch.Generator().manual_seed(12)
    R, B, Hq, D = 8, 2, 3, 5
    outs = torch.randn(R, B, Hq, D, generator=g, dtype=torch.float64)
    lses = torch.rand(R, B, Hq, generator=g, dtype=torch.float64) * 10 + 5
    packed = torch.cat([outs, lses[..., None]], -1)
    lens = torch.ones(R, B, dtype=torch.int32)
    o, L = oracle.model_combine(packed, "rank", global_kv_lens=lens)
    wts = torch.softmax(lses, 0)
    assert torch.allclose(o, (wts[..., None] * outs).sum(0), atol=1e-13)
    assert torch.allclose(L, torch.logsumexp(lses, 0), atol=1e-13)
    perm = torch.randperm(R, generator=g)
    o2, L2 = oracle.model_combine(packed[perm], "rank", global_kv_lens=lens)
    assert torch.allclose(o, o2, atol=1e-13) and torch.allclose(L, L2, atol=1e-13)
    # ranks with kv_len == 0 are skipped whatever their slot holds (flash_decode.py:513-515)
    lens[2, 0] = 0
    lens[5, :] = 0
    poisoned = packed.clone()
    poisoned[2, 0] = float("nan")
    poisoned[5] = float("nan")
    o3, L3 = oracle.model_combine(poisoned, "rank", global_kv_lens=lens)
    for b in range(B):
        keep = [r for r in range(R) if lens[r, b] > 0]
        wb = torch.softmax(lses[keep, b], 0)
        assert torch.allclose(o3[b], (wb[..., None] * outs[keep, b]).sum(0), atol=1e-13)
        assert torch.allclose(L3[b], torch.logsumexp(lses[keep, b], 0), atol=1e-13)
    # nothing valid -> defined result (the reference yields NaN)
    o4, L4 = oracle.model_combine(packed, "rank", global_kv_lens=torch.zeros(R, B, dtype=torch.int32))
    assert torch.all(o4 == 0) and torch.all(torch.isneginf(L4))
    # extra partials are merged like further ranks
    o5, L5 = oracle.model_combine(packed[:3], "rank", global_kv_lens=torch.ones(3, B, dtype=torch.int32),
                                  extra_out=outs[3:], extra_lse=lses[3:])
    assert torch.allclose(o5, o, atol=1e-13) and torch.allclose(L5, L, atol=1e-13)


def test_sp_decode_equals_decode_over_concatenated_cache():
    """test_sp_decode_attn.py:163-198: merging per-shard (out, lse) == attention over all KV."""
    R, B, Hq, Hkv, D, P, per_rank = 4, 2, 6, 2, 8, 2, [11, 6]
    g = torch.Generator().manual_seed(13)
    q = torch.randn(B, Hq, D, generator=g, dtype=torch.float64)
    k_sh, v_sh, bts = [], [], []
    pages = 8
    for r in range(R):
        k_sh.append(torch.randn(pages, P, Hkv, D, generator=g, dtype=torch.float64))
        v_sh.append(torch.randn(pages, P, Hkv, D, generator=g, dtype=torch.float64))
        bts.append(torch.stack([torch.randperm(pages, generator=g)[:6] for _ in range(B)]).to(torch.int32))
    # ragged shards: rank r holds per_rank[b] tokens, except rank 1 of sequence 0 which holds none
    lens = torch.tensor([[per_rank[b] for b in range(B)] for _ in range(R)], dtype=torch.int32)
    lens[1, 0] = 0
    o, L = oracle.model_sp_decode(q, k_sh, v_sh, lens.tolist(), bts, 0.35, kv_split=4, compute_dtype=torch.float64)
    # oracle on the concatenation, token by token
    for b in range(B):
        ks, vs = [], []
        for r in range(R):
            n = int(lens[r, b])
            if n:
                pg = bts[r][b, :-(-n // P)].long()
                ks.append(k_sh[r][pg].reshape(-1, Hkv, D)[:n])
                vs.append(v_sh[r][pg].reshape(-1, Hkv, D)[:n])
        kcat = torch.cat(ks)[:, None]      # one token per page
        vcat = torch.cat(vs)[:, None]
        n = kcat.shape[0]
        ob, Lb = oracle.ref_paged_attn_lse(q[b:b + 1], kcat, vcat, [n], torch.arange(n, dtype=torch.int32)[None],
                                           0.35, compute_dtype=torch.float64)
        assert torch.allclose(o[b], ob[0], atol=1e-12) and torch.allclose(L[b], Lb[0], atol=1e-12)


# ------------------------------------------------------------------ fp8

def test_fp8_table_matches_torch_conversion():
    tab = oracle.fp8_e4m3fn_decode_table()
    ref = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    both_nan = np.isnan(tab) & np.isnan(ref)
    assert np.array_equal(np.isnan(tab), np.isnan(ref)) and both_nan.sum() == 2
    assert np.array_equal(tab[~both_nan], ref[~both_nan])
    assert tab[0x7e] == 448.0 and tab[0x01] == 2.0 ** -9 and tab[0x38] == 1.0 and tab[0xb8] == -1.0


def test_fp8_quantise_dequantise_round_trip():
    g = torch.Generator().manual_seed(14)
    x = torch.randn(5, 4, 3, 16, generator=g)
    qb, scale = oracle.quantize_fp8_cache(x)
    assert qb.dtype == torch.uint8 and scale.shape == (3,)
    assert torch.allclose(scale, x.abs().amax(dim=(0, 1, 3)) / 448.0)
    back = oracle.dequant_fp8_cache(qb, scale)
    # e4m3 has 3 mantissa bits: relative error <= 2^-4 for normal values, absolute <= scale * 2^-10 below
    err = (back - x).abs()
    bound = torch.maximum(x.abs() * 2.0 ** -4, scale.view(1, 1, -1, 1) * 2.0 ** -10)
    assert (err <= bound * 1.0001).all()
    # the largest element of every head maps to +-448 exactly
    assert torch.equal(back.abs().amax(dim=(0, 1, 3)), scale * 448.0)


# ------------------------------------------------------------------ write side: rotary + cache update

def test_cos_sin_table_definition():
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, 8, 2, dtype=torch.float32) / 8))   # D = 8: 4 frequencies
    tab = oracle.ref_set_cos_sin_cache(inv_freq, 16)
    assert tab.shape == (16, 8)
    assert torch.equal(tab[0], torch.tensor([1.0] * 4 + [0.0] * 4))                    # angle 0
    # row t: first half cos(t * f_i), second half sin(t * f_i); f_0 = 1, f_1 = 10000^(-1/4) = 0.1
    assert abs(float(tab[3, 0]) - math.cos(3.0)) < 1e-6 and abs(float(tab[3, 4]) - math.sin(3.0)) < 1e-6
    assert abs(float(tab[5, 1]) - math.cos(0.5)) < 1e-6 and abs(float(tab[5, 5]) - math.sin(0.5)) < 1e-6


def test_rope_is_complex_rotation():
    g = torch.Generator().manual_seed(5)
    B, T, H, D = 2, 3, 4, 16
    x = torch.randn(B, T, H, D, generator=g)
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    tab = oracle.ref_set_cos_sin_cache(inv_freq, 64)
    pos = torch.randint(0, 64, (B, T), generator=g)
    got = oracle.ref_rope(x, tab, pos).double()
    # independent: element pair (i, i + D/2) is the complex number x1 + j x2, multiplied by exp(j * pos * f_i)
    z = torch.complex(x[..., :D // 2].double(), x[..., D // 2:].double())
    ang = pos.double()[:, :, None, None] * inv_freq.double()
    zr = z * torch.exp(1j * ang)
    want = torch.cat([zr.real, zr.imag], dim=-1)
    assert (got - want).abs().max() < 1e-5
    # a swapped sign or half would break the norm or the identity at angle 0
    assert torch.allclose(got.norm(dim=-1), x.double().norm(dim=-1), atol=1e-5)
    assert torch.equal(oracle.ref_rope(x, tab, torch.zeros(B, T, dtype=torch.long)), x)
    # angles add: rotating by p then by q (second table row as a fresh rotation) equals rotating by p + q
    p1, p2 = torch.full((B, T), 7), torch.full((B, T), 12)
    twice = oracle.ref_rope(oracle.ref_rope(x, tab, p1), tab, p2)
    once = oracle.ref_rope(x, tab, p1 + p2)
    assert (twice - once).abs().max() < 1e-5
    # out-of-table positions are clamped
    assert torch.equal(oracle.ref_rope(x, tab, torch.full((B, T), 1000)), oracle.ref_rope(x, tab, torch.full((B, T), 63)))


def test_rope_rounds_to_activation_dtype():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(1, 2, 2, 8, generator=g).to(torch.bfloat16)
    tab = oracle.ref_set_cos_sin_cache(torch.tensor([1.0, 0.5, 0.25, 0.125]), 8)
    got = oracle.ref_rope(x, tab, torch.tensor([[1, 5]]))
    assert got.dtype == torch.bfloat16
    want = oracle.ref_rope(x.float(), tab, torch.tensor([[1, 5]])).to(torch.bfloat16)
    assert torch.equal(got, want)


def test_fp8_rounding_against_brute_force_search():
    g = np.random.default_rng(3)
    tab = oracle.fp8_e4m3fn_decode_table()
    finite = tab[~np.isnan(tab)]
    mids = (np.sort(finite)[1:].astype(np.float64) + np.sort(finite)[:-1].astype(np.float64)) / 2   # every tie point
    vals = np.concatenate([
        g.normal(size=400) * 3, g.uniform(-448, 448, 300), g.uniform(-2 ** -6, 2 ** -6, 200),   # normals, subnormals
        finite.astype(np.float64), mids, np.nextafter(mids.astype(np.float32), np.float32(1e9)).astype(np.float64),
        np.nextafter(mids.astype(np.float32), np.float32(-1e9)).astype(np.float64), [0.0, 448.0, -448.0, 2 ** -10, 2 ** -9],
    ]).astype(np.float32)
    got = oracle.ref_quantize_fp8(torch.from_numpy(vals).view(-1, 1, 1), torch.ones(1)).view(-1).numpy()
    want = oracle.brute_force_fp8(vals)
    zero = vals == 0
    assert np.array_equal(got[~zero], want[~zero])
    assert np.all((got[zero] & 0x7F) == 0)
    # scale divides, and values beyond the largest finite magnitude saturate instead of becoming NaN
    q = oracle.ref_quantize_fp8(torch.tensor([[[1000.0, -1000.0, 3.0]]]), torch.tensor([2.0]))
    assert q.view(-1).tolist() == [0x7E, 0xFE, int(oracle.brute_force_fp8(np.array([1.5], dtype=np.float32))[0])]


@pytest.mark.parametrize("P", [1, 4, 16])
def test_append_round_trip_through_gather(P):
    from oracle.ref_decode import _gather_kv
    g = torch.Generator().manual_seed(11 + P)
    B, Hkv, D, num_pages = 3, 2, 8, 40
    lens = [9, 1, 17]
    maxp = max(-(-n // P) for n in lens)
    perm = torch.randperm(num_pages, generator=g)
    bt = torch.full((B, maxp), -7, dtype=torch.int32)
    used = 0
    for b, n in enumerate(lens):
        need = -(-n // P)
        bt[b, :need] = perm[used:used + need].to(torch.int32)
        used += need
    src_k = [torch.randn(n, Hkv, D, generator=g) for n in lens]
    src_v = [torch.randn(n, Hkv, D, generator=g) for n in lens]
    poison = 12345.0
    kc = torch.full((num_pages, P, Hkv, D), poison)
    vc = torch.full((num_pages, P, Hkv, D), poison)
    cur = torch.zeros(B, dtype=torch.int32)
    # append in ragged chunks: 1 token, then 3, then the rest one sequence at a time
    for chunk in (1, 3, 100):
        for b in range(B):
            lo = int(cur[b])
            hi = min(lo + chunk, lens[b])
            if hi == lo:
                continue
            one_bt, one_len = bt[b:b + 1], cur[b:b + 1]
            grown = oracle.ref_kv_append(src_k[b][lo:hi][None], src_v[b][lo:hi][None], kc, vc, one_bt, one_len)
            assert int(grown[0]) == hi
            cur[b] = hi
    for b, n in enumerate(lens):
        assert torch.equal(_gather_kv(kc, bt[b], n), src_k[b])
        assert torch.equal(_gather_kv(vc, bt[b], n), src_v[b])
    # exactly sum(lens) token rows were written, everything else still holds the poison
    assert int((kc[..., 0, 0] != poison).sum()) == sum(lens) and int((vc[..., 0, 0] != poison).sum()) == sum(lens)


def test_append_capacity_and_fp8():
    g = torch.Generator().manual_seed(2)
    P, Hkv, D = 4, 2, 8
    bt = torch.tensor([[1, 0]], dtype=torch.int32)                    # capacity 8 tokens
    kc = torch.zeros(3, P, Hkv, D, dtype=torch.uint8)
    vc = torch.zeros(3, P, Hkv, D, dtype=torch.uint8)
    k = torch.randn(1, 5, Hkv, D, generator=g)
    v = torch.randn(1, 5, Hkv, D, generator=g)
    ks, vs = torch.tensor([0.01, 0.02]), torch.tensor([0.03, 0.005])
    grown = oracle.ref_kv_append(k, v, kc, vc, bt, torch.tensor([6], dtype=torch.int32), ks, vs)
    assert int(grown[0]) == 8                                         # tokens 6, 7 stored, 8..10 dropped
    assert torch.equal(kc[0, 2], oracle.ref_quantize_fp8(k[0, 0], ks)) and torch.equal(vc[0, 3], oracle.ref_quantize_fp8(v[0, 1], vs))
    assert int(kc[2].sum()) == 0 and int(kc[1].sum()) == 0 and int(kc[0, :2].sum()) == 0
    # dequantised values are within half an fp8 step (2^-4 relative) of the source
    deq = oracle.dequant_fp8_cache(kc[0:1, 2:3], ks)[0, 0]
    assert ((deq - k[0, 0]).abs() <= 0.0625 * k[0, 0].abs() + 0.01 * 2 ** -9 + 1e-7).all()


def test_rms_norm_against_library_and_closed_forms():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(3, 2, 4, 32, generator=g)
    w = 1 + 0.2 * torch.randn(32, generator=g)
    got = oracle.ref_rms_norm(x, w, 1e-6)
    lib = torch.nn.functional.rms_norm(x.view(-1, 32), (32,), weight=w, eps=1e-6).view_as(x)
    assert (got - lib).abs().max() < 2e-6
    # eps = 0: invariant under scaling of the row; with w = 1 every output row has RMS 1
    ones = torch.ones(32)
    assert torch.allclose(oracle.ref_rms_norm(x * 7.5, ones, 0.0), oracle.ref_rms_norm(x, ones, 0.0), atol=1e-6)
    assert torch.allclose(oracle.ref_rms_norm(x, ones, 0.0).pow(2).mean(-1), torch.ones(3, 2, 4), atol=1e-5)
    # constant row c: c / sqrt(c^2 + eps) * w
    c = torch.full((1, 1, 1, 32), 3.0)
    assert torch.allclose(oracle.ref_rms_norm(c, w, 1.0), (3.0 / (10.0 ** 0.5)) * w.view(1, 1, 1, 32), atol=1e-6)
    # rounded once to the activation dtype
    xb = x.to(torch.bfloat16)
    assert torch.equal(oracle.ref_rms_norm(xb, w.to(torch.bfloat16), 1e-6),
                       oracle.ref_rms_norm(xb.double(), w.to(torch.bfloat16).double(), 1e-6).to(torch.bfloat16))
