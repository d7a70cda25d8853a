"""Seeded random sweep over shapes and launch options of the decode path against the CPU oracle: every MFMA and
VALU kernel, tile boundaries (kv_len around multiples of 16 / 32 / 64), more waves than tiles, empty sequences,
sibling-head workgroups, caller-visible and internal partials, the scheduler and the fused combine."""
import random

import pytest
import torch

from helpers import assert_lse_close, assert_out_close, assert_out_rel, oracle_decode, run_decode

pytestmark = pytest.mark.gpu

CASES = 160


def _case(i):
    rng = random.Random(9000 + i)
    D = rng.choice([64, 128, 128, 256])
    kind = rng.choice(["bf16", "fp16", "fp8", "fp32"]) if D != 64 else rng.choice(["bf16", "fp16", "fp32"])
    Hkv = rng.choice([1, 2, 4, 8])
    G = rng.choice([1, 2, 3, 4, 6, 8, 16, 20])
    P = rng.choice([1, 4, 16, 16, 32, 128])
    B = rng.choice([1, 2, 3, 5, 9])
    edge = [0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 257, 511, 513]
    lens = [rng.choice(edge) if rng.random() < 0.6 else rng.randint(1, 1500) for _ in range(B)]
    if max(lens) == 0:
        lens[0] = 40
    return dict(D=D, kind=kind, Hq=Hkv * G, Hkv=Hkv, P=P, lens=lens, kv_split=rng.choice([1, 2, 5, 8, 32]),
                soft_cap=rng.choice([0.0, 0.0, 30.0]), waves=rng.choice([0, 0, 1, 2, 4, 8]),
                variant=rng.choice(["plain", "plain", "persistent", "intra"]), fuse=rng.random() < 0.2,
                plan=rng.random() < 0.5, path=rng.choice(["auto", "auto", "valu"]))


@pytest.mark.parametrize("i", range(CASES))
def test_random_shape(fd, i):
    _check_case(fd, _case(i), i)


@pytest.mark.parametrize("i", range(40))
def test_random_shape_fp8_head_dim_64(fd, i):
    """The same sweep pinned to 64-byte fp8 rows, which have an MFMA kernel of their own (K and V both through LDS)."""
    c = _case(500 + i)
    c.update(D=64, kind="fp8")
    _check_case(fd, c, 500 + i)


def _check_case(fd, c, i):
    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp8": torch.bfloat16, "fp32": torch.float32}[c["kind"]]
    wl = fd.utils.make_paged_workload(f"rand{i}", c["lens"], c["Hq"], c["Hkv"], c["D"], c["P"], dtype, c["kv_split"],
                                      seed=7000 + i, soft_cap=c["soft_cap"], fp8_kv=c["kind"] == "fp8", pool_slack_pages=3)
    kw = dict(path=c["path"], waves_per_block=c["waves"], plan_splits=c["plan"])
    if c["variant"] != "intra":
        kw["fuse_combine"] = c["fuse"]
    ref, ref_lse = oracle_decode(wl)
    fp32 = dtype == torch.float32
    if c["variant"] == "intra":
        g = wl.to("cuda:0")
        if g.k_scale is not None:
            kw.update(k_scale=g.k_scale, v_scale=g.v_scale)
        res = fd.gqa_fwd_batch_decode_intra_rank(g.q, g.k_cache, g.v_cache, None, None, g.kv_lens, g.block_table, g.scale,
                                                 g.soft_cap, kv_split=g.kv_split, **kw)
        torch.cuda.synchronize()
        out, lse = res[..., :c["D"]].cpu(), res[..., c["D"]].float().cpu()
        lse_rtol = 1e-5 if fp32 else 1e-2      # the LSE column has the output's dtype
    else:
        out, lse = run_decode(fd, wl, variant=c["variant"], **kw)
        lse_rtol = 1e-5 if fp32 else 1e-3
    assert_out_close(out, ref, atol=2e-4 if fp32 else 2e-2)
    assert_lse_close(lse, ref_lse, rtol=lse_rtol)


# ---- second sweep: batches up to 80 sequences in block tables wider than the sequences (garbage beyond the used
# pages), the library's own split count, length hints, the item scheduler, groups up to 40 query heads
SERVING_CASES = 100


def _serving_case(i):
    rng = random.Random(12000 + i)
    D = rng.choice([64, 128, 128, 128, 256])
    kind = rng.choice(["bf16", "fp16", "fp8"]) if D != 64 else rng.choice(["bf16", "fp16"])
    Hkv = rng.choice([1, 2, 4, 8])
    G = rng.choice([1, 4, 4, 7, 8, 16, 24, 40]) if D == 128 else rng.choice([1, 4, 8])
    B = rng.choice([1, 2, 6, 17, 40, 80])
    P = rng.choice([1, 16, 16, 64])
    top = rng.choice([40, 700, 3000])
    lens = [rng.choice([0, 1, 63, 64, 65, 1023, 1024, 1025]) if rng.random() < 0.3 else rng.randint(1, top)
            for _ in range(B)]
    lens[0] = max(lens[0], 1)
    widen = rng.choice([1, 1, 8, 64, 700])
    hint = rng.choice([None, None, "exact", "low", "high"])
    return dict(D=D, kind=kind, Hq=Hkv * G, Hkv=Hkv, P=P, lens=lens, widen=widen, hint=hint,
                kv_split=rng.choice([-1, -1, 32, 4]), variant=rng.choice(["plain", "persistent", "persistent"]),
                soft_cap=rng.choice([0.0, 0.0, 50.0]))


@pytest.mark.parametrize("i", range(SERVING_CASES))
def test_random_serving_shape(fd, i):
    c = _serving_case(i)
    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp8": torch.bfloat16}[c["kind"]]
    wl = fd.utils.make_paged_workload(f"serve{i}", c["lens"], c["Hq"], c["Hkv"], c["D"], c["P"], dtype, c["kv_split"],
                                      seed=15000 + i, soft_cap=c["soft_cap"], fp8_kv=c["kind"] == "fp8")
    used = wl.block_table.shape[1]
    gen = torch.Generator().manual_seed(i)
    wide = torch.randint(-9, 1 << 28, (len(c["lens"]), used * c["widen"]), generator=gen, dtype=torch.int32)
    for b, n in enumerate(c["lens"]):
        pages = -(-n // c["P"])
        wide[b, :pages] = wl.block_table[b, :pages]
    wl.block_table = wide
    kw = {}
    if c["hint"] is not None:
        kw["max_kv_len"] = {"exact": max(c["lens"]), "low": max(1, max(c["lens"]) // 3), "high": 10 ** 7}[c["hint"]]
    ref, ref_lse = oracle_decode(wl)
    out, lse = run_decode(fd, wl, variant=c["variant"], **kw)
    assert_out_close(out, ref, atol=2e-2)
    assert_lse_close(lse, ref_lse, rtol=1e-3)


# ---- third sweep: exactly the caller's split count on head_dim 128 with sequences long enough for chunked work items
# (a workgroup walks several splits, a wave parks finished or raw partials in LDS): internal partials and
# caller-visible [B, Hq, S, D + 1] buffers of every element type, groups up to 32 query heads
EXACT_CASES = 60


def _exact_case(i):
    rng = random.Random(21000 + i)
    kind = rng.choice(["bf16", "fp16", "fp8"])
    Hkv = rng.choice([1, 2, 4, 8])
    G = rng.choice([1, 4, 4, 8, 8, 16, 20, 32])
    B = rng.choice([1, 2, 3, 8, 9])
    P = rng.choice([1, 16, 16, 64])
    top = rng.choice([600, 3000, 9000])
    lens = [rng.choice([0, 1, 63, 64, 65, 2047, 2048, 2049]) if rng.random() < 0.25 else rng.randint(1, top)
            for _ in range(B)]
    lens[0] = max(lens[0], top // 2)
    return dict(kind=kind, Hq=Hkv * G, Hkv=Hkv, P=P, lens=lens, kv_split=rng.choice([2, 3, 7, 16, 24, 32, 64]),
                soft_cap=rng.choice([0.0, 0.0, 30.0]), visible=rng.choice([None, None, "f32", "bf16", "f16"]),
                offset=rng.random() < 0.3, variant=rng.choice(["plain", "plain", "persistent"]))


@pytest.mark.parametrize("i", range(EXACT_CASES))
def test_random_exact_split_shape(fd, i):
    c = _exact_case(i)
    D = 128
    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp8": torch.bfloat16}[c["kind"]]
    wl = fd.utils.make_paged_workload(f"exact{i}", c["lens"], c["Hq"], c["Hkv"], D, c["P"], dtype, c["kv_split"],
                                      seed=23000 + i, soft_cap=c["soft_cap"], fp8_kv=c["kind"] == "fp8")
    ref, ref_lse = oracle_decode(wl)
    kw, mid = {}, None
    lse_rtol, rms_rtol, max_rtol = 1e-3, 1e-2, 2e-2
    if c["visible"] is None:
        kw["plan_splits"] = False
    else:
        mdt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[c["visible"]]
        B, S = len(c["lens"]), c["kv_split"]
        n = B * c["Hq"] * S * (D + 1)
        flat = torch.full((n + 1,), float("nan"), dtype=mdt, device="cuda:0")
        # (some buffers start one element past an aligned address)
        mid = (flat[1:] if c["offset"] else flat[:n]).view(B, c["Hq"], S, D + 1)
        kw["output_split"] = mid
        if mdt != torch.float32:
            lse_rtol = 1e-2   # the partial LSEs are held in 16 bits as well ...
        if mdt == torch.bfloat16:
            # ... in bf16 with 8 bits of mantissa: an LSE near 9 is off by up to 0.02, and so are the merge weights
            rms_rtol, max_rtol = 3e-2, 6e-2
    out, lse = run_decode(fd, wl, variant=c["variant"], **kw)   # persistent: (sequence, range) items in issue order
    if mid is not None:
        assert not torch.isnan(mid).any(), "a partial slot was not written"
    assert_out_close(out, ref, atol=2e-2, rel=False)
    assert_out_rel(out, ref, rms_rtol=rms_rtol, max_rtol=max_rtol)
    assert_lse_close(lse, ref_lse, rtol=lse_rtol)
