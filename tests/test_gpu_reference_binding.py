"""The minimal ctypes binding a maintainer of the reference would add (reference_binding.py, a module that imports
nothing from the package) drives the C ABI correctly: decode against the oracle, rotary + cache write bit-exact."""
import importlib.util
import os

import pytest
import torch

import oracle
from helpers import DEV, assert_out_close, oracle_decode

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def binding(fd):
    path = os.path.join(os.path.dirname(os.path.abspath(fd.__file__)), "reference_binding.py")
    spec = importlib.util.spec_from_file_location("fd_reference_binding", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kv_split", [-1, 4])
def test_decode_through_the_binding(fd, binding, dtype, kv_split):
    wl = fd.utils.make_paged_workload("binding", [1320, 18, 463, 2049], 32, 8, 128, 16, dtype, 32, seed=23)
    g = wl.to(DEV)
    out = binding.gqa_fwd_batch_decode(g.q, g.k_cache, g.v_cache, None, [1] * 4, g.kv_lens, g.block_table, g.scale,
                                       kv_split=kv_split)
    torch.cuda.synchronize()
    ref, _ = oracle_decode(wl)
    assert_out_close(out.cpu(), ref)
    # caller-visible partials in the reference layout [B, Hq, S, D + 1]
    S = 8
    mid = torch.full((4, 32, S, 129), float("nan"), dtype=torch.float32, device=DEV)
    res = torch.empty(4, 32, 128, dtype=dtype, device=DEV)
    same = binding.gqa_fwd_batch_decode(g.q, g.k_cache, g.v_cache, None, None, g.kv_lens, g.block_table, g.scale,
                                        output_split=mid, output_combine=res, kv_split=S)
    torch.cuda.synchronize()
    assert same is res
    assert_out_close(res.cpu(), ref)
    assert not torch.isnan(mid[..., 128]).any()


@pytest.mark.parametrize("new_tokens", [1, 5])
def test_rope_and_cache_write_through_the_binding(binding, new_tokens):
    gen = torch.Generator().manual_seed(31)
    B, Hq, Hkv, D, P, T = 3, 8, 2, 128, 16, new_tokens
    lens = torch.tensor([5, 16, 27], dtype=torch.int32)
    bt = torch.randperm(12, generator=gen).to(torch.int32)[:9].view(B, 3)
    q = torch.randn(B, T, Hq, D, generator=gen).to(torch.bfloat16)
    k = torch.randn(B, T, Hkv, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(B, T, Hkv, D, generator=gen).to(torch.bfloat16)
    kc = torch.randn(12, P, Hkv, D, generator=gen).to(torch.bfloat16)
    vc = torch.randn(12, P, Hkv, D, generator=gen).to(torch.bfloat16)
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    tab = oracle.ref_set_cos_sin_cache(inv_freq, 64)
    pos = lens[:, None].long() + torch.arange(T)[None, :]
    ref_k, ref_v = kc.clone(), vc.clone()
    oracle.ref_kv_append(oracle.ref_rope(k, tab, pos), v, ref_k, ref_v, bt, lens)
    ref_q = oracle.ref_rope(q, tab, pos)

    q_g, kc_g, vc_g = q.to(DEV), kc.to(DEV), vc.to(DEV)
    lens_out = torch.zeros(B, dtype=torch.int32, device=DEV)
    binding.rope_and_update_cache(q_g, k.to(DEV), v.to(DEV), kc_g, vc_g, bt.to(DEV), lens.to(DEV), lens_out,
                                  tab.to(DEV), pos.to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(lens_out.cpu(), lens + T)
    assert torch.equal(q_g.cpu().view(torch.int16), ref_q.view(torch.int16))
    assert torch.equal(kc_g.cpu().view(torch.int16), ref_k.view(torch.int16))
    assert torch.equal(vc_g.cpu().view(torch.int16), ref_v.view(torch.int16))
