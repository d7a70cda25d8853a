"""Writes the golden fixtures of the write side (tests/golden/write_side/*.npz): rotary embedding, per-head RMS
norm, paged KV append and fp8 quantisation.

The reference holds no vectors for these steps, so the expected outputs come from this repository's CPU oracle
(oracle/ref_kv_append.py), which tests/test_oracle_pinning.py pins against closed forms, a library routine and a
brute-force search.  Nothing from the reference tree is imported or executed.  16-bit tensors are stored as raw
bit patterns.

    python tests/golden/write_side/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(HERE))))
import oracle  # noqa: E402


def to_bits(t):
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


def make(name, lens, T, Hq, Hkv, D, P, dtype, seed, fp8=False, norm=False, rope=True):
    g = torch.Generator().manual_seed(seed)
    B = len(lens)
    pages_per_seq = max(-(-(n + T) // P) for n in lens)
    pages = B * pages_per_seq + 2
    bt = torch.randperm(pages, generator=g)[:B * pages_per_seq].to(torch.int32).view(B, pages_per_seq)
    q = torch.randn(B, T, Hq, D, generator=g).to(dtype)
    k = torch.randn(B, T, Hkv, D, generator=g).to(dtype)
    v = torch.randn(B, T, Hkv, D, generator=g).to(dtype)
    kv_lens = torch.tensor(lens, dtype=torch.int32)
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    tab = oracle.ref_set_cos_sin_cache(inv_freq, 64)
    pos = (kv_lens[:, None] + torch.arange(T)).long()
    rec = dict(dtype=str(dtype).replace("torch.", ""), kv_lens=kv_lens.numpy(), block_table=bt.numpy(), page_size=np.int32(P),
               q=to_bits(q), k=to_bits(k), v=to_bits(v), fp8=np.bool_(fp8), norm=np.bool_(norm), rope=np.bool_(rope))
    qq, kk = q, k
    if norm:
        qw = (1 + 0.25 * torch.randn(D, generator=g)).to(dtype)
        kw = (1 + 0.25 * torch.randn(D, generator=g)).to(dtype)
        rec.update(q_norm_weight=to_bits(qw), k_norm_weight=to_bits(kw), norm_eps=np.float32(1e-6))
        qq, kk = oracle.ref_rms_norm(q, qw, 1e-6), oracle.ref_rms_norm(k, kw, 1e-6)
    if rope:
        rec.update(cos_sin=tab.numpy(), position_ids=pos.numpy())
        qq, kk = oracle.ref_rope(qq, tab, pos), oracle.ref_rope(kk, tab, pos)
    if fp8:
        kc = torch.randint(0, 120, (pages, P, Hkv, D), generator=g).to(torch.uint8)
        vc = torch.randint(0, 120, (pages, P, Hkv, D), generator=g).to(torch.uint8)
        ks = (kk.float().abs().amax(dim=(0, 1, 3)) / 448.0).contiguous()
        vs = (v.float().abs().amax(dim=(0, 1, 3)) / 300.0).contiguous()      # some V values saturate
        rec.update(k_scale=ks.numpy(), v_scale=vs.numpy())
    else:
        kc = torch.randn(pages, P, Hkv, D, generator=g).to(dtype)
        vc = torch.randn(pages, P, Hkv, D, generator=g).to(dtype)
        ks = vs = None
    rec.update(k_cache_before=to_bits(kc), v_cache_before=to_bits(vc))
    grown = oracle.ref_kv_append(kk, v, kc, vc, bt, kv_lens, ks, vs)
    rec.update(q_out=to_bits(qq), k_cache_after=to_bits(kc), v_cache_after=to_bits(vc), kv_lens_out=grown.numpy())
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **rec)
    print(name, {k_: getattr(v_, "shape", v_) for k_, v_ in rec.items()})


if __name__ == "__main__":
    make("rope_append_bf16", [0, 5, 16, 31], 1, 8, 2, 128, 16, torch.bfloat16, seed=1)
    make("rope_append_fp16_d64_page1_t3", [2, 0, 9], 3, 4, 4, 64, 1, torch.float16, seed=2)
    make("rope_append_bf16_fp8_cache", [7, 15, 40], 2, 16, 2, 128, 16, torch.bfloat16, seed=3, fp8=True)
    make("norm_rope_append_bf16_d256", [3, 12], 1, 4, 1, 256, 8, torch.bfloat16, seed=4, norm=True)
    make("append_only_fp32", [1, 30], 2, 2, 2, 128, 16, torch.float32, seed=5, rope=False)
