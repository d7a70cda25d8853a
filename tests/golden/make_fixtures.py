"""Writes the golden fixtures of the flash-decode path (tests/golden/*.npz).

The reference holds no golden vectors, known-answer files or fixtures for this path (its tests
compare against a PyTorch oracle on random inputs), so these vectors are produced by this
repository's own CPU oracle (oracle/ref_decode.py), which tests/test_oracle_pinning.py pins against
closed forms, torch SDPA and a scalar float64 brute force.  Nothing from the reference tree is
imported or executed.  Inputs are stored as raw bit patterns (uint16 for fp16/bf16, uint8 for
fp8-e4m3) so that loading them involves no rounding.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402

BITS = {torch.float16: torch.int16, torch.bfloat16: torch.int16}


def to_bits(t):
    if t.dtype in BITS:
        return t.view(BITS[t.dtype]).numpy().view(np.uint16)
    return t.numpy()


def make(name, kv_lens, Hq, Hkv, D, P, dtype, kv_split, seed, soft_cap=0.0, fp8=False, pool_pages=None):
    g = torch.Generator().manual_seed(seed)
    B = len(kv_lens)
    maxp = max(1, max(-(-n // P) for n in kv_lens))
    pages = pool_pages or (sum(-(-n // P) for n in kv_lens) + 3)
    q = torch.randn(B, Hq, D, generator=g).to(dtype)
    k = torch.randn(pages, P, Hkv, D, generator=g)
    v = torch.randn(pages, P, Hkv, D, generator=g)
    bt = torch.randint(0, pages, (B, maxp), generator=g, dtype=torch.int32)   # with replacement, like the reference
    rec = dict(kv_lens=np.array(kv_lens, np.int32), block_table=bt.numpy(), scale=np.float32(D ** -0.5),
               soft_cap=np.float32(soft_cap), kv_split=np.int32(kv_split), dtype=str(dtype).replace("torch.", ""),
               q=to_bits(q))
    if fp8:
        kq, ks = oracle.quantize_fp8_cache(k)
        vq, vs = oracle.quantize_fp8_cache(v)
        rec.update(k_cache=kq.numpy(), v_cache=vq.numpy(), k_scale=ks.numpy(), v_scale=vs.numpy(), kv_dtype="fp8_e4m3")
        kf, vf = oracle.dequant_fp8_cache(kq, ks), oracle.dequant_fp8_cache(vq, vs)
    else:
        kc, vc = k.to(dtype), v.to(dtype)
        rec.update(k_cache=to_bits(kc), v_cache=to_bits(vc), kv_dtype=rec["dtype"])
        kf, vf = kc.float(), vc.float()
    out, lse = oracle.ref_paged_attn_lse(q.float(), kf, vf, kv_lens, bt, D ** -0.5, soft_cap=soft_cap)
    rec.update(out=out.numpy(), lse=lse.numpy())
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **rec)
    print(name, {k_: getattr(v_, "shape", v_) for k_, v_ in rec.items()})


if __name__ == "__main__":
    make("plumbing_fp32_contiguous", [64], 8, 2, 128, 64, torch.float32, 4, seed=1, pool_pages=1)
    make("paged_fp16_group4", [70, 18, 1], 8, 2, 128, 16, torch.float16, 32, seed=2)
    make("paged_bf16_group6_softcap", [54, 33], 6, 1, 128, 1, torch.bfloat16, 32, seed=3, soft_cap=30.0)
    make("paged_fp16_mha_d256", [40, 7], 2, 2, 256, 16, torch.float16, 8, seed=4)
    make("paged_fp8_group8", [65, 17], 8, 1, 128, 16, torch.bfloat16, 16, seed=5, fp8=True)
