"""Timing helper and seeded synthetic workloads for the flash-decode path.

``perf_func`` keeps the reference's measurement method
(``python/triton_dist/utils.py:269-281``): events around ``iters`` back-to-back
calls after ``warmup_iters`` warm-up calls, mean milliseconds per call.

The workload builders generate every tensor on the CPU from a fixed
``torch.Generator`` seed, so a CPU checker and the GPU kernels can be fed
identical bits; ``.to(device)`` moves a workload.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Dict, List, Optional, Tuple

import torch


def perf_func(func, iters, warmup_iters):
    """``(last result, mean milliseconds per call)`` of ``iters`` back-to-back calls after ``warmup_iters`` untimed
    ones, timed by two events on the current stream -- the reference's method and signature (utils.py:269-281)."""
    result = None
    for _ in range(warmup_iters):
        result = func()
    begin, end = (torch.cuda.Event(enable_timing=True) for _ in range(2))
    begin.record()
    for _ in range(iters):
        result = func()
    end.record()
    end.synchronize()
    return result, begin.elapsed_time(end) / iters


@dataclasses.dataclass
class DecodeWorkload:
    """One decode step's inputs.  K/V caches are ``[num_pages, P, Hkv, D]``."""
    name: str
    q: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    kv_lens: torch.Tensor            # int32 [B]
    block_table: torch.Tensor        # int32 [B, max_pages]
    scale: float
    kv_split: int
    soft_cap: float = 0.0
    k_scale: Optional[torch.Tensor] = None    # fp32 [Hkv] (fp8 cache only)
    v_scale: Optional[torch.Tensor] = None
    extra_out: Optional[torch.Tensor] = None  # [E, B, Hq, D] partials of other ranks
    extra_lse: Optional[torch.Tensor] = None  # [E, B, Hq] fp32

    def to(self, device) -> "DecodeWorkload":
        kw = {}
        for f in dataclasses.fields(self):
            v = getattr(self, f.name)
            kw[f.name] = v.to(device) if isinstance(v, torch.Tensor) else v
        return DecodeWorkload(**kw)

    @property
    def shape(self) -> Dict[str, int]:
        B, Hq, D = self.q.shape
        _, P, Hkv, _ = self.k_cache.shape
        return dict(B=B, Hq=Hq, Hkv=Hkv, D=D, P=P, S=self.kv_split)

    def algorithmic_bytes(self, out_itemsize: Optional[int] = None) -> int:
        """Compulsory HBM traffic of one decode step: every referenced K/V token once, Q, the used
        block-table entries, kv_lens, the final output and its fp32 LSE (+ fp8 scales, + the extra
        partials read by the combine).  Split workspaces are implementation overhead and excluded."""
        B, Hq, D = self.q.shape
        _, P, Hkv, Dv = self.v_cache.shape
        lens = [int(x) for x in self.kv_lens.tolist()]
        kv_item = self.k_cache.element_size()
        out_item = out_itemsize if out_itemsize is not None else self.q.element_size()
        total = sum(lens) * Hkv * (D + Dv) * kv_item
        total += B * Hq * D * self.q.element_size()
        total += sum(-(-n // P) for n in lens) * 4 + B * 4
        total += B * Hq * Dv * out_item + B * Hq * 4
        if self.k_scale is not None:
            total += 2 * Hkv * 4
        if self.extra_out is not None:
            E = self.extra_out.shape[0]
            total += E * (B * Hq * Dv * self.extra_out.element_size() + B * Hq * 4)
        return total

    def flops(self) -> int:
        B, Hq, D = self.q.shape
        Dv = self.v_cache.shape[-1]
        return sum(int(x) for x in self.kv_lens.tolist()) * Hq * (2 * D + 2 * Dv)


def _randn(gen, shape, dtype):
    return torch.randn(shape, generator=gen, dtype=torch.float32).to(dtype)


def make_paged_workload(name: str, kv_lens: List[int], Hq: int, Hkv: int, D: int, P: int, dtype: torch.dtype,
                        kv_split: int, seed: int, soft_cap: float = 0.0, fp8_kv: bool = False,
                        pool_slack_pages: int = 0, shuffle: bool = True,
                        kv_value_scale: float = 1.0) -> DecodeWorkload:
    """Shuffled paged cache: one global ``randperm`` of the pool sliced per sequence.

    fp8_kv: K/V ~ N(0,1) are quantised to OCP e4m3 with per-KV-head scales absmax/448.
    """
    gen = torch.Generator(device="cpu").manual_seed(seed)
    B = len(kv_lens)
    pages_per_seq = [-(-n // P) for n in kv_lens]
    max_pages = max(1, max(pages_per_seq))
    num_pages = max(1, sum(pages_per_seq)) + pool_slack_pages
    q = _randn(gen, (B, Hq, D), dtype)
    k_src = torch.randn((num_pages, P, Hkv, D), generator=gen, dtype=torch.float32) * kv_value_scale
    v_src = torch.randn((num_pages, P, Hkv, D), generator=gen, dtype=torch.float32) * kv_value_scale
    perm = torch.randperm(num_pages, generator=gen) if shuffle else torch.arange(num_pages)
    block_table = torch.zeros((B, max_pages), dtype=torch.int32)
    off = 0
    for b, n in enumerate(pages_per_seq):
        block_table[b, :n] = perm[off:off + n].to(torch.int32)
        off += n
    k_scale = v_scale = None
    if fp8_kv:
        def quant(x):
            absmax = x.abs().amax(dim=(0, 1, 3)).clamp_min(1e-12)
            s = (absmax / 448.0).to(torch.float32)
            return (x / s.view(1, 1, -1, 1)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn), s
        k_cache, k_scale = quant(k_src)
        v_cache, v_scale = quant(v_src)
    else:
        k_cache, v_cache = k_src.to(dtype), v_src.to(dtype)
    return DecodeWorkload(name=name, q=q, k_cache=k_cache, v_cache=v_cache,
                          kv_lens=torch.tensor(kv_lens, dtype=torch.int32), block_table=block_table,
                          scale=1.0 / math.sqrt(D), kv_split=kv_split, soft_cap=soft_cap, k_scale=k_scale,
                          v_scale=v_scale)


def make_config(idx: int, scale_down: int = 1) -> DecodeWorkload:
    """The five benchmark/parity configurations (seed = 1000 + idx).

    ``scale_down`` divides the KV lengths (and config 4's batch) so that a CPU checker finishes in
    seconds; 1 gives the full-size workload.
    """
    seed = 1000 + idx
    if idx == 1:   # plumbing: contiguous fp32 cache, one page of kv_len tokens, 4 splits
        n = 1024 // scale_down
        return make_paged_workload("config1_fp32_contiguous", [n], 8, 2, 128, n, torch.float32, 4, seed, shuffle=False)
    if idx == 2:   # Llama-3-8B shape
        n = 8192 // scale_down
        return make_paged_workload("config2_llama3_8b_b8_kv8192", [n] * 8, 32, 8, 128, 16, torch.bfloat16, 32, seed)
    if idx == 3:   # one GPU's shard of a 1M-token context + 7 partials of the other ranks
        n = 131072 // scale_down
        wl = make_paged_workload("config3_sp_shard_131072", [n], 32, 8, 128, 16, torch.bfloat16, 32, seed)
        gen = torch.Generator(device="cpu").manual_seed(seed + 500)
        wl.extra_out = torch.randn((7, 1, 32, 128), generator=gen, dtype=torch.float32).to(torch.bfloat16)
        wl.extra_lse = torch.rand((7, 1, 32), generator=gen, dtype=torch.float32) * 10.0 + 5.0
        return wl
    if idx == 4:   # ragged continuous batching
        gen = torch.Generator(device="cpu").manual_seed(seed + 500)
        B = max(2, 64 // scale_down)
        lens = torch.randint(512 // scale_down, 32768 // scale_down + 1, (B,), generator=gen).tolist()
        return make_paged_workload("config4_ragged_b64", lens, 32, 8, 128, 16, torch.bfloat16, 32, seed,
                                   pool_slack_pages=64)
    if idx == 5:   # fp8 KV cache
        n = 16384 // scale_down
        B = max(1, 32 // scale_down)
        return make_paged_workload("config5_fp8_kv", [n] * B, 64, 8, 128, 16, torch.bfloat16, 64, seed, fp8_kv=True)
    raise ValueError(f"unknown config {idx}")


def make_config5_bf16_twin(scale_down: int = 1) -> DecodeWorkload:
    """Config 5's shape with a bf16 cache, for the fp8-vs-bf16 speed ratio."""
    n = 16384 // scale_down
    B = max(1, 32 // scale_down)
    return make_paged_workload("config5_bf16_twin", [n] * B, 64, 8, 128, 16, torch.bfloat16, 64, 1005)
