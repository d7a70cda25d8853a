#!/usr/bin/env python3
"""Flash-decode benchmark: one decode step = split-KV GQA paged decode + LSE combine on one MI355X.

    python bench.py [--gpus 1] [--steps 100] [--warmup 20] [--config 2]

Prints ONE JSON line.  ``value`` is microseconds per decode step with all inputs resident in
HBM; the step rotates over several independent KV pools so the 256 MB Infinity Cache cannot
serve the working set.  ``roofline`` prices the split-KV kernel (the dominant one) against
the 8 TB/s HBM peak with the algorithmic bytes of a step; ``cpu_baseline`` is the CPU oracle
(the reference's PyTorch decode restated) timed on this host's cores on the same inputs.
"""
from __future__ import annotations

import argparse
import importlib
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration 1-5 (2 = Llama-3-8B shape, the one the metric is quoted on)")
    ap.add_argument("--pools", type=int, default=4, help="independent KV pools the steps rotate over")
    ap.add_argument("--clock-ramp-ms", type=float, default=250.0,
                    help="least untimed run of the step before the warm-up steps (until its time has settled, at "
                         "most 20 times as long), so that an idle or just vacated GPU is in its steady state")
    ap.add_argument("--variant", default="plain", choices=["plain", "persistent"])
    ap.add_argument("--path", default="auto", choices=["auto", "valu", "mfma"])
    ap.add_argument("--waves", type=int, default=0)
    ap.add_argument("--fuse", action="store_true", help="fuse the combine into the tail of the split kernel")
    ap.add_argument("--kv-split", type=int, default=0,
                    help="override the workload's kv_split (experiments); -1: the library's own choice")
    ap.add_argument("--exact-splits", action="store_true",
                    help="use exactly the workload's kv_split splits instead of the library's plan (fd_plan_splits)")
    ap.add_argument("--caller-partials", default=None, choices=["fp32", "fp16", "bf16"],
                    help="the caller hands in output_split [B, Hq, S, D + 1] of this type, as the reference's perf "
                         "scripts and its sequence-parallel layer do: exactly kv_split observable partials")
    ap.add_argument("--launch-decomposition", action="store_true",
                    help="also time, as HIP-graph replays (no host in the loop): the split kernel alone, split + combine, "
                         "split + a 64-element fill kernel, and that fill kernel alone -- what the second launch of a "
                         "step costs whatever it computes")
    ap.add_argument("--no-graph", action="store_true", help="skip the HIP-graph replay of the step")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-targets", action="store_true",
                    help="skip the other north-star figures (exact split counts, configs 3, 4, 5) that the default "
                         "run measures besides the headline")
    ap.add_argument("--no-write-side", action="store_true",
                    help="skip the timing of the step before the decode (rotary + KV append)")
    ap.add_argument("--cpu-seqs", type=int, default=0, help="sequences the CPU baseline times (0 = choose)")
    ap.add_argument("--bf16-twin", action="store_true", help="config 5's shape with a bf16 cache")
    ap.add_argument("--shape", default=None,
                    help="B,kv_len,Hq,Hkv,D,P[,bf16|fp16|fp8]: a uniform batch of another shape instead of a numbered "
                         "config (secondary measurements: other head dims, groups, batch sizes)")
    ap.add_argument("--copy-ref", action="store_true",
                    help="also run a plain 256 MiB device copy a few times: a kernel of known traffic against which "
                         "a counter run (FETCH_SIZE / WRITE_SIZE) of this same command is scaled")
    ap.add_argument("--traffic-json", default=None,
                    help="JSON file {\"traffic\": bytes per split-kernel launch} measured with the counter runs; "
                         "copied into roofline.traffic")
    return ap.parse_args()


def _time_us(torch, fn, steps, warmup):
    """GPU time per call of fn over `steps` back-to-back calls (HIP events on the current stream).  One untimed
    lead-in call sits between the synchronize and the first event: the device is busy with it while the host queues
    the first event and the first timed calls, so the region holds `steps` calls back to back and not also the
    host's latency of the first launch after an idle queue (about 14 us, i.e. +0.7 us per call at 20 calls)."""
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    fn(-1)
    e0.record()
    for i in range(steps):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / steps


def make_pools(torch, wl, dev, n):
    """Independent KV pools for the steps to rotate over: pool 0 holds the seeded data (the one checked against
    the CPU baseline), the others other random bits of the same distribution."""
    pools = [(wl.k_cache, wl.v_cache)]
    for _ in range(1, max(1, n)):
        if wl.k_cache.dtype in (torch.float16, torch.bfloat16, torch.float32):
            k = torch.empty_like(wl.k_cache).normal_()
            v = torch.empty_like(wl.v_cache).normal_()
        else:  # fp8 bit patterns: shuffle pages of pool 0
            perm = torch.randperm(wl.k_cache.shape[0], device=dev)
            k = wl.k_cache[perm].contiguous()
            v = wl.v_cache[perm].contiguous()
        pools.append((k, v))
    return pools


def _flash_decode(fd):
    return importlib.import_module(fd.__name__ + ".kernels.flash_decode")


def make_step(torch, fd, wl, pools, S, dev, variant="plain", exact=False, path="auto", waves=0, fuse=False,
              caller_partials=None, auto_order=True):
    """The decode step of a workload as a callable of the step index, plus its output and LSE tensors.
    caller_partials: a dtype -- the caller hands in ``output_split [B, Hq, S, D + 1]`` of that type, as the reference's
    sequence-parallel layer does on every call (sp_flash_decode_layer.py:95-110): exactly S observable partials."""
    B, Hq, D = wl.q.shape
    out = torch.empty(B, Hq, D, dtype=wl.q.dtype, device=dev)
    lse = torch.empty(B, Hq, dtype=torch.float32, device=dev)
    # the workspace the library asks for (partials, their LSEs, the issue order): with it the step allocates nothing
    fk, L = _flash_decode(fd), fd._lib
    flags = (L.FD_STEP_EXACT_SPLITS if exact else 0) | (L.FD_STEP_SCHEDULE if variant == "persistent" else 0) \
        | (0 if auto_order else L.FD_STEP_NO_ORDER) | (L.FD_STEP_FUSED if fuse else 0)
    need = fk.workspace_bytes(wl.q, wl.k_cache, wl.block_table, S, flags=flags, fp8=wl.k_scale is not None, path=path,
                              waves_per_block=waves, num_extra=0 if wl.extra_out is None else wl.extra_out.shape[0])
    workspace = torch.empty(max(need, 4) // 4 + 64, dtype=torch.float32, device=dev)
    q_lens = [1] * B
    kw = dict(output_combine=out, kv_split=S, lse_out=lse, path=path, waves_per_block=waves, fuse_combine=fuse)
    if not auto_order:
        kw["auto_order"] = False
    if wl.k_scale is not None:
        kw.update(k_scale=wl.k_scale, v_scale=wl.v_scale)
    if wl.extra_out is not None:
        kw.update(extra_partials=(wl.extra_out, wl.extra_lse))
    if exact:
        kw["plan_splits"] = False
    if caller_partials is not None:
        kw["output_split"] = torch.empty(B, Hq, S, D + 1, dtype=caller_partials, device=dev)
    fn = fd.gqa_fwd_batch_decode_persistent if variant == "persistent" else fd.gqa_fwd_batch_decode

    def step(i):   # persistent: the scheduling launch is part of the step (inside the wrapper)
        k, v = pools[i % len(pools)]
        return fn(wl.q, k, v, workspace, q_lens, wl.kv_lens, wl.block_table, wl.scale, wl.soft_cap, **kw)
    return step, out, lse, workspace


def settle(torch, step, ramp_ms):
    """An idle GPU takes a while to reach its clocks, and a machine on which a process has just released tens of GiB
    of device memory is busy with that for a few seconds more (measured: the first run after such a process read 5 %
    slow, the same command seconds later did not).  Runs the step untimed, in batches timed with events, until the
    batch time has settled (three batches in a row within 1 % of the best one) -- at least ramp_ms, at most 20 times
    that.  Returns the milliseconds spent."""
    t_ramp = time.perf_counter()
    i_ramp, best, settled = 0, float("inf"), 0
    r0, r1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    while ramp_ms > 0:
        r0.record()
        for _ in range(100):
            step(i_ramp)
            i_ramp += 1
        r1.record()
        torch.cuda.synchronize()
        took = r0.elapsed_time(r1)
        settled = settled + 1 if 0.99 * best <= took <= 1.01 * best else 0
        best = min(best, took)
        waited_ms = (time.perf_counter() - t_ramp) * 1e3
        if (waited_ms >= ramp_ms and settled >= 3) or waited_ms >= 20 * ramp_ms:
            break
    return (time.perf_counter() - t_ramp) * 1e3


def measure_target(torch, fd, dev, wl_cpu, steps, warmup, pools_n, ramp_ms, resident=None, step_factory=None,
                   **step_kw):
    """One north-star target measured the way the headline is: the whole decode step (split + combine) of a
    workload, rotating over independent pools, after the clocks have settled.  Its pools go back to torch's
    caching allocator, not to the driver: a GPU that has just been handed back gigabytes is slow for a few seconds
    (the next target measured up to 4 % slow that way)."""
    if resident is not None:   # (workload, pools) that are on the GPU already
        wl, pools = resident
    else:
        wl = wl_cpu.to(dev)
        pools = make_pools(torch, wl, dev, pools_n)
    if step_factory is not None:   # another caller of the path: step_factory(workload, pools) -> step(i)
        step = step_factory(wl, pools)
    else:
        step, _, _, _ = make_step(torch, fd, wl, pools, wl.kv_split, dev, **step_kw)
    settle(torch, step, ramp_ms)
    us = _time_us(torch, step, steps, warmup)
    nbytes = wl_cpu.algorithmic_bytes()
    return round(us, 3), round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)


def _binding_step(torch, fd, dev, caller_partials):
    """The decode step through ``reference_binding.gqa_fwd_batch_decode`` (positional reference signature)."""
    import importlib.util
    path = os.path.join(os.path.dirname(os.path.abspath(fd.__file__)), "reference_binding.py")
    spec = importlib.util.spec_from_file_location("fd_reference_binding_bench", path)
    rb = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(rb)

    def factory(wl, pools):
        B, Hq, D = wl.q.shape
        S = wl.kv_split
        out_split = torch.empty(B, Hq, S, D + 1, dtype=torch.float32, device=dev)
        out = torch.empty(B, Hq, D, dtype=wl.q.dtype, device=dev)
        q_lens = [1] * B

        need = rb._lib.fd_workspace_bytes(__import__("ctypes").byref(rb.FdParams(
            Hq, wl.k_cache.shape[2], D, wl.k_cache.shape[1], S, wl.k_cache.shape[0], wl.block_table.shape[1],
            rb._DT[wl.q.dtype], rb._DT[wl.k_cache.dtype], 0, rb._DT[out.dtype])), B, 0, 0)
        workspace = torch.empty(max(int(need), 256), dtype=torch.uint8, device=dev)

        def step(i):
            k, v = pools[i % len(pools)]
            if caller_partials:   # as the perf scripts and the sequence-parallel layer call it (test_decode_attn.py:322-331)
                return rb.gqa_fwd_batch_decode(wl.q, k, v, None, q_lens, wl.kv_lens, wl.block_table, wl.scale,
                                               wl.soft_cap, out_split, out, S)
            # as the reference's tests call it (test_decode_attn.py:158): no output_split, the library plans
            return rb.gqa_fwd_batch_decode(wl.q, k, v, workspace, q_lens, wl.kv_lens, wl.block_table, wl.scale,
                                           wl.soft_cap, None, out, S)
        return step
    return factory


def _sp_layer_step(torch, fd, dev, reference_settings):
    """``SpGQAFlashDecodeAttention(num_ranks=8).forward`` on one rank's shard with the other ranks' partials given."""
    def factory(wl, pools):
        B, Hq, D = wl.q.shape
        _, P, Hkv, _ = wl.k_cache.shape
        R = wl.extra_out.shape[0] + 1
        layer = fd.SpGQAFlashDecodeAttention(0, 0, R, 1, Hq, Hkv, D, D, page_size=P, scale=wl.scale,
                                             soft_cap=wl.soft_cap, max_allowed_batch=B,
                                             **({"partial_dtype": None} if reference_settings else {}))
        out_split = None
        if reference_settings:
            layer.kv_split = 32                                    # sp_flash_decode_layer.py:62
            out_split = torch.empty(B, Hq, 32, D + 1, dtype=wl.q.dtype, device=dev)   # :95-96
        lens = torch.ones(R, B, dtype=torch.int32, device=dev)
        lens[0] = wl.kv_lens
        remote = (wl.extra_out, wl.extra_lse)

        def step(i):
            k, v = pools[i % len(pools)]
            return layer(wl.q, k, v, lens, wl.block_table, remote_partials=remote, output_split=out_split)
        return step
    return factory


def measure_targets(torch, fd, dev, steps, warmup, c2_resident):
    """Every north-star figure besides the headline, in this same process, each as (microseconds per decode step,
    fraction of the 8 TB/s peak on the step's algorithmic bytes): config 2 with exactly the 32 splits the workload
    names; config 5 (fp8 KV) and its bf16 twin, planned and with exactly 64 splits, and their ratios (target >= 1.7);
    config 3, planned and with exactly 32 splits; config 4 scheduled, through the plain wrapper and unscheduled."""
    U = fd.utils
    t = {}
    # the headline times exactly the steps the command line asks for; these side figures take at least 100 steps and
    # 20 warm-up steps each (a 20-step region of 1 ms reads about 1 % long)
    steps, warmup = max(steps, 100), max(warmup, 20)

    def put(key, res):
        t[key + "_us"], t[key + "_frac"] = res

    # config 2 on the very pools the headline was measured on (the same memory: where a process's allocations lie
    # decides how far the address translation reaches, which is worth a few per cent at this size)
    put("c2_exact_32_splits", measure_target(torch, fd, dev, U.make_config(2), steps, warmup, 4, 100.0,
                                             resident=c2_resident, exact=True))
    # the reference's literal call: the caller owns the partials, [B, Hq, 32, D + 1] (sp_flash_decode_layer.py:95-110
    # allocates them in q.dtype; the perf scripts in fp32, test_decode_attn.py:322) -- exactly 32 observable partials
    put("c2_caller_partials_fp32", measure_target(torch, fd, dev, U.make_config(2), steps, warmup, 4, 100.0,
                                                  resident=c2_resident, caller_partials=torch.float32))
    put("c2_caller_partials_bf16", measure_target(torch, fd, dev, U.make_config(2), steps, warmup, 4, 100.0,
                                                  resident=c2_resident, caller_partials=torch.bfloat16))
    # ... and through the stand-alone ctypes binding a maintainer of the reference tree would add (nothing of this
    # package's Python between the call and the library): without output_split, as the reference's tests call it --
    # the library plans the step -- and with fp32 partials of the caller's own, as its perf scripts do
    put("c2_reference_binding", measure_target(torch, fd, dev, U.make_config(2), steps, warmup, 4, 100.0,
                                               resident=c2_resident, step_factory=_binding_step(torch, fd, dev, False)))
    put("c2_reference_binding_caller_partials",
        measure_target(torch, fd, dev, U.make_config(2), steps, warmup, 4, 100.0, resident=c2_resident,
                       step_factory=_binding_step(torch, fd, dev, True)))
    c5, c5t = U.make_config(5), U.make_config5_bf16_twin()
    put("c5_caller_partials_bf16", measure_target(torch, fd, dev, c5, steps, warmup, 4, 100.0,
                                                  caller_partials=torch.bfloat16))
    put("c5_fp8", measure_target(torch, fd, dev, c5, steps, warmup, 4, 100.0))
    put("c5_fp8_exact_64_splits", measure_target(torch, fd, dev, c5, steps, warmup, 4, 100.0, exact=True))
    put("c5_bf16_twin", measure_target(torch, fd, dev, c5t, steps, warmup, 4, 100.0))
    put("c5_bf16_twin_exact_64_splits", measure_target(torch, fd, dev, c5t, steps, warmup, 4, 100.0, exact=True))
    t["c5_bf16_over_fp8"] = round(t["c5_bf16_twin_us"] / t["c5_fp8_us"], 3)
    t["c5_bf16_over_fp8_exact_64_splits"] = round(t["c5_bf16_twin_exact_64_splits_us"] / t["c5_fp8_exact_64_splits_us"], 3)
    del c5, c5t
    c3 = U.make_config(3)
    put("c3_sp_shard_plus_7_partials", measure_target(torch, fd, dev, c3, steps, warmup, 4, 100.0))
    put("c3_exact_32_splits", measure_target(torch, fd, dev, c3, steps, warmup, 4, 100.0, exact=True))
    # the caller of the path: SpGQAFlashDecodeAttention.forward on this shard as rank 0 of 8, the 7 seeded partials
    # standing in for what the other ranks' allgather would deliver -- with the layer's defaults, and with the
    # reference's settings (32 splits, partials visible to the caller and staged in q.dtype)
    put("c3_sp_layer_forward", measure_target(torch, fd, dev, c3, steps, warmup, 4, 100.0,
                                              step_factory=_sp_layer_step(torch, fd, dev, False)))
    put("c3_sp_layer_forward_reference_settings",
        measure_target(torch, fd, dev, c3, steps, warmup, 4, 100.0, step_factory=_sp_layer_step(torch, fd, dev, True)))
    del c3
    c4 = U.make_config(4)
    n4 = steps // 4   # a step of config 4 is 15 times config 2's
    put("c4_ragged_scheduled", measure_target(torch, fd, dev, c4, n4, 5, 2, 100.0, variant="persistent"))
    # the plain wrapper orders the work of a batch this large itself, as the scheduled one does; "unscheduled" is that
    # wrapper with the ordering switched off: sequences issued in index order
    put("c4_ragged_plain_wrapper", measure_target(torch, fd, dev, c4, n4, 5, 2, 100.0))
    put("c4_ragged_unscheduled", measure_target(torch, fd, dev, c4, n4, 5, 2, 100.0, auto_order=False))
    del c4
    return t


def measure_write_side(torch, fd, wl, dev, steps, warmup, decode_step, pools, kv_split):
    """The step before the decode at this workload's shape: rotary of q and k plus the append of one token per
    sequence (one launch), alone and followed by the decode step; and the same kernel at prefill size, where it is
    an HBM-bound copy, priced against 8 TB/s with its algorithmic bytes (q, k, v read once; rotated q, K and V
    written once; one cos/sin row per token)."""
    B, Hq, D = wl.q.shape
    _, P, Hkv, _ = wl.k_cache.shape
    fp8 = wl.k_scale is not None
    act = wl.q.dtype
    cache_dtype = wl.k_cache.dtype
    isz, csz = torch.empty(0, dtype=act).element_size(), wl.k_cache.element_size()
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    ang = torch.outer(torch.arange(8192, dtype=torch.float32), inv_freq)
    cos_sin = torch.cat((ang.cos(), ang.sin()), dim=-1).to(dev)
    scales = dict(k_scale=wl.k_scale, v_scale=wl.v_scale) if fp8 else {}

    def setup(T):
        pages = -(-(T + 1) // P)
        kc = torch.zeros(B * pages, P, Hkv, D, dtype=cache_dtype, device=dev)
        vc = torch.zeros_like(kc)
        bt = torch.randperm(B * pages, device=dev).to(torch.int32).view(B, pages)
        lens = torch.zeros(B, dtype=torch.int32, device=dev)
        qkv = torch.randn(B, T, (Hq + 2 * Hkv) * D, device=dev).to(act)
        q, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
        pos = torch.arange(T, device=dev).repeat(B, 1)
        q4 = q.view(B, T, Hq, D)
        q_out = torch.empty(B, T, Hq, D, dtype=act, device=dev)
        lens_out = torch.empty_like(lens)

        def run(_):
            fd.rope_kv_append(k.view(B, T, Hkv, D), v.view(B, T, Hkv, D), kc, vc, bt, lens, kv_lens_out=lens_out,
                              cos_sin=cos_sin, position_ids=pos, q=q4, q_out=q_out, **scales)
        return run

    one = setup(1)
    t_append = _time_us(torch, one, steps, warmup)

    def both(i):
        one(i)
        decode_step(i)
    t_both = _time_us(torch, both, steps, warmup)

    # the drop-in call of the reference's attention block on this workload's own pools: rotary + append (which also
    # ranks the sequences for the decode's issue order when the batch is large enough) + split-KV decode + combine
    qkv1 = torch.randn(B, 1, (Hq + 2 * Hkv) * D, device=dev).to(act)
    q1, k1, v1 = [t.view(B, 1, -1, D) for t in qkv1.split([Hq * D, Hkv * D, Hkv * D], dim=-1)]
    pos1 = wl.kv_lens[:, None].long().clamp(max=cos_sin.shape[0] - 1)
    grown = torch.empty_like(wl.kv_lens)

    def fused(i):
        k, v = pools[i % len(pools)]
        fd.flash_attn_with_kvcache(q1, k, v, k=k1, v=v1, cache_seqlens=wl.kv_lens, block_table=wl.block_table,
                                   causal=True, softcap=wl.soft_cap, num_splits=kv_split, cos_sin_cache=cos_sin,
                                   position_ids=pos1, kv_lens_out=grown, **scales)
    t_fused = _time_us(torch, fused, steps, warmup)

    T = max(P, (4096 * 8 // B) // P * P)          # about 32k new tokens in total
    big = setup(T)
    t_big = _time_us(torch, big, max(5, steps // 5), 3)
    tokens = B * T
    nbytes = tokens * (2 * Hq * D * isz + 2 * Hkv * D * (isz + csz) + D * 4)
    return {
        "kernel": "fd_kv_append_kernel (rotary of q and k + paged append" + (" + fp8 quantisation)" if fp8 else ")"),
        "decode_shape_us": round(t_append, 3), "append_plus_decode_step_us": round(t_both, 3),
        "flash_attn_with_kvcache_us": round(t_fused, 3),
        "prefill_shape": {"new_tokens_per_seq": T, "us": round(t_big, 2), "algorithmic_bytes": nbytes,
                          "achieved_gbps": round(nbytes / (t_big * 1e-6) / 1e9, 1),
                          "frac_of_hbm_peak": round(nbytes / (t_big * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)},
    }


def measure_decode_block(torch, fd, wl, dev, steps, warmup):
    """The caller of the path: one attention block at decode time (QKV projection, rotary + append, split-KV
    decode, combine, output projection) for a model whose hidden size is Hq * D, on a paged cache holding this
    workload's lengths -- launched eagerly from Python, and replayed from a HIP graph as a serving loop would."""
    B, Hq, D = wl.q.shape
    _, P, Hkv, _ = wl.k_cache.shape
    if wl.q.dtype not in (torch.bfloat16, torch.float16):
        return None
    hidden = Hq * D
    dt = wl.q.dtype
    fp8 = wl.k_scale is not None
    max_len = -(-(int(wl.kv_lens.max()) + 64) // P) * P
    attn = fd.layers.TP_Attn()
    w = lambda *shape: (torch.randn(*shape, device=dev) * 0.02).to(dt)  # noqa: E731
    attn.init_from_weights(w(Hq * D, hidden), w(Hkv * D, hidden), w(Hkv * D, hidden), w(hidden, Hq * D), head_dim=D)
    cache = fd.layers.PagedKV_Cache(num_layers=1, batch_size=B, max_length=max_len, kv_heads=Hkv, head_dim=D, dtype=dt,
                                    page_size=P, fp8=fp8)
    cache.kv_offset.copy_(wl.kv_lens)
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32, device=dev) / D))
    tab = fd.layers._set_cos_sin_cache(inv_freq, max_len)
    x = torch.randn(B, 1, hidden, device=dev).to(dt)
    pos = wl.kv_lens[:, None].long()

    def eager(_):
        attn.fwd(x, pos, tab, cache, 0)
    t_eager = _time_us(torch, eager, steps, warmup)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        eager(0)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        attn.fwd(x, pos, tab, cache, 0)
    t_graph = _time_us(torch, lambda _: graph.replay(), steps, warmup)
    return {"hidden_size": hidden, "launches": "2 GEMMs (hipBLASLt) + norm/rotary/append + split-KV decode (+ combine)",
            "eager_us": round(t_eager, 3), "hip_graph_us": round(t_graph, 3)}


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import torch

    fd = importlib.import_module("triton-distributed_amd")
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the flash-decode library has no CPU path", file=sys.stderr)
        sys.exit(2)
    importlib.import_module("triton-distributed_amd.build").ensure_built()   # loads what is built; builds only if nothing is
    fd.load_library()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.shape:
        f = args.shape.split(",")
        B_, n_, hq_, hkv_, d_, p_ = (int(x) for x in f[:6])
        kind = f[6] if len(f) > 6 else "bf16"
        wl_cpu = fd.utils.make_paged_workload(
            f"shape_b{B_}_kv{n_}_hq{hq_}_hkv{hkv_}_d{d_}_p{p_}_{kind}", [n_] * B_, hq_, hkv_, d_, p_,
            torch.float16 if kind == "fp16" else torch.bfloat16, 32, 2000, fp8_kv=kind == "fp8")
    elif args.bf16_twin:
        wl_cpu = fd.utils.make_config5_bf16_twin()
    else:
        wl_cpu = fd.utils.make_config(args.config)
    wl = wl_cpu.to(dev)
    B, Hq, D = wl.q.shape
    S = args.kv_split or wl.kv_split
    algo_bytes = wl_cpu.algorithmic_bytes()

    pools = make_pools(torch, wl, dev, args.pools)
    caller_dt = {None: None, "fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}[args.caller_partials]
    step, out, lse, workspace = make_step(torch, fd, wl, pools, S, dev, variant=args.variant, exact=args.exact_splits,
                                          path=args.path, waves=args.waves, fuse=args.fuse, caller_partials=caller_dt)

    # ---- whole-step timing
    ramp_ms = settle(torch, step, args.clock_ramp_ms)
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    step(-1)   # untimed lead-in (see _time_us): the timed region starts with the queue non-empty
    e0.record()
    for i in range(args.steps):
        step(i)
    e1.record()
    issue_us = (time.perf_counter() - t0) * 1e6 / (args.steps + 1)   # host time to enqueue a step (nothing waited for)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 * args.steps / (args.steps + 1)   # host clock over steps + 1 calls
    gpu_ms = e0.elapsed_time(e1)
    ms_per_step = max(gpu_ms, 0.0) / args.steps
    us_per_step = ms_per_step * 1e3

    # ---- the same step as a prepared object (arguments marshalled once, one library call per step): what a serving
    # loop that keeps its buffers would call; GPU time per step and the host's time to enqueue one
    prepared_us = prepared_issue_us = None
    if args.variant in ("plain", "persistent") and not args.exact_splits and not args.fuse and caller_dt is None:
        kw_p = dict(variant=args.variant, output_combine=out, kv_split=S, lse_out=lse, path=args.path,
                    waves_per_block=args.waves, workspace=workspace)
        if wl.k_scale is not None:
            kw_p.update(k_scale=wl.k_scale, v_scale=wl.v_scale)
        if wl.extra_out is not None:
            kw_p.update(extra_partials=(wl.extra_out, wl.extra_lse))
        prepared = fd.PreparedDecode(wl.q, wl.k_cache, wl.v_cache, wl.kv_lens, wl.block_table, wl.scale, wl.soft_cap,
                                     **kw_p)

        def prepared_step(i):
            k, v = pools[i % len(pools)]
            return prepared(k_cache=k, v_cache=v)
        prepared_us = _time_us(torch, prepared_step, args.steps, args.warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            prepared_step(i)
        prepared_issue_us = (time.perf_counter() - t0) * 1e6 / args.steps
        torch.cuda.synchronize()

    # ---- the same step replayed from a HIP graph (a serving loop captures its step): 8 steps per graph, rotating
    # over the pools like the eager loop
    graph_us = None
    if not args.no_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step(0)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(8):
                step(i)
        graph_us = _time_us(torch, lambda _: graph.replay(), max(5, args.steps // 4), 3) / 8
        del graph

    # ---- dominant kernel alone (split-KV), HIP events on the launch stream
    from ctypes import byref
    lib = fd.load_library()
    fk = importlib.import_module("triton-distributed_amd.kernels.flash_decode")
    L = fd._lib
    # the plan the step above ran with (fd_plan_decode), so that this leg launches the same split kernel
    flags = (L.FD_STEP_EXACT_SPLITS if args.exact_splits else 0) | (L.FD_STEP_SCHEDULE if args.variant == "persistent" else 0) \
        | (L.FD_STEP_FUSED if args.fuse else 0) | (L.FD_STEP_CALLER_PARTIALS if caller_dt is not None else 0)
    plan = fk.decode_plan(wl.q, wl.k_cache, wl.block_table, S, flags=flags, out_dtype=L.fd_dtype_of(out),
                          mid_dtype=L.FD_F32 if caller_dt is None else L.fd_dtype_of(torch.empty(0, dtype=caller_dt)),
                          fp8=wl.k_scale is not None, path=args.path, waves_per_block=args.waves,
                          num_extra=0 if wl.extra_out is None else wl.extra_out.shape[0])
    S_eff = plan.num_splits
    p = fk._make_params(wl.q, wl.k_cache, wl.block_table, S_eff, wl.soft_cap, plan.mid_dtype, L.fd_dtype_of(out),
                        wl.k_scale, wl.v_scale, args.path, args.waves, None, plan.split_align, plan.split_adapt)
    n_o = B * Hq * S_eff * D
    split_ws = torch.empty(B * Hq * S_eff * (D + 1), dtype=torch.float32, device=dev)
    mid = split_ws[:n_o].view(B, Hq, S_eff, D)
    lse_split = split_ws[n_o:n_o + B * Hq * S_eff].view(B, Hq, S_eff)
    lse_split_ptr = lse_split.data_ptr()
    if caller_dt is not None:   # the reference's layout: rows of D + 1 elements, the LSE in the last one
        mid = torch.empty(B, Hq, S_eff, D + 1, dtype=caller_dt, device=dev)
        lse_split_ptr = None
    hstream = torch.cuda.current_stream().cuda_stream
    order_ptr = None
    if plan.order_kind == L.FD_ORDER_ITEMS:
        # the issue order the scheduled step uses: (sequence, range) items, computed once for this leg
        items = fk.item_order_buffer(B, S_eff, dev)
        L.check(lib.fd_schedule_items(hstream, wl.kv_lens.data_ptr(), B, items.data_ptr(), byref(p)))
        p.seq_order_items = 1
        order_ptr = items.data_ptr()
    elif plan.order_kind == L.FD_ORDER_SEQUENCES:
        order_keep = fd.schedule_sequences(wl.kv_lens)
        order_ptr = order_keep.data_ptr()

    def split_only(i):
        k, v = pools[i % len(pools)]
        fd._lib.check(lib.fd_split_kv(
            hstream, wl.q.data_ptr(), k.data_ptr(), v.data_ptr(), mid.data_ptr(), lse_split_ptr,
            float(wl.scale), wl.block_table.data_ptr(), wl.kv_lens.data_ptr(), B,
            wl.q.stride(0), wl.q.stride(1), k.stride(-3), k.stride(-2), v.stride(-3), v.stride(-2),
            mid.stride(0), mid.stride(1), mid.stride(2), wl.block_table.stride(0), order_ptr, byref(p)))

    # (the graph capture above left the device idle for a few milliseconds: back to steady clocks first)
    settle(torch, split_only, min(args.clock_ramp_ms, 50.0))
    for i in range(args.warmup):
        split_only(i)
    torch.cuda.synchronize()
    split_only(-1)   # untimed lead-in, as for the whole step
    e0.record()
    for i in range(args.steps):
        split_only(i)
    e1.record()
    torch.cuda.synchronize()
    split_us = e0.elapsed_time(e1) * 1e3 / args.steps
    achieved = algo_bytes / (split_us * 1e-6) / 1e9

    # ---- what the second launch costs: graph replays of 20 launches each (best of 7 timings of 10 replays)
    decomposition = None
    if args.launch_decomposition:
        tiny = torch.zeros(64, device=dev)

        def replay_us(fn, n=20):
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                fn(0)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for i in range(n):
                    fn(i)
            for _ in range(20):
                g.replay()
            best = float("inf")
            for _ in range(7):
                torch.cuda.synchronize()
                e0.record()
                for _ in range(10):
                    g.replay()
                e1.record()
                torch.cuda.synchronize()
                best = min(best, e0.elapsed_time(e1) * 1e3 / (10 * n))
            return round(best, 3)

        def split_graph(i):   # (the capture stream differs from the stream the leg above launched on)
            k, v = pools[i % len(pools)]
            fd._lib.check(lib.fd_split_kv(
                torch.cuda.current_stream().cuda_stream, wl.q.data_ptr(), k.data_ptr(), v.data_ptr(), mid.data_ptr(),
                lse_split_ptr, float(wl.scale), wl.block_table.data_ptr(), wl.kv_lens.data_ptr(), B,
                wl.q.stride(0), wl.q.stride(1), k.stride(-3), k.stride(-2), v.stride(-3), v.stride(-2),
                mid.stride(0), mid.stride(1), mid.stride(2), wl.block_table.stride(0), order_ptr, byref(p)))

        def split_then_fill(i):
            split_graph(i)
            tiny.zero_()
        decomposition = {
            "method": "HIP-graph replays of 20 launches (or launch pairs), best of 7 timings of 10 replays, us per launch (pair)",
            "split_kernel_us": replay_us(split_graph),
            "split_plus_combine_us": replay_us(step),
            "split_plus_64_element_fill_us": replay_us(split_then_fill),
            "fill_kernel_alone_us": replay_us(lambda i: tiny.zero_()),
        }
        decomposition["second_launch_floor_us"] = round(
            decomposition["split_plus_64_element_fill_us"] - decomposition["split_kernel_us"], 3)
        decomposition["combine_work_beyond_the_floor_us"] = round(
            decomposition["split_plus_combine_us"] - decomposition["split_plus_64_element_fill_us"], 3)

    if args.copy_ref:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(3)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    # HBM bytes per split-kernel launch from the committed counter runs (profiles/*__hbm_traffic.json,
    # FETCH_SIZE + WRITE_SIZE scaled by a copy kernel of known size); None when this workload has none
    traffic = traffic_source = None
    import glob
    candidates = [args.traffic_json] if args.traffic_json else sorted(
        glob.glob(os.path.join(ROOT, "profiles", "*__hbm_traffic.json")))
    for path in candidates:
        if path and os.path.exists(path):
            with open(path) as f:
                rec = json.load(f)
            if args.traffic_json or (rec.get("workload") == wl.name and args.path == "auto"):
                traffic = rec.get("traffic")
                traffic_source = os.path.relpath(path, ROOT)
                break

    # ---- result of pool 0 for the check against the CPU baseline
    step(0)
    torch.cuda.synchronize()
    out_gpu, lse_gpu = out.float().cpu(), lse.cpu()

    result = {
        "metric": "us/decode step + achieved HBM GB/s (% of 8 TB/s), GQA paged decode, 1 GPU",
        "value": round(us_per_step, 3),
        "unit": "us/decode step",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        # the type the path computes in: the MFMA operands' (KV dequantised to it), or f32 on the VALU path
        "dtype": {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}[wl.q.dtype],
        "dtype_detail": ("fp8-e4m3 KV dequantised to the query's " if wl.k_scale is not None else "KV and Q ")
                        + f"{str(wl.q.dtype).replace('torch.', '')}, fp32 accumulate and softmax",
        "data": "synthetic",
        "config": {"workload": wl.name, "batch": B, "q_heads": Hq, "kv_heads": wl.k_cache.shape[2], "head_dim": D,
                   "page_size": wl.k_cache.shape[1], "kv_splits": S, "kv_splits_used": S_eff,
                   "launch_plan": dict(plan.launch, split_adapt=plan.split_adapt, split_align=plan.split_align,
                                       partial_dtype=["f32", "f16", "bf16"][plan.mid_dtype],
                                       order_kind=["none", "sequences", "items"][plan.order_kind],
                                       workspace_bytes=plan.workspace_bytes),
                   "kv_len_total": int(wl_cpu.kv_lens.sum()), "kv_pools_rotated": len(pools),
                   "variant": args.variant, "path": args.path, "fused_combine": args.fuse,
                   "caller_partials": args.caller_partials},
        "hbm_gbps_step": round(algo_bytes / (us_per_step * 1e-6) / 1e9, 1),
        "hbm_pct_of_peak_step": round(100.0 * algo_bytes / (us_per_step * 1e-6) / 1e9 / HBM_PEAK_GBPS, 2),
        "algorithmic_bytes": algo_bytes,
        "library_build_id": lib.fd_build_id().decode(),
        "host_wall_ms_per_step": round(wall_ms / args.steps, 6),
        # the host's own share: wall time per step up to the last enqueue, before the synchronize (the wall figure
        # above ends after it and so can never be below the GPU's time per step)
        "host_issue_us_per_step": round(issue_us, 3),
        "hip_graph_replay_us_per_step": None if graph_us is None else round(graph_us, 3),
        "prepared_step_us": None if prepared_us is None else round(prepared_us, 3),
        "prepared_step_host_issue_us": None if prepared_issue_us is None else round(prepared_issue_us, 3),
        "clock_ramp_ms": round(ramp_ms),
        "timing": "HIP events around exactly `steps` back-to-back steps; 1 untimed lead-in step between the "
                  "synchronize and the first event keeps the host's first-launch latency out of the region",
        "roofline": {"bound": "hbm", "kernel": "fd_split_*_kernel (split-KV decode)", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "kernel_us": round(split_us, 3),
                     # traffic is not measured by this run: it is the figure of the committed counter runs
                     # (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, scaled by a copy of known size) for this workload
                     "traffic_source": traffic_source},
    }

    # MFMA work of the split kernel (secondary figure: the path is HBM-bound).  Issued flops follow from the tiling:
    # per 32 tokens of one (sequence, KV head, block of <=16 query heads) 16 MFMAs of 16x16x32 (16 384 flop each);
    # the committed counter run (profiles/*mfma_utilisation.md) reads exactly this number.
    G = Hq // wl.k_cache.shape[2]
    if D == 128 and args.path != "valu" and wl.q.dtype != torch.float32:
        tokens = int(wl_cpu.kv_lens.sum())
        nhb = -(-G // 16)
        issued = tokens * wl.k_cache.shape[2] * nhb * 16 * 16384 / 32
        result["mfma"] = {"useful_flop_per_step": wl_cpu.flops(), "issued_flop_per_step": int(issued),
                          "issued_tflops": round(issued / (split_us * 1e-6) / 1e12, 1),
                          "frac_of_dense_bf16_peak": round(issued / (split_us * 1e-6) / 2.5e15, 4)}

    headline = args.config == 2 and not args.shape and not args.bf16_twin and args.variant == "plain" \
        and not args.exact_splits and args.path == "auto" and not args.fuse and not args.kv_split \
        and not args.caller_partials
    targets = None
    if headline and not args.no_targets:
        targets = measure_targets(torch, fd, dev, args.steps, args.warmup, (wl, pools))

    if decomposition is not None:
        result["launch_decomposition"] = decomposition
    if not args.no_write_side:
        result["write_side"] = measure_write_side(torch, fd, wl, dev, args.steps, args.warmup, step, pools, S)
        block = measure_decode_block(torch, fd, wl, dev, args.steps, args.warmup)
        if block is not None:
            result["decode_block"] = block

    if not args.no_cpu_baseline:
        import oracle  # the checker, timed as the CPU baseline only
        n_seq = args.cpu_seqs or (B if algo_bytes < 6e8 else max(1, min(B, 4)))
        rows = list(range(n_seq))
        torch_threads = torch.get_num_threads()
        lens = [int(x) for x in wl_cpu.kv_lens.tolist()]
        P = wl_cpu.k_cache.shape[1]
        used = torch.unique(torch.cat([wl_cpu.block_table[i, :-(-lens[i] // P)].long() for i in rows]))
        remap = torch.zeros(wl_cpu.k_cache.shape[0], dtype=torch.long)
        remap[used] = torch.arange(used.numel())
        bt = torch.zeros_like(wl_cpu.block_table[rows])
        for j, i in enumerate(rows):
            npg = -(-lens[i] // P)
            bt[j, :npg] = remap[wl_cpu.block_table[i, :npg].long()].to(torch.int32)
        kc, vc = wl_cpu.k_cache[used], wl_cpu.v_cache[used]
        if wl_cpu.k_scale is not None:
            kc = oracle.dequant_fp8_cache(kc.view(torch.uint8), wl_cpu.k_scale)
            vc = oracle.dequant_fp8_cache(vc.view(torch.uint8), wl_cpu.v_scale)
        kc, vc, qc = kc.float(), vc.float(), wl_cpu.q[rows].float()
        sub_lens = [lens[i] for i in rows]
        times = []
        ref = ref_lse = None
        t_begin = time.perf_counter()
        it = 0
        while it < 4 or (time.perf_counter() - t_begin < 10.0 and it < 60):  # 1 warm-up, then >= 3 runs / about 10 s
            t = time.perf_counter()
            ref, ref_lse = oracle.ref_paged_attn_lse(qc, kc, vc, sub_lens, bt, wl_cpu.scale, soft_cap=wl_cpu.soft_cap)
            if it:
                times.append(time.perf_counter() - t)
            it += 1
        frac_tokens = sum(sub_lens) / max(1, sum(lens))
        cpu_us = statistics.median(times) * 1e6 / frac_tokens
        if wl_cpu.extra_out is None:
            err_o = (out_gpu[rows] - ref).abs().max().item()
            fin = torch.isfinite(ref_lse)
            err_l = ((lse_gpu[rows] - ref_lse)[fin].abs() / ref_lse[fin].abs().clamp_min(1.0)).max().item()
            result["check_vs_cpu_baseline"] = {"max_abs_err_out": round(err_o, 6), "max_rel_err_lse": round(err_l, 8)}
        result["cpu_baseline"] = {
            "value": round(cpu_us, 1), "unit": "us/decode step", "cores": torch_threads, "kind": "port",
            "sample": f"oracle.ref_paged_attn_lse (fp32 PyTorch restatement of the reference's ref_paged_attn) on "
                      f"sequences 0..{n_seq - 1} of {B} of the same seeded workload, median of {len(times)} runs "
                      f"({sum(times):.1f} s of CPU work), scaled by "
                      f"1/{frac_tokens:.4f} (token share) to the whole step; host cpu_count={os.cpu_count()}",
        }
    if targets is not None:
        result["targets"] = targets   # last on the line: the other north-star figures, (us per step, fraction of peak)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
