"""The launch plan on shapes it was not tuned on: 20 seeded shapes away from the benchmark configurations and the
published sweep (odd batch sizes, lengths that are no powers of two, other head counts, page sizes and cache types).
On each the planned step (the library's own split count, ranges and partial type) must not be slower than the plain
launch of exactly 32 splits -- what the reference would run (flash_decode.py:779) -- by more than 3 % (plus 0.5 us of
timer noise on steps of a few microseconds).  Times are GPU times of a HIP-graph replay, best of five."""
import random

import pytest
import torch

from helpers import DEV

pytestmark = pytest.mark.gpu

HEADS = [(32, 8), (64, 8), (40, 8), (16, 16), (96, 12), (28, 4), (24, 2), (48, 6), (8, 1), (128, 8)]


def _shapes(n, seed):
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        hq, hkv = rng.choice(HEADS)
        batch = rng.choice([1, 2, 3, 5, 6, 7, 9, 11, 13, 17, 23, 29, 37, 47])
        longest = rng.choice([1500, 2500, 3700, 6000, 9000, 12000, 20000, 27000, 45000, 70000])
        if batch * longest * hkv > 6_000_000:      # keep a shape under ~1.5 GB of K + V
            continue
        kind = rng.choice(["bf16", "bf16", "fp16", "fp8"])
        page = rng.choice([16, 16, 1, 32])
        ragged = rng.random() < 0.5
        out.append((batch, longest, hq, hkv, kind, page, ragged, rng.randrange(1 << 30)))
    return out


def _time_us(step):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(10):
            step()
    for _ in range(3):
        graph.replay()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(5):
        torch.cuda.synchronize()
        e0.record()
        for _ in range(4):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1e3 / 40)
    return best


def test_planned_step_is_not_slower_than_32_splits_on_held_out_shapes(fd):
    report, failures = [], []
    for batch, longest, hq, hkv, kind, page, ragged, seed in _shapes(20, 20261):
        gen = torch.Generator(device=DEV).manual_seed(seed)
        D = 128
        dtype = torch.float16 if kind == "fp16" else torch.bfloat16
        if ragged:
            lens = torch.randint(longest // 8, longest + 1, (batch,), generator=gen, device=DEV, dtype=torch.int32)
        else:
            lens = torch.full((batch,), longest, device=DEV, dtype=torch.int32)
        pages_per_seq = -(-longest // page)
        pages = batch * pages_per_seq
        q = torch.randn(batch, hq, D, generator=gen, device=DEV, dtype=torch.float32).to(dtype)
        kw = {}
        if kind == "fp8":
            k = torch.randint(0, 120, (pages, page, hkv, D), generator=gen, device=DEV, dtype=torch.uint8)
            v = torch.randint(0, 120, (pages, page, hkv, D), generator=gen, device=DEV, dtype=torch.uint8)
            kw = dict(k_scale=torch.full((hkv,), 0.01, device=DEV), v_scale=torch.full((hkv,), 0.01, device=DEV))
        else:
            k = torch.randn(pages, page, hkv, D, generator=gen, device=DEV, dtype=torch.float32).to(dtype)
            v = torch.randn(pages, page, hkv, D, generator=gen, device=DEV, dtype=torch.float32).to(dtype)
        table = torch.randperm(pages, generator=gen, device=DEV).to(torch.int32).view(batch, pages_per_seq)
        out = torch.empty(batch, hq, D, dtype=dtype, device=DEV)
        ws = torch.empty(64 << 20, dtype=torch.uint8, device=DEV)

        def run(**more):
            return fd.gqa_fwd_batch_decode(q, k, v, ws, None, lens, table, D ** -0.5, output_combine=out, **kw, **more)

        planned = _time_us(lambda: run(kv_split=-1))
        fixed32 = _time_us(lambda: run(kv_split=32, plan_splits=False))
        line = (f"B={batch} longest={longest} heads={hq}/{hkv} {kind} page={page} ragged={ragged}: planned "
                f"{planned:.1f} us, 32 splits {fixed32:.1f} us")
        report.append(line)
        if planned > 1.03 * fixed32 + 0.5:
            failures.append(line)
        del k, v, ws
    print("\n".join(report))
    assert not failures, "\n".join(failures)
