"""The write-through partial stores (inline assembly, taken by default only from 16 MB of partials on) against the
plain stores on small shapes: every partial, LSE and output must agree bit for bit.  The library reads
FD_STORE_THROUGH once per process, so each mode runs in a child process of its own."""
import os
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.gpu

CHILD = r"""
import importlib, sys, torch
from ctypes import byref
sys.path.insert(0, sys.argv[1])
importlib.import_module("triton-distributed_amd.build").ensure_built()
fd = importlib.import_module("triton-distributed_amd")
fk = importlib.import_module("triton-distributed_amd.kernels.flash_decode")
L, lib, dev = fd._lib, fd.load_library(), "cuda:0"
res = {}
cases = [("bf16_g4", [1320, 18, 463, 2049, 0, 777], 32, 8, torch.bfloat16, False),
         ("fp16_g16", [300, 4096], 64, 4, torch.float16, False),
         ("fp8_g8", [1500, 64, 3000], 64, 8, torch.bfloat16, True),
         ("bf16_g32", [900, 2500], 64, 2, torch.bfloat16, False)]
for name, lens, hq, hkv, dt, fp8 in cases:
    wl = fd.utils.make_paged_workload(name, lens, hq, hkv, 128, 16, dt, 32, seed=5, fp8_kv=fp8).to(dev)
    B, Hq, D = wl.q.shape
    kw = dict(k_scale=wl.k_scale, v_scale=wl.v_scale) if fp8 else {}
    for S in (4, 32):
        # caller-visible partials in the reference layout, fp32 and 16-bit (chunked work items at 32 splits)
        for mid in (torch.float32, dt):
            split = torch.zeros(B, Hq, S, D + 1, dtype=mid, device=dev)
            out = fd.gqa_fwd_batch_decode(wl.q, wl.k_cache, wl.v_cache, None, None, wl.kv_lens, wl.block_table, wl.scale,
                                          output_split=split, kv_split=S, **kw)
            res[f"{name}/caller/{S}/{mid}"] = (split.cpu(), out.cpu())
        # the library's own layout with exactly S splits, through fd_split_kv so that the partials can be read back
        for mid in (L.FD_F32, L.fd_dtype_of(wl.q)):
            p = fk._make_params(wl.q, wl.k_cache, wl.block_table, S, 0.0, mid, L.fd_dtype_of(wl.q), wl.k_scale, wl.v_scale,
                                "auto", 0, None, 64, 0)
            part = torch.zeros(B, Hq, S, D, dtype=torch.float32 if mid == L.FD_F32 else dt, device=dev)
            lse = torch.zeros(B, Hq, S, dtype=torch.float32, device=dev)
            L.check(lib.fd_split_kv(None, wl.q.data_ptr(), wl.k_cache.data_ptr(), wl.v_cache.data_ptr(), part.data_ptr(),
                                    lse.data_ptr(), float(wl.scale), wl.block_table.data_ptr(), wl.kv_lens.data_ptr(), B,
                                    wl.q.stride(0), wl.q.stride(1), wl.k_cache.stride(1), wl.k_cache.stride(2),
                                    wl.v_cache.stride(1), wl.v_cache.stride(2), part.stride(0), part.stride(1),
                                    part.stride(2), wl.block_table.stride(0), None, byref(p)))
            res[f"{name}/own/{S}/{mid}"] = (part.cpu(), lse.cpu())
torch.cuda.synchronize()
torch.save(res, sys.argv[2])
"""


def _run(mode, path):
    env = dict(os.environ, FD_STORE_THROUGH=str(mode))
    r = subprocess.run([sys.executable, "-c", CHILD, ROOT, path], env=env, stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True, timeout=280)
    assert r.returncode == 0, r.stdout[-3000:]


def test_write_through_stores_give_the_same_bits_as_plain_stores(fd, tmp_path):
    through, plain = str(tmp_path / "through.pt"), str(tmp_path / "plain.pt")
    _run(1, through)    # every partial store written through (sc0 sc1)
    _run(2, plain)      # never
    a, b = torch.load(through, weights_only=True), torch.load(plain, weights_only=True)
    assert a.keys() == b.keys() and len(a) == 4 * 2 * 4
    for key in a:
        for x, y in zip(a[key], b[key]):
            assert x.dtype == y.dtype and x.shape == y.shape
            assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)), key
    # and they are partials of something: the combined outputs are finite and not all zero
    assert all(torch.isfinite(v[1].float()).all() and v[1].float().abs().sum() > 0
               for k, v in a.items() if "/caller/" in k)
