"""The plain-C restatement of the decode oracle (oracle/c/ref_decode.c) against the Python one: two independent
implementations of the same definition must agree on paging, GQA head mapping, soft cap, LSE and empty sequences."""
import ctypes
import importlib.util
import os

import numpy as np
import pytest
import torch

import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _load_builder():
    spec = importlib.util.spec_from_file_location("oracle_c_build", os.path.join(ROOT, "oracle", "c", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="module")
def cref():
    lib = ctypes.CDLL(_load_builder().build_oracle())
    f = ctypes.c_void_p
    lib.ref_paged_decode_f32.restype = ctypes.c_int
    lib.ref_paged_decode_f32.argtypes = [f, f, f, f, f] + [ctypes.c_int32] * 7 + [ctypes.c_float, ctypes.c_float, f, f]
    return lib


def _run_c(lib, q, k, v, bt, lens, scale, soft_cap):
    q, k, v = (np.ascontiguousarray(t.numpy(), dtype=np.float32) for t in (q, k, v))
    bt = np.ascontiguousarray(bt.numpy(), dtype=np.int32)
    lens = np.asarray(lens, dtype=np.int32)
    B, Hq, D = q.shape
    pages, P, Hkv, _ = k.shape
    out = np.zeros_like(q)
    lse = np.zeros((B, Hq), dtype=np.float32)
    ptr = lambda a: a.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    rc = lib.ref_paged_decode_f32(ptr(q), ptr(k), ptr(v), ptr(bt), ptr(lens), B, Hq, Hkv, D, P, pages, bt.shape[1],
                                  scale, soft_cap, ptr(out), ptr(lse))
    assert rc == 0
    return torch.from_numpy(out), torch.from_numpy(lse)


@pytest.mark.parametrize("Hq,Hkv,D,P,soft_cap", [(8, 2, 32, 4, 0.0), (6, 1, 16, 1, 30.0), (4, 4, 64, 16, 0.0), (12, 3, 8, 7, 5.0)])
def test_c_oracle_matches_python_oracle(cref, Hq, Hkv, D, P, soft_cap):
    g = torch.Generator().manual_seed(Hq * 100 + D)
    lens = [37, 0, 1, 4 * P + 3]
    B, pages = len(lens), 40
    maxp = max(1, max(-(-n // P) for n in lens))
    q = torch.randn(B, Hq, D, generator=g)
    k = torch.randn(pages, P, Hkv, D, generator=g)
    v = torch.randn(pages, P, Hkv, D, generator=g)
    bt = torch.randint(0, pages, (B, maxp), generator=g, dtype=torch.int32)
    scale = D ** -0.5
    out_c, lse_c = _run_c(cref, q, k, v, bt, lens, scale, soft_cap)
    out_p, lse_p = oracle.ref_paged_attn_lse(q, k, v, lens, bt, scale, soft_cap=soft_cap)
    assert torch.allclose(out_c, out_p.float(), atol=2e-6, rtol=1e-5)
    fin = torch.isfinite(lse_p)
    assert torch.equal(torch.isfinite(lse_c), fin)
    assert torch.allclose(lse_c[fin], lse_p.float()[fin], atol=2e-6, rtol=1e-6)
    assert torch.equal(out_c[1], torch.zeros(Hq, D)) and torch.isinf(lse_c[1]).all()     # the empty sequence


def test_c_oracle_clamps_page_ids_and_rejects_bad_shapes(cref):
    q = torch.randn(1, 2, 8)
    k = torch.randn(3, 4, 1, 8)
    v = torch.randn(3, 4, 1, 8)
    good, _ = _run_c(cref, q, k, v, torch.tensor([[2, 0]], dtype=torch.int32), [6], 1.0, 0.0)
    clamped, _ = _run_c(cref, q, k, v, torch.tensor([[99, -5]], dtype=torch.int32), [6], 1.0, 0.0)
    assert torch.equal(good, clamped)
    z = ctypes.c_void_p(0)
    assert cref.ref_paged_decode_f32(z, z, z, z, z, 1, 3, 2, 8, 4, 3, 2, 1.0, 0.0, z, z) == -1     # Hq % Hkv != 0
