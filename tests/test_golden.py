"""Golden fixtures (tests/golden/*.npz): the oracle must reproduce them on the CPU, the HIP path
must match them on the GPU."""
import glob
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import DEV, assert_lse_close, assert_out_close

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))
_DT = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}


def _load(path):
    z = np.load(path, allow_pickle=False)
    dt = _DT[str(z["dtype"])]

    def bits(a):
        t = torch.from_numpy(a.copy())
        return t if dt == torch.float32 else t.view(torch.int16).view(dt)
    rec = dict(q=bits(z["q"]), kv_lens=z["kv_lens"].tolist(), bt=torch.from_numpy(z["block_table"].copy()),
               scale=float(z["scale"]), soft_cap=float(z["soft_cap"]), kv_split=int(z["kv_split"]),
               out=torch.from_numpy(z["out"].copy()), lse=torch.from_numpy(z["lse"].copy()), k_scale=None, v_scale=None)
    if str(z["kv_dtype"]) == "fp8_e4m3":
        rec.update(k=torch.from_numpy(z["k_cache"].copy()), v=torch.from_numpy(z["v_cache"].copy()),
                   k_scale=torch.from_numpy(z["k_scale"].copy()), v_scale=torch.from_numpy(z["v_scale"].copy()))
    else:
        rec.update(k=bits(z["k_cache"]), v=bits(z["v_cache"]))
    return rec


def test_fixtures_exist():
    assert len(GOLDEN) >= 5


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_oracle_reproduces_fixture(path):
    r = _load(path)
    if r["k_scale"] is not None:
        kf, vf = oracle.dequant_fp8_cache(r["k"], r["k_scale"]), oracle.dequant_fp8_cache(r["v"], r["v_scale"])
    else:
        kf, vf = r["k"].float(), r["v"].float()
    out, lse = oracle.ref_paged_attn_lse(r["q"].float(), kf, vf, r["kv_lens"], r["bt"], r["scale"],
                                         soft_cap=r["soft_cap"])
    assert torch.allclose(out, r["out"], atol=2e-6, rtol=1e-5)
    assert torch.allclose(lse, r["lse"], atol=2e-6, rtol=1e-6)
    # the split/combine model lands on the same values
    o2, l2, _ = oracle.model_gqa_fwd_batch_decode(r["q"].float(), kf, vf, r["kv_lens"], r["bt"], r["scale"],
                                                  soft_cap=r["soft_cap"], kv_split=r["kv_split"])
    assert torch.allclose(o2, r["out"], atol=1e-5) and torch.allclose(l2, r["lse"], atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("variant", ["plain", "persistent", "fused"])
@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_hip_path_matches_fixture(fd, path, variant):
    r = _load(path)
    B, Hq, _ = r["q"].shape
    lse = torch.empty(B, Hq, dtype=torch.float32, device=DEV)
    kw = {}
    if r["k_scale"] is not None:
        kw.update(k_scale=r["k_scale"].to(DEV), v_scale=r["v_scale"].to(DEV))
    if variant == "fused":
        kw["fuse_combine"] = True
    fn = fd.gqa_fwd_batch_decode_persistent if variant == "persistent" else fd.gqa_fwd_batch_decode
    out = fn(r["q"].to(DEV), r["k"].to(DEV), r["v"].to(DEV), None, [1] * B,
             torch.tensor(r["kv_lens"], dtype=torch.int32, device=DEV), r["bt"].to(DEV), r["scale"], r["soft_cap"],
             kv_split=r["kv_split"], lse_out=lse, **kw)
    torch.cuda.synchronize()
    fp32 = r["q"].dtype == torch.float32
    assert_out_close(out, r["out"], atol=2e-4 if fp32 else 2e-2)
    assert_lse_close(lse, r["lse"], rtol=1e-5 if fp32 else 1e-3)
