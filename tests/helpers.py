"""Shared helpers of the GPU parity tests: run the HIP path, run the CPU oracle on the same bits."""
import torch

import oracle

DEV = "cuda:0"

# north-star gates
OUT_ATOL_16BIT = 2e-2      # max-abs on bf16/fp16 outputs
LSE_RTOL = 1e-3            # relative on LSE


def oracle_decode(wl, rows=None):
    """fp32 oracle on a workload (optionally only the sequences in ``rows``).

    Only the pages the chosen sequences reference are converted to fp32 (the table is remapped
    into that compact copy), so full-size pools stay cheap; fp8 caches are dequantised first.
    """
    q, lens, bt = wl.q, wl.kv_lens.tolist(), wl.block_table
    if rows is not None:
        q, lens, bt = q[rows], [lens[i] for i in rows], bt[rows]
    P = wl.k_cache.shape[1]
    used = torch.unique(torch.cat([bt[i, :-(-n // P)].long() for i, n in enumerate(lens)] + [torch.zeros(1).long()]))
    remap = torch.zeros(wl.k_cache.shape[0], dtype=torch.long)
    remap[used] = torch.arange(used.numel())
    bt_c = torch.zeros_like(bt)
    for i, n in enumerate(lens):
        npg = -(-n // P)
        bt_c[i, :npg] = remap[bt[i, :npg].long()].to(bt.dtype)
    k, v = wl.k_cache[used], wl.v_cache[used]
    if wl.k_scale is not None:
        k = oracle.dequant_fp8_cache(k.view(torch.uint8), wl.k_scale)
        v = oracle.dequant_fp8_cache(v.view(torch.uint8), wl.v_scale)
    return oracle.ref_paged_attn_lse(q.float(), k.float(), v.float(), lens, bt_c, wl.scale, soft_cap=wl.soft_cap)


def assert_lse_close(lse, ref, rtol=LSE_RTOL):
    lse, ref = lse.float().cpu(), ref.float().cpu()
    fin = torch.isfinite(ref)
    assert torch.equal(torch.isfinite(lse), fin), "LSE finiteness differs"
    assert torch.equal(lse[~fin], ref[~fin])
    # relative error with an absolute floor of 1 so that |lse| ~ 0 is not penalised
    err = (lse[fin] - ref[fin]).abs() / ref[fin].abs().clamp_min(1.0)
    assert err.numel() == 0 or err.max().item() <= rtol, f"LSE rel err {err.max().item():.3e} > {rtol}"


def assert_out_close(out, ref, atol=OUT_ATOL_16BIT, rtol=0.0, rel=True):
    """The north-star gate (max-abs), and with ``rel`` the scale-aware gate below on top of it."""
    out, ref = out.float().cpu(), ref.float().cpu()
    assert torch.isfinite(out).all(), "non-finite output"
    err = (out - ref).abs()
    bound = atol + rtol * ref.abs()
    assert (err <= bound).all(), f"max abs err {err.max().item():.3e} (atol {atol}, rtol {rtol})"
    if rel:
        assert_out_rel(out, ref)


# Scale-aware gate.  With thousands of N(0,1) value rows per sequence the outputs are 0.01-0.02 in magnitude, as large
# as the north-star's absolute tolerance, so that gate alone would pass an output that is wrong by a constant factor.
# Rounding the output to bf16 alone is 2^-9 relative per element (rms about 1.5e-3); 16-bit partials add as much again.
OUT_RMS_RTOL = 1e-2        # rms(out - ref) / rms(ref)
OUT_MAX_RTOL = 2e-2        # max|out - ref| / max|ref|


def assert_out_rel(out, ref, rms_rtol=OUT_RMS_RTOL, max_rtol=OUT_MAX_RTOL):
    """Error relative to the size of the reference values, per call (all elements together)."""
    out, ref = out.double().cpu(), ref.double().cpu()
    assert torch.isfinite(out).all(), "non-finite output"
    if ref.numel() == 0 or not ref.any():
        assert not out.any()
        return
    diff = out - ref
    rms = (diff.pow(2).mean().sqrt() / ref.pow(2).mean().sqrt()).item()
    mx = (diff.abs().max() / ref.abs().max()).item()
    assert rms <= rms_rtol, f"rms error {rms:.3e} of the reference's rms (limit {rms_rtol})"
    assert mx <= max_rtol, f"max error {mx:.3e} of the reference's largest value (limit {max_rtol})"


def run_decode(fd, wl, variant="plain", **kw):
    """Moves the workload to the GPU, runs the HIP path, returns (out, lse) on the CPU."""
    g = wl.to(DEV)
    B, Hq, D = g.q.shape
    lse = torch.empty(B, Hq, dtype=torch.float32, device=DEV)
    fn = {"plain": fd.gqa_fwd_batch_decode, "intra": fd.gqa_fwd_batch_decode_intra_rank,
          "persistent": fd.gqa_fwd_batch_decode_persistent}[variant]
    if g.k_scale is not None:
        kw.setdefault("k_scale", g.k_scale)
        kw.setdefault("v_scale", g.v_scale)
    out = fn(g.q, g.k_cache, g.v_cache, None, [1] * B, g.kv_lens, g.block_table, g.scale, g.soft_cap,
             kv_split=g.kv_split, lse_out=lse, **kw)
    torch.cuda.synchronize()
    return out.cpu(), lse.cpu()
