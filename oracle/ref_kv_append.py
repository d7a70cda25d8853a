"""CPU restatement of the step before the decode: rotary embedding and the KV-cache update.
TEST INFRASTRUCTURE ONLY.

``ref_set_cos_sin_cache`` and ``ref_rope`` follow
``python/triton_dist/layers/amd/tp_attn.py:62-69`` (table: ``freqs = outer(t, inv_freq)``,
row = ``cos(freqs)`` then ``sin(freqs)``, D/2 each) and ``:72-125`` (kernel:
``out1 = x1*cos - x2*sin``, ``out2 = x2*cos + x1*sin`` with x1 / x2 the two halves of a
head row, computed in fp32 because the table is fp32, stored in x's dtype).  Every product
and sum is rounded separately here (numpy float32, no fused multiply-add); whether the
reference's compiler contracts them is not observable in its sources, so agreement with the
reference's kernel is to one ulp of the activation dtype, while agreement of the HIP kernel
with this file is bit-exact.

``ref_kv_append`` restates the cache update.  The reference's cache is dense
(``python/triton_dist/models/kv_cache.py:36-50``: ``[layers, B, L, Hkv, D]``, tokens of
sequence b at ``[b, offset:offset+T]``); the decode path reads a paged pool
``[pages, P, Hkv, D]`` through an int32 block table
(``python/triton_dist/test/nvidia/test_decode_attn.py:150-156`` and ``:93-99``), so the
update here is "token n of sequence b lives at page ``block_table[b, n // P]``, slot
``n % P``" -- the inverse of that gather.  fp8 caches store
``clamp(x / scale[kv head], +-448)`` rounded to e4m3fn (nearest even).

``ref_rms_norm`` restates the per-head RMS norm the block applies to q and k before the rotation
(``tp_attn.py:52-59, 252-258``); it is evaluated in float64, so a float32 implementation agrees with it
to rounding of the activation dtype, not bit for bit.

Pinning status (tests/test_oracle_pinning.py): the norm by ``torch.nn.functional.rms_norm`` (fp32, CPU), by
scale invariance at eps = 0 and by the constant-row closed form; the rotation by complex multiplication in
float64, by norm preservation, by position 0 being the identity and by additivity of
angles; the table by its definition at hand-computed points; the append by the round trip
through ``ref_decode._gather_kv`` (append token by token, gather, compare with the source
sequence, bit-exact) and by untouched-slot poison checks; the fp8 rounding by a brute-force
nearest-value search (ties to even mantissa) over ``fp8_e4m3fn_decode_table``.  Nothing here
is "parity unpinned".
"""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from .ref_decode import fp8_e4m3fn_decode_table


def ref_set_cos_sin_cache(inv_freq: torch.Tensor, max_length: int) -> torch.Tensor:
    """[max_length, 2 * len(inv_freq)] table: cos then sin of ``t * inv_freq`` (tp_attn.py:62-69)."""
    t = torch.arange(max_length, dtype=inv_freq.dtype)
    freqs = torch.outer(t, inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1)


def ref_rope(x: torch.Tensor, cos_sin: torch.Tensor, position_ids: torch.Tensor) -> torch.Tensor:
    """x [B, T, H, D] -> rotated tensor of the same dtype (tp_attn.py:72-125)."""
    B, T, H, D = x.shape
    half = D // 2
    xf = x.to(torch.float32).numpy()
    cs = cos_sin.to(torch.float32).numpy()
    pos = position_ids.to(torch.long).numpy().clip(0, cs.shape[0] - 1)
    cos = cs[pos][:, :, None, :half]          # [B, T, 1, half]
    sin = cs[pos][:, :, None, half:2 * half]
    x1, x2 = xf[..., :half], xf[..., half:]
    o1 = (x1 * cos).astype(np.float32) - (x2 * sin).astype(np.float32)
    o2 = (x2 * cos).astype(np.float32) + (x1 * sin).astype(np.float32)
    out = np.concatenate([o1, o2], axis=-1).astype(np.float32)
    return torch.from_numpy(out).to(x.dtype)


def ref_rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """Per-row RMS norm over the last dimension, ``x * rsqrt(mean(x^2) + eps) * w`` (tp_attn.py:52-59: torch's
    ``rms_norm`` on the rows of ``[.., heads, head_dim]``), evaluated in float64 and rounded once to x's dtype."""
    xd = x.to(torch.float64)
    rstd = torch.rsqrt(xd.pow(2).mean(dim=-1, keepdim=True) + eps)
    return (xd * rstd * weight.to(torch.float64)).to(x.dtype)


def ref_quantize_fp8(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """x [..., Hkv, D] (any float dtype), scale [Hkv] -> uint8 e4m3fn bit patterns."""
    y = x.to(torch.float32) / scale.to(torch.float32).view(-1, 1)
    return y.clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)


def brute_force_fp8(values: np.ndarray) -> np.ndarray:
    """Nearest finite e4m3fn byte of each float (|v| <= 448), ties to the even mantissa.  O(256) per value."""
    tab = fp8_e4m3fn_decode_table().astype(np.float64)
    finite = [b for b in range(256) if not np.isnan(tab[b])]
    out = np.zeros(values.shape, dtype=np.uint8)
    flat = values.astype(np.float64).ravel()
    res = out.ravel()
    for i, v in enumerate(flat):
        best, best_d = None, None
        for b in finite:
            if (b & 0x80) != (0x80 if np.signbit(v) else 0):
                continue
            d = abs(tab[b] - v)
            if best is None or d < best_d or (d == best_d and (b & 1) == 0 and (best & 1) == 1):
                best, best_d = b, d
        res[i] = best
    return out


def ref_kv_append(k_new: torch.Tensor, v_new: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  block_table: torch.Tensor, kv_lens: torch.Tensor, k_scale: Optional[torch.Tensor] = None,
                  v_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Writes k_new / v_new [B, T, Hkv, D] into the pools in place; returns the grown lengths [B] int32.

    A uint8 cache is fp8-e4m3fn and needs the scales.  Tokens beyond the block table's capacity are dropped
    and the returned length is capped there.
    """
    B, T = k_new.shape[:2]
    P = k_cache.shape[1]
    cap = block_table.shape[1] * P
    out_lens = torch.empty(B, dtype=torch.int32)
    for b in range(B):
        start = max(int(kv_lens[b]), 0)
        out_lens[b] = min(start + T, cap)
        for t in range(T):
            n = start + t
            if n >= cap:
                continue
            page = int(block_table[b, n // P])
            page = min(max(page, 0), k_cache.shape[0] - 1)
            slot = n % P
            for new, cache, scale in ((k_new, k_cache, k_scale), (v_new, v_cache, v_scale)):
                row = new[b, t]
                if cache.dtype == torch.uint8:
                    cache[page, slot] = ref_quantize_fp8(row, scale)
                else:
                    cache[page, slot] = row.to(torch.float32).to(cache.dtype)
    return out_lens
