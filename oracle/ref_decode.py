"""CPU restatement of the reference's PyTorch decode oracle.  TEST INFRASTRUCTURE ONLY.

Follows ``ref_paged_attn`` in
``python/triton_dist/test/nvidia/test_decode_attn.py:70-120`` (an identical copy
lives in ``test_sp_decode_attn.py:82-132``): per sequence, gather the first
``ceil(kv_len / page)`` block-table entries, flatten to token rows, keep the
first ``kv_len`` rows, repeat KV heads so that *consecutive* query heads share a
KV head, scores = (q * scale) . k, optional soft-cap, softmax, P . V.

Deliberate differences from the reference text (its quirks are not algorithm):
  * the caller's query is not scaled in place (reference line 90-91 does);
  * P is not rounded to V's dtype before P.V (reference line 114): everything is
    computed in ``compute_dtype`` (fp32 by default, fp64 when pinning), which is
    the "softmax(QK^T*scale)V computed in fp32" definition of correctness;
  * ``soft_cap`` defaults to 0.0, not None (reference line 79 vs 111).

The reference oracle returns no log-sum-exp.  ``lse`` here is the natural-log
``logsumexp`` of the (soft-capped) scaled scores, which is what the kernels emit
(``e_max + tl.log(e_sum)``, ``kernels/nvidia/flash_decode.py:239`` and ``:448``).

Pinning status (see tests/test_oracle_pinning.py): decode output and LSE are
pinned by closed forms (equal keys, kv_len == 1, dominant key, shift
invariance), by ``torch.nn.functional.scaled_dot_product_attention`` on the
gathered cache, and by an independent pure-Python float64 brute force; paging by
permutation / poison / duplicate-page invariants; the fp8 table by
``torch.float8_e4m3fn`` conversion.  Nothing here is "parity unpinned" at
tolerance level.  Bit-level parity with Triton's ``fast_expf``/``tl.dot``
rounding is unpinned (no fixtures exist in the reference and its compiler is
not vendored); the reference's own tests only claim 1e-2.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import numpy as np
import torch


def _gather_kv(cache: torch.Tensor, block_row: torch.Tensor, kv_len: int) -> torch.Tensor:
    """Token rows [kv_len, Hkv, D] of one sequence (test_decode_attn.py:93-99)."""
    page = cache.shape[1]
    n_pages = (kv_len + page - 1) // page
    idx = block_row[:n_pages].to(torch.long)
    return cache[idx].reshape(-1, cache.shape[2], cache.shape[3])[:kv_len]


def ref_paged_attn_lse(
    query: torch.Tensor,          # [B, Hq, D]   (decode: one query token per sequence)
    key_cache: torch.Tensor,      # [num_pages, P, Hkv, D]
    value_cache: torch.Tensor,    # [num_pages, P, Hkv, Dv]
    kv_lens: Sequence[int],
    block_tables: torch.Tensor,   # [B, max_pages] int
    scale: float,
    soft_cap: float = 0.0,
    compute_dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (out [B,Hq,Dv], lse [B,Hq]) in ``compute_dtype``.

    A sequence with kv_len == 0 yields out = 0 and lse = -inf (the reference
    would produce NaN from 0/0; the build defines the empty case).
    """
    B, Hq, _ = query.shape
    Hkv = key_cache.shape[2]
    assert Hq % Hkv == 0
    group = Hq // Hkv
    bt = block_tables.detach().cpu()
    outs, lses = [], []
    for i in range(B):
        kv_len = int(kv_lens[i])
        q = query[i].to(compute_dtype) * scale                       # [Hq, D]   (:90-91, not in place)
        if kv_len == 0:
            outs.append(torch.zeros(Hq, value_cache.shape[3], dtype=compute_dtype))
            lses.append(torch.full((Hq,), float("-inf"), dtype=compute_dtype))
            continue
        k = _gather_kv(key_cache, bt[i], kv_len).to(compute_dtype)    # [kv, Hkv, D]
        v = _gather_kv(value_cache, bt[i], kv_len).to(compute_dtype)
        if group != 1:                                                # (:101-103)
            k = torch.repeat_interleave(k, group, dim=1)
            v = torch.repeat_interleave(v, group, dim=1)
        attn = torch.einsum("hd,khd->hk", q, k)                      # (:104), query_len == 1
        if soft_cap is not None and soft_cap > 0.0:                  # (:111-112)
            attn = soft_cap * torch.tanh(attn / soft_cap)
        # decode: the causal mask triu(ones(1,kv_len), diagonal=kv_len) is empty (:105-106)
        lses.append(torch.logsumexp(attn, dim=-1))
        p = torch.softmax(attn, dim=-1)                              # (:114)
        outs.append(torch.einsum("hk,khd->hd", p, v))                # (:115)
    return torch.stack(outs, 0), torch.stack(lses, 0)


def ref_paged_attn(query, key_cache, value_cache, query_lens, kv_lens, block_tables, scale,
                   sliding_window: Optional[int] = None, soft_cap: float = 0.0) -> torch.Tensor:
    """Signature-compatible wrapper (test_decode_attn.py:70-80) for decode (all query_lens == 1)."""
    assert sliding_window is None, "the decode path never passes a sliding window"
    assert all(int(x) == 1 for x in query_lens)
    out, _ = ref_paged_attn_lse(query, key_cache, value_cache, kv_lens, block_tables, scale,
                                soft_cap=soft_cap or 0.0)
    return out


# --------------------------------------------------------------------------- fp8 (OCP e4m3fn)

def fp8_e4m3fn_decode_table() -> np.ndarray:
    """All 256 OCP FP8 E4M3 ("fn": no inf, NaN = S.1111.111) values as float32.

    Integer restatement of the published format: 1 sign, 4 exponent (bias 7),
    3 mantissa bits; exponent 0 is subnormal (m/8 * 2^-6); 0x7f / 0xff are NaN.
    """
    tab = np.zeros(256, dtype=np.float64)
    for byte in range(256):
        s = -1.0 if byte & 0x80 else 1.0
        e = (byte >> 3) & 0xF
        m = byte & 0x7
        if e == 0xF and m == 0x7:
            val = float("nan")
        elif e == 0:
            val = s * (m / 8.0) * 2.0 ** (-6)
        else:
            val = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
        tab[byte] = val
    return tab.astype(np.float32)


def dequant_fp8_cache(cache_u8: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """[pages,P,Hkv,D] uint8 (e4m3fn bit patterns) x per-KV-head fp32 scale -> fp32 cache."""
    tab = torch.from_numpy(fp8_e4m3fn_decode_table())
    vals = tab[cache_u8.to(torch.long)]
    return vals * scale.to(torch.float32).view(1, 1, -1, 1)


def quantize_fp8_cache(cache_f32: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-KV-head scale = absmax/448; q = clamp(x/scale, +-448) rounded to e4m3fn.

    Returns (uint8 bit patterns, scale [Hkv] fp32).  Rounding is torch's
    float32 -> float8_e4m3fn conversion (round to nearest even).
    """
    absmax = cache_f32.abs().amax(dim=(0, 1, 3)).clamp_min(1e-12)
    scale = (absmax / 448.0).to(torch.float32)
    q = (cache_f32 / scale.view(1, 1, -1, 1)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q.view(torch.uint8), scale
