"""CPU model of the reference's split-KV and combine recurrences.  TEST INFRASTRUCTURE ONLY.

Restates, tile by tile, what the Triton kernels in
``python/triton_dist/kernels/nvidia/flash_decode.py`` compute:

  * split ranges                      -- lines 193-195 (repeated at 339-341, 424-426, 739-741)
  * token -> cache row                -- lines 203-206
  * per-split online softmax          -- lines 197-239 (BLOCK_N = 64 tokens per tile, line 770)
  * plain / intra-rank / inter-rank combine -- lines 331-360, 416-449, 505-532
  * the sequence-parallel composition -- ``layers/nvidia/sp_flash_decode_layer.py:83-185``
    with the allgather replaced by stacking the per-shard results.

All softmax state is fp32 as in the reference (lines 197-199); ``exp`` is the
exact one (the reference's ``fast_expf`` is an approximation, so only
tolerance-level agreement is meaningful).  ``round_p_to`` reproduces the
reference's down-cast of P to V's dtype before P.V (line 230) when a dtype is
given; by default P stays fp32.

Pinning: split ranges by brute force partition checks; the recurrences by the
algebraic identity "merge of normalised partials == attention over the union"
against ``ref_decode.ref_paged_attn_lse`` in float64, by permutation invariance
and by the closed form sum_r softmax(lse)_r * out_r (tests/test_oracle_pinning.py).
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch

BLOCK_N = 64  # flash_decode.py:770


def split_range(kv_len: int, num_splits: int, s: int) -> Tuple[int, int]:
    """[start, end) of split ``s`` (flash_decode.py:193-195).  Empty iff end <= start."""
    per = -(-kv_len // num_splits)
    start = per * s
    end = min(start + per, kv_len)
    return start, end


def _cache_row(block_row, n: int, page_size: int) -> int:
    """Flat token row of logical token ``n`` (flash_decode.py:203-205)."""
    page = int(block_row[n // page_size])
    return page * page_size + n % page_size


def model_split_kv(
    q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, kv_lens: Sequence[int],
    block_table: torch.Tensor, scale: float, num_splits: int, soft_cap: float = 0.0,
    round_p_to: Optional[torch.dtype] = None, compute_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """Returns output_split [B, Hq, S, Dv+1] (partial out in [:Dv], partial LSE at [Dv]).

    Empty splits hold 0 / -inf (the reference leaves NaN there, line 236; its
    combine never reads them, line 343).
    """
    B, Hq, D = q.shape
    _, P, Hkv, Dv = v_cache.shape
    G = Hq // Hkv
    kflat = k_cache.reshape(-1, Hkv, k_cache.shape[3])
    vflat = v_cache.reshape(-1, Hkv, Dv)
    bt = block_table.detach().cpu().tolist()
    out = torch.zeros(B, Hq, num_splits, Dv + 1, dtype=compute_dtype)
    out[..., Dv] = float("-inf")
    for b in range(B):
        kv_len = int(kv_lens[b])
        for s in range(num_splits):
            start, end = split_range(kv_len, num_splits, s)
            if end <= start:
                continue
            rows = torch.tensor([_cache_row(bt[b], n, P) for n in range(start, end)], dtype=torch.long)
            for hk in range(Hkv):
                qh = q[b, hk * G:(hk + 1) * G].to(compute_dtype)          # heads sharing kv head hk (line 167)
                m = torch.full((G,), float("-inf"), dtype=compute_dtype)
                l = torch.zeros(G, dtype=compute_dtype)
                acc = torch.zeros(G, Dv, dtype=compute_dtype)
                for t0 in range(0, end - start, BLOCK_N):                 # line 201
                    r = rows[t0:t0 + BLOCK_N]
                    k = kflat[r, hk].to(compute_dtype)                    # [n, D]
                    v = vflat[r, hk].to(compute_dtype)
                    qk = (qh @ k.T) * scale                               # lines 208, 216
                    if soft_cap > 0:
                        qk = soft_cap * torch.tanh(qk / soft_cap)         # lines 218-219
                    m_new = torch.maximum(qk.max(dim=1).values, m)        # line 226
                    alpha = torch.exp(m - m_new)                          # line 227
                    p = torch.exp(qk - m_new[:, None])                    # line 228
                    pv = p if round_p_to is None else p.to(round_p_to).to(compute_dtype)
                    acc = acc * alpha[:, None] + pv @ v                   # lines 229-230
                    l = l * alpha + p.sum(dim=1)                          # line 232
                    m = m_new
                out[b, hk * G:(hk + 1) * G, s, :Dv] = acc / l[:, None]    # line 236
                out[b, hk * G:(hk + 1) * G, s, Dv] = m + torch.log(l)     # line 239
    return out


def _merge(partials_o, partials_lse, valid):
    """Sequential LSE merge (flash_decode.py:345-354).  Returns (out, lse)."""
    Dv = partials_o[0].shape[-1]
    dt = partials_o[0].dtype
    m = float("-inf")
    l = 0.0
    acc = torch.zeros(Dv, dtype=dt)
    for o, L, ok in zip(partials_o, partials_lse, valid):
        if not ok:
            continue
        L = float(L)
        m_new = max(L, m)
        old = math.exp(m - m_new) if m != float("-inf") else 0.0
        w = math.exp(L - m_new) if L != float("-inf") else 0.0
        acc = acc * old + w * o
        l = l * old + w
        m = m_new
    if l == 0.0:
        return torch.zeros(Dv, dtype=dt), float("-inf")   # reference: 0/0 = NaN; build: 0, -inf
    return acc / l, m + math.log(l)


def model_combine(
    mid_o: torch.Tensor, mode: str, kv_lens=None, global_kv_lens=None,
    extra_out: Optional[torch.Tensor] = None, extra_lse: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Merge partials.  Returns (out [B,Hq,Dv], lse [B,Hq]) in mid_o's dtype.

    mode "split": mid_o [B,Hq,S,Dv+1]; split s valid iff its range is non-empty
                  (flash_decode.py:339-343, 424-428).
    mode "rank":  mid_o [R,B,Hq,Dv+1]; rank r valid iff global_kv_lens[r,b] > 0
                  (flash_decode.py:513-515).
    extra_out [E,B,Hq,Dv], extra_lse [E,B,Hq]: further always-valid partials
    merged after the others (the single-GPU stand-in for partials that other
    sequence-parallel ranks would contribute).
    """
    if mode == "split":
        B, Hq, S, D1 = mid_o.shape
    else:
        S, B, Hq, D1 = mid_o.shape
    Dv = D1 - 1
    out = torch.zeros(B, Hq, Dv, dtype=mid_o.dtype)
    lse = torch.zeros(B, Hq, dtype=mid_o.dtype)
    for b in range(B):
        for h in range(Hq):
            if mode == "split":
                n = int(kv_lens[b])
                valid = [split_range(n, S, s)[1] > split_range(n, S, s)[0] for s in range(S)]
                po = [mid_o[b, h, s, :Dv] for s in range(S)]
                pl = [mid_o[b, h, s, Dv] for s in range(S)]
            else:
                valid = [int(global_kv_lens[r][b]) > 0 for r in range(S)]
                po = [mid_o[r, b, h, :Dv] for r in range(S)]
                pl = [mid_o[r, b, h, Dv] for r in range(S)]
            if extra_out is not None:
                for e in range(extra_out.shape[0]):
                    po.append(extra_out[e, b, h].to(mid_o.dtype))
                    pl.append(extra_lse[e, b, h].to(mid_o.dtype))
                    valid.append(True)
            o, L = _merge(po, pl, valid)
            out[b, h] = o
            lse[b, h] = L
    return out, lse


def model_gqa_fwd_batch_decode(q, k_cache, v_cache, kv_lens, block_table, scale, soft_cap=0.0,
                               kv_split=-1, compute_dtype=torch.float32, round_p_to=None):
    """Split + plain combine, as ``gqa_fwd_batch_decode`` (flash_decode.py:763-844) chains them."""
    S = 32 if kv_split == -1 else kv_split                                # line 779
    mid = model_split_kv(q, k_cache, v_cache, kv_lens, block_table, scale, S, soft_cap,
                         round_p_to=round_p_to, compute_dtype=compute_dtype)
    out, lse = model_combine(mid, "split", kv_lens=kv_lens)
    return out, lse, mid


def model_sp_decode(q, k_shards, v_shards, global_kv_lens, block_tables, scale, soft_cap=0.0,
                    kv_split=32, compute_dtype=torch.float32):
    """Sequence-parallel decode on R shards (sp_flash_decode_layer.py:83-185).

    Per shard: split + intra-rank combine (out and merged LSE packed as
    [B,Hq,Dv+1], flash_decode.py:441-449); then the inter-rank merge over the
    stacked [R,B,Hq,Dv+1] results (the allgather is the stacking).
    """
    R = len(k_shards)
    packed = []
    for r in range(R):
        o, L, _ = model_gqa_fwd_batch_decode(q, k_shards[r], v_shards[r], global_kv_lens[r], block_tables[r],
                                             scale, soft_cap, kv_split, compute_dtype)
        packed.append(torch.cat([o, L[..., None]], dim=-1))
    gathered = torch.stack(packed, 0)
    return model_combine(gathered, "rank", global_kv_lens=global_kv_lens)
