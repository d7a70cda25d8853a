"""Sequence-parallel GQA flash-decode layer, one GPU's share.

Mirrors ``SpGQAFlashDecodeAttention`` in
``python/triton_dist/layers/nvidia/sp_flash_decode_layer.py:44-185``: constructor
arguments, attributes, ``forward(q, k_cache, v_cache, global_kv_lens,
block_table)`` and ``finalize()`` are the same.  The data flow is the
reference's:

  1. local split-KV decode + intra-rank combine on this rank's KV shard, with
     the merged LSE packed at column Dv            (:107-110)
  2. the result goes into this rank's slot of a staged buffer laid out as
     ``[num_ranks, B, Hq, Dv+1]``                   (:136-145)
  3. inter-rank LSE merge over the slots; rank r counts for sequence b iff
     ``global_kv_lens[r, b] > 0``                   (:173-183)

Step 2 is where the reference allgathers over NVSHMEM (:139).  Nothing here
spans more than one GPU: the other ranks' partials come from
``remote_partials`` -- ``(out [R-1, B, Hq, Dv], lse [R-1, B, Hq])`` in rank order
with this rank left out -- which the caller produces on the same device.  By
default a forward is two launches: the split kernel and one combine that merges
the local splits, writes that merge into this rank's slot (the slot a push to
the other ranks would be sent from) and merges it with the remote partials
where they are.  ``staged_exchange=True`` walks the reference's steps one by
one instead -- local result into its slot, the others' partials copied into
theirs, stand-alone inter-rank kernel over the slots -- which is the shape a
real exchange would take: a push-allgather writes the slots, step 3 follows.
With ``num_ranks == 1`` no remote partials are needed and steps 2 and 3 fall
away: the local decode writes the final output.

The staged partials are fp32 by default, so the LSE is not rounded to the
query's 16-bit dtype as in the reference (:95-97); pass ``partial_dtype=q.dtype``
for the reference's byte layout.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ..kernels.flash_decode import (gqa_fwd_batch_decode, gqa_fwd_batch_decode_intra_rank,
                                    kernel_inter_rank_gqa_fwd_batch_decode_combine_kv)


class SpGQAFlashDecodeAttention(torch.nn.Module):

    def __init__(self, rank, node, num_ranks, num_nodes, num_q_heads, num_kv_heads, q_head_dim, v_head_dim,
                 page_size=1, scale=1, soft_cap=0, max_allowed_batch=1, thrink_buffer_threshold=500, stages=20,
                 partial_dtype: Optional[torch.dtype] = torch.float32, staged_exchange: bool = False):
        super().__init__()
        self.rank = rank
        self.num_ranks = num_ranks
        self.node = node
        self.num_nodes = num_nodes
        self.workspace = None  # the decode kernels need no workspace
        self.num_q_heads = num_q_heads
        self.num_kv_heads = num_kv_heads
        self.q_head_dim = q_head_dim
        self.v_head_dim = v_head_dim
        self.page_size = page_size
        self.soft_cap = soft_cap
        self.scale = scale
        # The reference fixes 32 splits (sp_flash_decode_layer.py:62).  The partials never leave this layer, so the
        # count is left to the library: 32 for short shards, up to 256 for long ones.  Set it to 32 (and pass
        # ``partial_dtype=None``) for the reference's settings.
        self.kv_split = -1
        self.max_allowed_batch = max_allowed_batch
        self.stages = stages
        self.partial_dtype = partial_dtype
        # False: the other ranks' partials are merged where the caller holds them (two launches per forward);
        # True: they are first copied into their slots of the staged buffer and merged from there by the stand-alone
        # inter-rank kernel, step by step as in the reference
        self.staged_exchange = staged_exchange
        assert 0 <= rank < num_ranks

        # staging ring for the gathered partials (a plain device tensor: no symmetric heap on one GPU)
        self.max_allgather_buffer_size = self.num_ranks * self.num_q_heads * self.v_head_dim * 8  # bytes
        self.ag_buffer: Optional[torch.Tensor] = None
        self.signal_target = 0  # advances once per forward, selects the ring stage

        # track buffer size
        self.count_less_than_half = 0
        self.shrink_buffer_threshold = thrink_buffer_threshold

    def finalize(self):
        self.ag_buffer = None

    def _stage(self, nbytes: int, device) -> torch.Tensor:
        """Ring stage for this call, grown (doubled) or shrunk (halved) like the reference's buffer."""
        realloc = self.ag_buffer is None or self.ag_buffer.device != device
        while nbytes >= self.max_allgather_buffer_size:
            self.max_allgather_buffer_size *= 2
            realloc = True
        if nbytes < self.max_allgather_buffer_size // 2:
            self.count_less_than_half += 1
        if self.count_less_than_half >= self.shrink_buffer_threshold:
            if nbytes < self.max_allgather_buffer_size // 2:
                self.max_allgather_buffer_size //= 2
                realloc = True
            self.count_less_than_half = 0
        if realloc:
            self.ag_buffer = torch.empty((self.stages, self.max_allgather_buffer_size), dtype=torch.int8,
                                         device=device)
        return self.ag_buffer[self.signal_target % self.stages][:nbytes]

    def forward(self, q, k_cache, v_cache, global_kv_lens, block_table,
                remote_partials: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                output_split: Optional[torch.Tensor] = None):
        """
        q: each rank has the same q
        k_cache / v_cache: this rank's shard of the paged cache
        global_kv_lens: [num_ranks, B] int32, every rank's local kv length
        block_table: this rank's block table
        remote_partials: the other ranks' (out, lse), see the module docstring
        output_split: optional caller-visible split partials ``[B, Hq, kv_split, Dv+1]`` as the reference allocates
            them on every call (:95-96); needs ``self.kv_split`` set to that split count (the reference's is 32)
        """
        batch = q.shape[0]
        assert global_kv_lens.shape[0] == self.num_ranks
        assert global_kv_lens.shape[1] == batch
        assert batch <= self.max_allowed_batch, f"Only support {self.max_allowed_batch} queries decode now"
        if self.num_ranks > 1 and remote_partials is None:
            raise RuntimeError(
                "num_ranks > 1 needs remote_partials: this build runs on one GPU and performs no allgather")

        if self.num_ranks == 1:
            # nothing to merge across ranks: the local decode writes the final output itself (split + combine, no
            # staging and no third launch); the ring position still advances once per call
            final_output = torch.empty([batch, self.num_q_heads, self.v_head_dim], dtype=q.dtype, device=q.device)
            gqa_fwd_batch_decode(q, k_cache, v_cache, self.workspace, [1] * batch, global_kv_lens[0], block_table,
                                 self.scale, soft_cap=self.soft_cap, output_split=output_split,
                                 output_combine=final_output, kv_split=self.kv_split)
            self.signal_target += 1
            return final_output

        pdtype = self.partial_dtype or q.dtype
        d1 = self.v_head_dim + 1
        itemsize = torch.empty((), dtype=pdtype).element_size()
        nbytes_per_rank = batch * self.num_q_heads * d1 * itemsize
        stage = self._stage(nbytes_per_rank * self.num_ranks, q.device)
        all_ranks_output_combine = stage.view(pdtype).view([self.num_ranks, batch, self.num_q_heads, d1])
        final_output = torch.empty([batch, self.num_q_heads, self.v_head_dim], dtype=q.dtype, device=q.device)
        r_out, r_lse = remote_partials
        assert r_out.shape[0] == self.num_ranks - 1 and r_lse.shape[0] == self.num_ranks - 1

        if not self.staged_exchange:
            # Two launches: the split kernel, and ONE combine that does what the reference does in three steps -- the
            # intra-rank combine (:107-110), the copy of its result into this rank's slot of the staged buffer
            # (:136-138: the slot a push to the other ranks would be sent from) and the inter-rank combine (:173-183),
            # reading the other ranks' partials where the caller holds them instead of from their slots; rank r
            # counts for sequence b iff global_kv_lens[r, b] > 0, as in the reference's kernel.
            gqa_fwd_batch_decode(q, k_cache, v_cache, self.workspace, None, global_kv_lens[self.rank], block_table,
                                 self.scale, soft_cap=self.soft_cap, output_split=output_split,
                                 output_combine=final_output, kv_split=self.kv_split,
                                 extra_partials=(r_out, r_lse),
                                 rank_merge=(global_kv_lens, self.rank, all_ranks_output_combine[self.rank]))
            self.signal_target += 1
            return final_output

        # The reference's own sequence of steps, slot by slot (what a real exchange would feed): local decode straight
        # into this rank's slot (the reference copies it there, :136-138) ...
        gqa_fwd_batch_decode_intra_rank(q, k_cache, v_cache, self.workspace, [1] * batch, global_kv_lens[self.rank],
                                        block_table, self.scale, soft_cap=self.soft_cap,
                                        output_split=output_split,
                                        output_combine=all_ranks_output_combine[self.rank], kv_split=self.kv_split)

        # ... stand-in for the allgather: the other ranks' partials arrive from the caller ...
        others = [r for r in range(self.num_ranks) if r != self.rank]
        for i, r in enumerate(others):
            all_ranks_output_combine[r, :, :, :self.v_head_dim].copy_(r_out[i])
            all_ranks_output_combine[r, :, :, self.v_head_dim].copy_(r_lse[i])
        self.signal_target += 1

        # ... and the final combine, launched as the reference launches its Triton kernel
        kernel_inter_rank_gqa_fwd_batch_decode_combine_kv[(batch, self.num_q_heads, 1)](
            all_ranks_output_combine,
            final_output,
            global_kv_lens,
            batch,
            self.num_q_heads,
            all_ranks_output_combine.stride(1),  # batch
            all_ranks_output_combine.stride(2),  # head
            all_ranks_output_combine.stride(0),  # num_ranks
            final_output.stride(0),  # batch
            final_output.stride(1),  # head
            self.num_ranks,  # split_kv
            512,  # BLOCK_DV
            self.v_head_dim,  # Lv
        )
        return final_output
