"""Flash-decode kernels: the names the reference exports for this path from
``python/triton_dist/kernels/nvidia/__init__.py:32-35``."""
from .flash_decode import (  # noqa: F401
    gqa_fwd_batch_decode,
    gqa_fwd_batch_decode_aot,
    gqa_fwd_batch_decode_intra_rank,
    gqa_fwd_batch_decode_intra_rank_aot,
    gqa_fwd_batch_decode_persistent,
    gqa_fwd_batch_decode_persistent_aot,
    kernel_inter_rank_gqa_fwd_batch_decode_combine_kv,
    inter_rank_combine,
    schedule_sequences,
    PreparedDecode,
    decode_plan,
    workspace_bytes,
    get_split_kv_algo_info,
    get_combine_kv_algo_info,
    get_triton_split_kv_algo_info,
    get_triton_combine_kv_algo_info,
)
from .kv_append import (  # noqa: F401
    apply_rotary_pos_emb,
    flash_attn_with_kvcache,
    paged_kv_append,
    rope_kv_append,
)

__all__ = [
    "apply_rotary_pos_emb",
    "flash_attn_with_kvcache",
    "paged_kv_append",
    "rope_kv_append",
    "get_triton_combine_kv_algo_info",
    "get_triton_split_kv_algo_info",
    "get_combine_kv_algo_info",
    "get_split_kv_algo_info",
    "gqa_fwd_batch_decode_aot",
    "gqa_fwd_batch_decode_intra_rank_aot",
    "gqa_fwd_batch_decode_intra_rank",
    "gqa_fwd_batch_decode_persistent_aot",
    "gqa_fwd_batch_decode_persistent",
    "gqa_fwd_batch_decode",
    "kernel_inter_rank_gqa_fwd_batch_decode_combine_kv",
    "inter_rank_combine",
    "schedule_sequences",
    "PreparedDecode",
    "decode_plan",
    "workspace_bytes",
]
