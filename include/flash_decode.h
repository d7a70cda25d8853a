/*
 * flash_decode.h -- C ABI of the MI355X (gfx950) flash-decode library.
 *
 * One shared library, libflash_decode_gfx950.so, exports exactly the symbols
 * declared here.  All pointers are DEVICE pointers (tensor.data_ptr()), all
 * strides are in ELEMENTS and 64-bit, `stream` is a hipStream_t passed as
 * void* (NULL = the legacy default stream).  Every call only enqueues work on
 * `stream`; nothing synchronises with the host and kv_lens is never read on the
 * host.  Return value: 0 on success, a negative fd_status otherwise;
 * fd_last_error() then describes the failure for the calling thread.  The
 * library never aborts the process.
 *
 * The shape of this ABI follows what the reference generates for its
 * ahead-of-time compiled Triton kernels: `CUresult <kernel>_ex(CUstream,
 * <pointers, scalars, strides...>, struct algo_info)`
 * (python/triton_dist/tools/compile_aot.py:330-333, 405-435), with the argument
 * order of the Triton signatures in
 * python/triton_dist/kernels/nvidia/flash_decode.py:70-94 (split) and :242-276
 * (combine).  The reference's pybind lambda drops the return code
 * (compile_aot.py:375-379); here it is returned to the caller.
 */
#ifndef FLASH_DECODE_H_
#define FLASH_DECODE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FD_ABI_VERSION 3

#if defined(__GNUC__)
#define FD_API __attribute__((visibility("default")))
#else
#define FD_API
#endif

typedef enum fd_status {
  FD_OK = 0,
  FD_ERR_INVALID_ARG = -1,  /* NULL pointer, non-positive size, bad enum            */
  FD_ERR_UNSUPPORTED = -2,  /* dtype / head_dim / group combination not compiled   */
  FD_ERR_ALIGNMENT = -3,    /* pointer or stride not aligned for 128-bit accesses  */
  FD_ERR_LAUNCH = -4,       /* the HIP runtime refused the launch                  */
  FD_ERR_TOO_LARGE = -5     /* size beyond a documented maximum                    */
} fd_status;

typedef enum fd_dtype {
  FD_F32 = 0,
  FD_F16 = 1,
  FD_BF16 = 2,
  FD_FP8_E4M3 = 3           /* OCP e4m3fn bit patterns, KV cache only              */
} fd_dtype;

typedef enum fd_path {
  FD_PATH_AUTO = 0,         /* MFMA for a 16-bit query with a KV cache of the same
                               dtype or fp8-e4m3; else VALU                        */
  FD_PATH_VALU = 1,         /* force the VALU dot-product kernel                   */
  FD_PATH_MFMA = 2          /* force MFMA; FD_ERR_UNSUPPORTED if not applicable    */
} fd_path;

typedef enum fd_combine_mode {
  FD_COMBINE_SPLIT = 0,     /* validity by split range, flash_decode.py:339-343    */
  FD_COMBINE_SPLIT_LSE = 1, /* same + merged LSE at column Dv of the output row,
                               flash_decode.py:446-449                             */
  FD_COMBINE_RANK = 2       /* validity by seqlens[s*batch+b] > 0,
                               flash_decode.py:513-515                             */
} fd_combine_mode;

/*
 * Compile-time constants of the reference's Triton kernels (kv_group_num,
 * q_head_num, NUM_KV_SPLITS, PAGE_SIZE, soft_cap, K_DIM, V_DIM --
 * flash_decode.py:153-164; the `algo_info` struct of the AOT path,
 * flash_decode.py:103-109) plus what a typed C ABI needs to know about the
 * buffers.  Zero-initialise, then fill.
 */
/*
 * Sequence-parallel decode on one rank (SpGQAFlashDecodeAttention.forward,
 * python/triton_dist/layers/nvidia/sp_flash_decode_layer.py:83-185): the reference runs the local decode with the
 * intra-rank combine (:107-110), copies the result into this rank's slot of a staged buffer [R, B, Hq, Dv + 1]
 * (:136-138), allgathers the other slots (:139) and launches the inter-rank combine over all of them (:173-183).
 * With this block in fd_params the combine of fd_decode / fd_decode_planned / fd_combine (split modes) does the last
 * three steps in its one launch: it merges the local split partials, writes that merge into `local_out` -- the slot a
 * push to the other ranks would be sent from -- and merges it with the extra partials, which then stand for the other
 * ranks in rank order (this rank left out), each counting for sequence b iff its rank holds tokens of it
 * (flash_decode.py:513-515).
 */
typedef struct fd_rank_merge {
  const int32_t* rank_lens; /* global_kv_lens [num_extra + 1, batch] int32 (device): every rank's local kv length     */
  int32_t this_rank;        /* the row of rank_lens that is this rank's own; extra e is rank e < this_rank ? e : e + 1 */
  int32_t local_dtype;      /* fd_dtype of local_out                                                                  */
  void* local_out;          /* NULL, or [batch, Hq, Dv + 1]: merge of the local split partials, LSE at column Dv       */
  int64_t stride_lb, stride_lh; /* element strides of local_out                                                        */
} fd_rank_merge;

typedef struct fd_params {
  int32_t q_heads;          /* Hq                                                  */
  int32_t kv_heads;         /* Hkv; Hq % Hkv == 0                                  */
  int32_t head_dim;         /* Dk (= the query's head dim); 64, 128 or 256; also Dv
                               unless v_head_dim says otherwise                    */
  int32_t page_size;        /* tokens per page (any value >= 1)                    */
  int32_t num_splits;       /* NUM_KV_SPLITS                                       */
  int32_t num_pages;        /* pages in the pool: table entries are clamped to
                               [0, num_pages) before use                           */
  int32_t max_pages_per_seq;/* block_table.shape[1]; kv_len is clamped to
                               max_pages_per_seq * page_size                       */
  int32_t q_dtype;          /* fd_dtype of q                                       */
  int32_t kv_dtype;         /* fd_dtype of k_cache / v_cache                       */
  int32_t mid_dtype;        /* fd_dtype of the split partials (out_split / mid_o)  */
  int32_t out_dtype;        /* fd_dtype of the combined output                     */
  float soft_cap;           /* <= 0: off                                           */
  const float* k_scale;     /* [Hkv] fp32 dequant scales, FD_FP8_E4M3 only         */
  const float* v_scale;     /* [Hkv]                                               */
  int32_t path;             /* fd_path                                             */
  int32_t waves_per_block;  /* 0 = choose; else 1, 2, 4 or 8 wave64 per (KV head, split) -- lowered where a kernel allows fewer */
  const int32_t* seq_order_lens; /* NULL, or [batch] with seq_order: kv_lens[seq_order[r]]
                               at index r (fd_kv_append writes it), so that a workgroup
                               fetches its sequence and its length in one round trip */
  int32_t split_align;      /* 0: the reference's split ranges, per = ceil(kv_len / S).
                               A power of two <= 4096: per is rounded up to a multiple of it,
                               so that splits start on tile boundaries (trailing splits may be
                               empty).  The result of a step is the same; the partials are not
                               the reference's.  fd_combine applies the same rule.          */
  int32_t split_adapt;      /* 0: every sequence is cut into num_splits ranges (the reference).
                               k > 0 (a power of two; needs split_align > 0; num_splits may be any count): a range of a sequence
                               of n tokens holds max(ceil(n / num_splits), min(ceil(n / k), w))
                               tokens, w = ceil(n / 8) kept within [1024, 4096] -- at least k
                               ranges; beyond that 1024-token ranges up to 8 of them, 8 ranges up
                               to 4096 tokens each, 4096-token ranges up to num_splits of them --
                               so the ranges of a sequence depend on its own length and not on a
                               block table sized for the longest context.  The other ranges of the sequence are empty; with more
                               than 16 splits fd_decode does not even write their partials.
                               fd_plan_min_splits gives k.  fd_combine applies the same rule. */
  int32_t max_kv_len;       /* 0: unknown.  Else an upper bound of kv_lens that the caller happens to
                               know on the host (serving engines do): fd_plan_splits and the launch
                               shape use it instead of the block table's capacity, so a table sized
                               for the longest context costs nothing.  A hint only: longer sequences
                               are still decoded in full.  No counterpart in the reference.     */
  int32_t seq_order_items;  /* 0: seq_order / seq_order_out is a per-sequence order ([batch], see
                               fd_schedule and fd_kv_append).  1: it is the work-item order of
                               fd_schedule_items, int32 [2 * batch * num_splits].             */
  int32_t v_head_dim;       /* 0: Dv = head_dim.  Else 64, 128 or 256: the V cache's head dim, which the
                               reference takes from the V cache independently of K's (V_DIM next to K_DIM,
                               flash_decode.py:162-163, 765-774).  Partials and outputs then have Dv (+1)
                               columns and fd_combine works on Dv.  Dv != Dk: fp32 / fp16 / bf16 caches.
                               A K head dim of 128 with a V head dim of 64 or 256, a 16-bit cache and up
                               to 16 query heads per KV head runs on the MFMA kernel, everything else on
                               the VALU kernel (FD_ERR_UNSUPPORTED for the other shapes with
                               FD_PATH_MFMA, with an fp8 cache and in fd_kv_append).            */
  const fd_rank_merge* rank_merge; /* NULL, or how the extra partials of this step stand for other ranks (above);
                               not with a ticket buffer (the fused combine)                                   */
} fd_params;

/*
 * Kernel (1): split-KV GQA paged decode.
 * Replaces kernel_gqa_fwd_batch_decode_split_kv
 * (python/triton_dist/kernels/nvidia/flash_decode.py:130-239) and its launch
 * (flash_decode.py:788-824 grid/arguments).
 *
 *  q           [batch, Hq, D]            stride_q_bs, stride_q_h, last dim contiguous
 *  k_cache     [num_pages, P, Hkv, D]    stride_k_tok = stride(-3), stride_k_h = stride(-2);
 *                                        the pool is indexed by flat token row page*P + n%P
 *  v_cache     same with stride_v_*
 *  out_split   [batch, Hq, S, *]         normalised partial outputs, mid_dtype, strides
 *                                        stride_o_bs / stride_o_h / stride_o_split
 *  lse_split   NULL: partial LSE (natural log) is stored at column D of the out_split row
 *              (the reference layout [B,Hq,S,D+1]); else fp32 [batch, Hq, S] contiguous
 *  block_table [batch, max_pages] int32, row stride stride_table_bs; only the first
 *              ceil(kv_len/P) entries of a row are read
 *  seq_order   NULL, or [batch] int32 from fd_schedule: workgroups are issued in this
 *              sequence order (longest first)
 *
 * Split s of sequence b covers tokens [per*s, min(per*s+per, kv_len)), per =
 * ceil(kv_len/S).  An empty split stores out = 0, lse = -inf.
 */
FD_API int fd_split_kv(void* stream, const void* q, const void* k_cache, const void* v_cache,
                void* out_split, float* lse_split, float sm_scale,
                const int32_t* block_table, const int32_t* kv_lens, int32_t batch,
                int64_t stride_q_bs, int64_t stride_q_h,
                int64_t stride_k_tok, int64_t stride_k_h,
                int64_t stride_v_tok, int64_t stride_v_h,
                int64_t stride_o_bs, int64_t stride_o_h, int64_t stride_o_split,
                int64_t stride_table_bs,
                const int32_t* seq_order, const fd_params* params);

/*
 * Kernel (2): LSE-weighted combine.  One entry point covers the reference's
 * three combine kernels:
 *   FD_COMBINE_SPLIT      kernel_gqa_fwd_batch_decode_combine_kv            flash_decode.py:308-360
 *   FD_COMBINE_SPLIT_LSE  kernel_intra_rank_gqa_fwd_batch_decode_combine_kv flash_decode.py:393-449
 *   FD_COMBINE_RANK       kernel_inter_rank_gqa_fwd_batch_decode_combine_kv flash_decode.py:482-532
 *                         as launched by layers/nvidia/sp_flash_decode_layer.py:173-183
 *
 *  mid_o     partials, params->mid_dtype, element strides stride_mid_ob (batch),
 *            stride_mid_oh (head), stride_mid_os (split or rank); `num_partials` of them
 *            (params->num_splits is ignored here)
 *  mid_lse   NULL: LSE of a partial is at column D of its mid_o row; else fp32 with
 *            contiguous layout [batch, Hq, num_partials]
 *  out       [batch, Hq, D(+1)] params->out_dtype, strides stride_obs / stride_oh
 *  lse_out   NULL or fp32 [batch, Hq]: merged natural-log LSE (always fp32)
 *  seqlens   kv_lens [batch] (split modes) or global_kv_lens [num_partials, batch] (rank mode).  In the
 *            split modes a length is clamped to params->max_pages_per_seq * params->page_size when both
 *            are set, exactly as the split kernels clamp it, so both agree on which ranges exist.
 *  extra_out / extra_lse / num_extra
 *            further always-valid partials merged in the same pass:
 *            extra_out [num_extra, batch, Hq, D] contiguous in params->out_dtype,
 *            extra_lse [num_extra, batch, Hq] fp32.  They stand in, on one GPU, for the
 *            partials the reference's allgather delivers from other ranks
 *            (sp_flash_decode_layer.py:136-145).
 *
 * A row with no valid partial yields out = 0, lse = -inf (the reference yields NaN).
 */
FD_API int fd_combine(void* stream, const void* mid_o, const float* mid_lse, void* out, float* lse_out,
               const int32_t* seqlens, int32_t batch, int32_t q_heads, int32_t num_partials,
               int64_t stride_mid_ob, int64_t stride_mid_oh, int64_t stride_mid_os,
               int64_t stride_obs, int64_t stride_oh, int32_t mode,
               const void* extra_out, const float* extra_lse, int32_t num_extra,
               const fd_params* params);

/*
 * One decode step: split-KV decode + combine.  Replaces the host wrappers
 * gqa_fwd_batch_decode (flash_decode.py:763-844: the two launches at :788 and
 * :826) and gqa_fwd_batch_decode_intra_rank (flash_decode.py:847-928) with
 * combine_mode FD_COMBINE_SPLIT / FD_COMBINE_SPLIT_LSE.  Arguments as for
 * fd_split_kv and fd_combine; out_split / lse_split are the partial workspace
 * (written, and readable by the caller afterwards).
 *
 *  out_split NULL is allowed when params->num_splits == 1 and num_extra == 0: the single split's
 *            normalised partial is the result, so the split kernel writes `out` (and lse_out,
 *            or the LSE column in FD_COMBINE_SPLIT_LSE mode -- not both) directly and no
 *            combine kernel is launched.
 *  tickets   NULL: two launches (split kernel, then combine kernel).
 *            Otherwise at least batch * q_heads int32, zero-initialised once by the
 *            caller and not shared by calls that may run concurrently: the combine is
 *            fused into the split kernel -- the workgroup that finishes a (sequence,
 *            head block) last merges that group's partials -- which saves the second
 *            launch.  The library leaves the counters at zero.  (The reference's fused
 *            variant, flash_decode.py:587-760, instead spins on a grid barrier word in
 *            `workspace` and needs all workgroups co-resident; nothing here waits.)
 */
FD_API int fd_decode(void* stream, const void* q, const void* k_cache, const void* v_cache,
              void* out_split, float* lse_split, void* out, float* lse_out, float sm_scale,
              const int32_t* block_table, const int32_t* kv_lens, int32_t batch,
              int64_t stride_q_bs, int64_t stride_q_h,
              int64_t stride_k_tok, int64_t stride_k_h,
              int64_t stride_v_tok, int64_t stride_v_h,
              int64_t stride_o_bs, int64_t stride_o_h, int64_t stride_o_split,
              int64_t stride_table_bs, int64_t stride_obs, int64_t stride_oh,
              const int32_t* seq_order, int32_t combine_mode,
              const void* extra_out, const float* extra_lse, int32_t num_extra,
              int32_t* tickets, const fd_params* params);

/*
 * The launch policy of a decode step, in one place.  NUM_KV_SPLITS is a tuning constant in the reference (32 unless
 * the caller says otherwise, flash_decode.py:779) and its wrappers allocate their partial buffers themselves
 * (flash_decode.py:783-786); a caller that does not hand in `output_split` never sees the partials, so everything
 * about them -- how many, which token ranges, their element type, where they live, in which order the work is issued
 * -- is the library's choice.  fd_plan_decode reports that choice, fd_decode_planned applies it; a binding needs no
 * policy of its own.
 */
typedef enum fd_step_flags {
  FD_STEP_EXACT_SPLITS = 1,   /* exactly params->num_splits splits (the reference's ranges, rounded up to whole tiles)
                                 instead of the library's count; the partials still live in the workspace           */
  FD_STEP_SCHEDULE = 2,       /* the scheduled variant (gqa_fwd_batch_decode_persistent, flash_decode.py:931-1005):
                                 the step ranks its work on the device first -- (sequence, range) work items up to
                                 192 sequences, whole sequences up to 4096 -- and issues it largest first.  A step of
                                 64 sequences or more does so whether this flag is set or not                        */
  FD_STEP_NO_ORDER = 4,       /* never rank: workgroups are issued in index order                                    */
  FD_STEP_FUSED = 8,          /* fd_plan_decode only: plan for fd_decode with a ticket buffer (fp32 partials, no
                                 work items, no direct single-split output)                                          */
  FD_STEP_LSE_TWICE = 16,     /* fd_plan_decode only: the caller wants the merged LSE both in the output's column and
                                 in lse_out, which the direct single-split output cannot provide                     */
  FD_STEP_CALLER_PARTIALS = 32,/* fd_plan_decode only: the caller owns the partials ([B, Hq, S, Dv + 1] in
                                 params->mid_dtype, flash_decode.py:783): exactly params->num_splits splits with the
                                 reference's ranges; the plan only says how the step is issued                       */
  FD_STEP_ORDER_FROM_APPEND = 64 /* fd_plan_decode only: an fd_kv_append launch precedes the step and can compute the
                                 issue order in its trailing workgroups at no launch of its own; order_kind then
                                 says which kind to ask it for (from 16 sequences on)                                */
} fd_step_flags;

typedef enum fd_order_kind {
  FD_ORDER_NONE = 0,          /* index order                                                                        */
  FD_ORDER_SEQUENCES = 1,     /* fd_schedule: [batch] sequence indices, longest first                               */
  FD_ORDER_ITEMS = 2          /* fd_schedule_items: [2 * batch * num_splits] work items and their lengths           */
} fd_order_kind;

typedef struct fd_launch_plan {
  int32_t num_splits;         /* grid slots (ranges) per sequence                                                   */
  int32_t split_adapt;        /* fd_params.split_adapt of the step                                                  */
  int32_t split_align;        /* fd_params.split_align of the step                                                  */
  int32_t mid_dtype;          /* fd_dtype of the partials                                                           */
  int32_t direct;             /* 1: one split and nothing else to merge -- the split kernel writes `out` itself, no
                                 partials, no combine launch                                                        */
  int32_t order_kind;         /* fd_order_kind of the scheduling launch the step makes itself (FD_ORDER_NONE when the
                                 caller brings an order, asks for none, or the batch is not worth one)              */
  int32_t mfma;               /* 1: an MFMA split kernel, 0: the VALU kernel                                        */
  int32_t tile;               /* tokens per tile of that kernel                                                     */
  int32_t waves_per_head;     /* waves that share the tokens of one (KV head or head block, work item)              */
  int32_t members;            /* sibling KV heads (or head blocks, or V halves) per workgroup                       */
  int32_t chunk;              /* consecutive splits one workgroup walks (1: a workgroup per split)                  */
  int32_t head_block;         /* query-head slots a wave serves                                                     */
  int32_t grid[3];            /* launch grid of the split kernel                                                    */
  int32_t store_through;      /* 1: partials are written through to memory                                          */
  int32_t max_kv_len;         /* the length hint the step is planned with (0: the block table's capacity)           */
  int32_t reserved;
  int64_t partial_bytes;      /* partials in the workspace ([batch, Hq, num_splits, Dv] in mid_dtype)               */
  int64_t lse_bytes;          /* their fp32 LSEs ([batch, Hq, num_splits])                                          */
  int64_t order_bytes;        /* the issue order                                                                    */
  int64_t workspace_bytes;    /* all of it, each part on a 256-byte boundary                                        */
} fd_launch_plan;

/*
 * The plan of a decode step for a shape known on the host (kv_lens is never read): split count and ranges, partial
 * type, whether a scheduling launch is part of the step, the launch shape of the split kernel (for contiguous caches:
 * token stride = kv_heads * head_dim, head stride = head_dim) and the workspace the step needs.  params->num_splits is
 * the caller's hint -- <= 0: none; the reference's callers pass 32 -- which bounds the count from below only where it
 * exceeds the library's own bound max(32, min(256, capacity / 512)); with FD_STEP_EXACT_SPLITS or
 * FD_STEP_CALLER_PARTIALS it is the count (<= 0: 32).  params->mid_dtype, split_align, split_adapt and seq_order_items are
 * outputs here, not inputs (mid_dtype is an input with FD_STEP_CALLER_PARTIALS).  params->max_kv_len (rounded up to
 * 1024 tokens, so that a growing batch does not re-plan at every step) replaces the block table's capacity as the
 * longest sequence to plan for.  Returns 0 or a negative fd_status.  No counterpart in the reference.
 */
FD_API int fd_plan_decode(const fd_params* params, int32_t batch, int32_t num_extra, int32_t flags,
                          fd_launch_plan* plan);

/* fd_plan_decode(...).workspace_bytes, or a negative fd_status: what fd_decode_planned needs for this shape. */
FD_API int64_t fd_workspace_bytes(const fd_params* params, int32_t batch, int32_t num_extra, int32_t flags);

/*
 * Every argument of a planned decode step in one block, so that a binding can keep it between steps and touch only
 * what changed (the reference's wrappers marshal two dozen arguments per launch, flash_decode.py:788-844).
 */
typedef struct fd_decode_args {
  const void* q;              /* [batch, Hq, D]                                                                     */
  const void* k_cache;        /* [num_pages, P, Hkv, D]                                                             */
  const void* v_cache;
  void* workspace;            /* at least fd_workspace_bytes(...) bytes, 256-byte aligned, the caller's; its contents
                                 mean nothing between calls; calls that may overlap need one each                    */
  int64_t workspace_bytes;
  void* out;                  /* [batch, Hq, Dv] (+ 1 column with FD_COMBINE_SPLIT_LSE)                              */
  float* lse_out;             /* NULL or fp32 [batch, Hq]                                                            */
  const int32_t* block_table;
  const int32_t* kv_lens;
  const int32_t* seq_order;   /* NULL: the library ranks the work itself where that pays; else an order the caller
                                 computed (fd_schedule, fd_schedule_items with the plan's split fields, fd_kv_append),
                                 params.seq_order_items / seq_order_lens describing it                              */
  const void* extra_out;      /* as for fd_combine                                                                   */
  const float* extra_lse;
  int64_t stride_q_bs, stride_q_h, stride_k_tok, stride_k_h, stride_v_tok, stride_v_h;
  int64_t stride_table_bs, stride_obs, stride_oh;
  float sm_scale;
  int32_t batch;
  int32_t combine_mode;       /* FD_COMBINE_SPLIT or FD_COMBINE_SPLIT_LSE                                            */
  int32_t num_extra;
  int32_t flags;              /* fd_step_flags: FD_STEP_EXACT_SPLITS, FD_STEP_SCHEDULE, FD_STEP_NO_ORDER              */
  fd_params params;           /* num_splits is the hint described at fd_plan_decode                                  */
} fd_decode_args;

/*
 * One decode step as the library plans it: what gqa_fwd_batch_decode / _intra_rank / _persistent
 * (flash_decode.py:763-844, 847-928, 931-1005) do when the caller passes no output_split -- the wrappers there pick
 * 32 splits, allocate the partials and launch split and combine; here the library picks the plan of fd_plan_decode,
 * keeps partials, LSEs and the issue order in `workspace`, and enqueues the scheduling launch (if the plan has one),
 * the split kernel and the combine kernel (unless the plan is direct).  The result is the same for every plan.
 * Returns FD_ERR_INVALID_ARG when the workspace is missing, misaligned or too small (the message names the size).
 */
FD_API int fd_decode_planned(void* stream, const fd_decode_args* args);

/*
 * fd_decode for callers that cannot allocate device memory -- code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose wrappers allocate
 * their partial buffers with torch.empty on every call, flash_decode.py:783-786).  Same step and same kernels
 * as fd_decode with tickets == NULL, but the split partials (fp32 [batch, Hq, num_splits, head_dim] and their
 * LSEs, params->mid_dtype is ignored) live in a static device array inside the library instead of in
 * out_split / lse_split; the call itself allocates nothing (no hipMalloc, no hipFree, no allocating library
 * routine).  Limits and rules:
 *   - batch * q_heads * num_splits * (head_dim + 1) * 4 bytes must not exceed FD_NOALLOC_SCRATCH_BYTES, else
 *     FD_ERR_TOO_LARGE (nothing is launched); fd_plan_splits keeps all five benchmark configurations well
 *     inside it;
 *   - every GPU the library is used on holds its own copy of the array until the process ends;
 *   - all calls on one GPU share that array: calls that may overlap on one GPU (different streams, graphs
 *     replayed concurrently) race on it -- serialise them, or use fd_decode with workspaces of your own;
 *     the array keeps the last call's partials, which the next call overwrites before it reads them;
 *   - the first call on a device looks up the array's device address (hipGetSymbolAddress, once per device): make
 *     that call outside a stream capture -- one eager step before the graph is recorded -- since a symbol lookup is
 *     module set-up and not a capturable operation; every later call only launches kernels.
 */
#define FD_NOALLOC_SCRATCH_BYTES (16u << 20)
FD_API int fd_decode_noalloc(void* stream, const void* q, const void* k_cache, const void* v_cache,
              void* out, float* lse_out, float sm_scale,
              const int32_t* block_table, const int32_t* kv_lens, int32_t batch,
              int64_t stride_q_bs, int64_t stride_q_h,
              int64_t stride_k_tok, int64_t stride_k_h,
              int64_t stride_v_tok, int64_t stride_v_h,
              int64_t stride_table_bs, int64_t stride_obs, int64_t stride_oh,
              const int32_t* seq_order, int32_t combine_mode,
              const void* extra_out, const float* extra_lse, int32_t num_extra,
              const fd_params* params);

/*
 * Kernel (3): work scheduler.  Writes seq_order[batch]: sequence indices sorted by
 * kv_len descending (ties by index), computed on the device from kv_lens, so that
 * fd_split_kv issues the longest sequences' workgroups first and the hardware
 * dispatcher back-fills CUs with the short ones.  The reference's only scheduler is
 * the static round-robin of its persistent kernel (flash_decode.py:632-640).
 * With params->split_adapt > 0 the split kernels issue all sequences' first ranges, then all second
 * ranges, and so on, so this order only ranks the sequences inside such a slab; fd_schedule_items
 * (below) orders the individual ranges and is the better choice there (config 4: 664 vs 705 us).
 */
FD_API int fd_schedule(void* stream, const int32_t* kv_lens, int32_t batch, int32_t* seq_order);

/*
 * Kernel (3), per work item: the issue order of the (sequence, range) items of a decode step with
 * params->num_splits, split_align and split_adapt, for batches of up to 1024 sequences.
 * item_order[k], k < batch * num_splits, = sequence | range << 16: first the non-empty ranges, sequence by
 * sequence in descending (tokens per range, length) order (largest item first), then the empty ranges;
 * item_order[batch * num_splits + k] = the length of item k's sequence.  fd_decode / fd_split_kv take it as
 * seq_order with params->seq_order_items = 1 (same num_splits, split_align, split_adapt, max_pages_per_seq and
 * page_size; kv_lens unchanged in between).  With ranges that follow each sequence's own length this is what keeps the
 * busy workgroups of a ragged batch contiguous in issue order AND largest-first.  The reference has no counterpart
 * (static round-robin, flash_decode.py:632-640).
 */
FD_API int fd_schedule_items(void* stream, const int32_t* kv_lens, int32_t batch, int32_t* item_order,
                             const fd_params* params);

/*
 * How many splits the library would use for a decode step whose partials the caller does
 * not look at.  NUM_KV_SPLITS is a tuning constant in the reference (flash_decode.py:779:
 * 32 unless the caller says otherwise); the result of a step does not depend on it.  When
 * the partial workspace is internal, fewer and longer splits mean fewer workgroup
 * prologues and fewer partials for the combine.  Returns a count of at most
 * params->num_splits: the smallest power of two that (1) gives one workgroup per CU (256) with
 * the workgroup at its full width (sibling KV heads that share 512 bytes of a token row, or head
 * blocks of one KV head) -- or, where no power of two does because the heads do not divide the CU
 * count (12 KV heads), the count just under one workgroup per CU (42 with sibling heads, 21 without
 * them where a split would otherwise hold fewer than 512 tokens) --, raised (2) until the workgroups
 * are a whole number per CU or at
 * least four per CU, as long as a split of a full-length sequence keeps 512 tokens, and (3) in
 * a batch until no split of a full-length sequence exceeds 4096 tokens or 32 splits are reached (VALU kernel: about
 * 2048 waves with four per split instead of (1) and (2)); or a negative fd_status.
 * A caller that passes its own out_split to fd_decode / fd_split_kv keeps exactly
 * params->num_splits splits with the reference's ranges.
 */
FD_API int fd_plan_splits(const fd_params* params, int32_t batch);

/*
 * The part of fd_plan_splits' count that the shape needs to fill the chip (its rules 1 and 2, or the VALU
 * rule), without the part that only bounds the length of a split in a batch: the value for
 * fd_params.split_adapt.  No counterpart in the reference (one split count for all sequences,
 * flash_decode.py:193-195).  Returns the count rounded up to a power of two (>= 1, not clamped to params->num_splits) or a negative
 * fd_status.
 */
FD_API int fd_plan_min_splits(const fd_params* params, int32_t batch);

/*
 * What the reference's attention block does to q and k between the QKV projection and the
 * cache update (python/triton_dist/layers/amd/tp_attn.py:252-264), applied on the way in:
 *
 *  1. optional per-head RMS norm over head_dim (`layer_norm`, tp_attn.py:52-59, 252-258):
 *     y = x * rsqrt(mean(x^2) + eps) * w in fp32, rounded to the activation dtype;
 *  2. optional rotary position embedding (apply_rotary_pos_emb, tp_attn.py:72-125 kernel,
 *     :128-160 launch, :232-241 and :263-264 call sites): out[i] = x[i]*cos[i] - x[i+D/2]*sin[i],
 *     out[i+D/2] = x[i+D/2]*cos[i] + x[i]*sin[i] for i < D/2, in fp32, each product and sum
 *     rounded separately, the result rounded to the activation dtype.
 *
 * K rows get both before they are stored; q rows (if given) get both into q_out.
 */
typedef struct fd_qk_prep {
  const float* cos_sin;       /* NULL (no rotation), or [max_positions, D] fp32: D/2 cosines
                                 then D/2 sines per row (tp_attn.py:62-69), 16-byte aligned  */
  int64_t stride_cos_sin;     /* row stride in elements                                    */
  const void* position_ids;   /* [batch, new_tokens]                                       */
  int32_t position_dtype;     /* 0: int32, 1: int64                                        */
  int32_t max_positions;      /* positions are clamped into [0, max_positions)             */
  int64_t stride_pos_b, stride_pos_t;
  const void* q;              /* NULL, or [batch, new_tokens, Hq, D] in params->q_dtype     */
  void* q_out;                /* processed q, same dtype; may be q itself                  */
  int64_t stride_q_b, stride_q_t, stride_q_h;
  int64_t stride_qo_b, stride_qo_t, stride_qo_h;
  const void* q_norm_weight;  /* NULL (no norm of q), or [D] in params->q_dtype, 16-byte aligned */
  const void* k_norm_weight;  /* NULL (no norm of k), or [D] in params->q_dtype, 16-byte aligned */
  float q_norm_eps, k_norm_eps;
} fd_qk_prep;

/*
 * The step before the decode: appends `new_tokens` tokens of K and V per sequence to the
 * paged pool at logical positions kv_lens[b] .. kv_lens[b]+new_tokens-1, converting from the
 * activation dtype (params->q_dtype) to the cache dtype (params->kv_dtype; FD_FP8_E4M3 stores
 * clamp(x / scale[kv head], +-448) rounded to nearest even, with params->k_scale / v_scale).
 * The pool layout [num_pages, P, Hkv, D] with an int32 block table is the one the decode
 * reads (python/triton_dist/test/nvidia/test_decode_attn.py:150-156); the reference itself
 * only has a dense cache whose update is a slice assignment
 * (python/triton_dist/models/kv_cache.py:43-50, called at layers/amd/tp_attn.py:265), which
 * is this layout with one page per sequence.  With `prep`, K is normalised and / or rotated
 * before it is stored and, if prep->q is given, so is Q in the same launch.
 *
 *  k_new, v_new  [batch, new_tokens, Hkv, D], element strides stride_*n_b / _t / _h, last dim
 *                contiguous, 16-byte aligned rows.  Both NULL: only prep->q is processed.
 *  kv_lens       [batch] tokens already in the cache (not modified)
 *  kv_lens_out   NULL, or [batch] (not kv_lens itself): min(kv_lens[b] + new_tokens, capacity)
 *  seq_order_out NULL, or [2 * batch] int32 (batch <= 4096): entries [0, batch) are what
 *                fd_schedule would return for kv_lens_out -- the issue order for the decode that
 *                follows, computed by a few trailing workgroups of this launch instead of a
 *                launch of its own -- and entries [batch, 2 * batch) are kv_lens_out in that
 *                order (params->seq_order_lens of the decode)
 *  A token whose position is at or beyond max_pages_per_seq * page_size is not written.
 */
FD_API int fd_kv_append(void* stream, const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                 const int32_t* block_table, const int32_t* kv_lens, int32_t* kv_lens_out,
                 int32_t* seq_order_out, int32_t batch, int32_t new_tokens,
                 int64_t stride_kn_b, int64_t stride_kn_t, int64_t stride_kn_h,
                 int64_t stride_vn_b, int64_t stride_vn_t, int64_t stride_vn_h,
                 int64_t stride_k_tok, int64_t stride_k_h,
                 int64_t stride_v_tok, int64_t stride_v_h,
                 int64_t stride_table_bs, const fd_qk_prep* prep, const fd_params* params);

/* Message for the last non-zero status returned on this thread ("" if none). */
FD_API const char* fd_last_error(void);

/* FD_ABI_VERSION the library was built with. */
FD_API int fd_abi_version(void);

/*
 * Identifies the sources the library was built from: the build script passes a hash of every source and header
 * (FD_BUILD_ID), "unknown" for a build made some other way.  A loader compares it with the hash of the sources
 * it sees to detect a stale library (triton-distributed_amd/build.py::ensure_built).  No counterpart in the
 * reference.
 */
FD_API const char* fd_build_id(void);

#ifdef __cplusplus
}
#endif
#endif /* FLASH_DECODE_H_ */
