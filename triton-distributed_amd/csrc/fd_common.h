// Shared device-side types and helpers for the gfx950 flash-decode kernels.
//
// Everything here is written for CDNA4 wave64: "lane" is 0..63, a "row" of a
// wave is 16 consecutive lanes (the granularity of the 16x16 MFMA operand
// layouts), cross-lane traffic uses ds_bpermute via __shfl*.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>
#include <stdint.h>

#include "../../include/flash_decode.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

#define FD_LOG2E 1.4426950408889634f
#define FD_LN2 0.6931471805599453f

// Arguments of the split-KV kernels (one struct passed by value in kernarg space).
struct SplitArgs {
  const void* q;
  const void* k;
  const void* v;
  void* out;             // partial outputs, mid_dtype
  float* lse;            // nullptr: LSE at column D of the out row
  const int32_t* bt;
  const int32_t* kv_lens;
  const int32_t* order;  // nullptr: identity
  const int32_t* order_lens;  // nullptr, or kv_lens[order[r]] at index r
  int32_t order_items;   // 1: order holds batch * S work items (sequence | range << 16), order_lens their lengths
  const float* k_scale;
  const float* v_scale;
  int64_t sq_b, sq_h, sk_t, sk_h, sv_t, sv_h, so_b, so_h, so_s, sbt;
  float sm_scale, soft_cap;
  int32_t batch, Hq, Hkv, G, S, P, max_pages, num_pages;
  uint32_t div_magic, div_shift;  // n / P == (uint64(n) * div_magic) >> div_shift for 0 <= n < 2^31
  int32_t q_dtype, mid_dtype;
  int32_t nhb;      // head blocks per KV head
  int32_t hbsz;     // query heads per head block (MFMA kernels: up to 16, or up to 32 with two column blocks per wave)
  int32_t hpw;      // adjacent KV heads per workgroup (one wave each; x token sub-ranges = waves)
  int32_t nsub;     // token sub-ranges of a split (waves per KV head); the workgroup has hpw * nsub waves
  int32_t member_hb;  // 1: the hpw members of a workgroup are head blocks of ONE KV head (groups with more query
                      // heads than a wave serves: the blocks read the same K/V rows in step, so the rows come
                      // from HBM once)
  int32_t grid_x;   // workgroups per (sequence, split)
  int32_t vec_out;  // 1: four values of an out row go out in one store -- fp32 rows (any 4-byte boundary will do for a
                    // 128-bit store), 16-bit rows that start on multiples of four elements (64-bit stores)
  int32_t no_lse;   // 1: the partial LSE is not stored (single split written straight to a [B,Hq,D] output)
  uint32_t s_magic, s_shift;      // n / S, same scheme as div_magic
  int32_t per_mask;               // split_align - 1 (0: the reference's ranges): tokens per split are rounded up
  int32_t adapt;                  // fd_params.split_adapt: ranges per sequence by its own length (0: always S)
  int32_t skip_empty;             // 1: a workgroup whose range is empty writes nothing (the combine knows the ranges)
  int32_t chunk;                  // consecutive splits one workgroup walks (1: one split per workgroup).  Above 1 every
                                  // wave owns whole splits -- ceil(chunk / nsub) consecutive ones -- and stores one
                                  // partial per split itself, so the caller sees exactly S partials in the reference
                                  // layout while the chip sees S / chunk long work items
  int32_t store_through;          // 1: partials are written through to memory (sc0 sc1) instead of being left dirty in
                                  // the XCD's L2 until the kernel ends; pays off for tens of MB of partials
  int32_t park;                   // chunked work items: finished partials a wave parks in LDS besides its last one
                                  // (which goes to the wave's tile staging buffer)
  // V head dim != K head dim on the head_dim-128 MFMA kernel.  dv = V head dim (the column of an in-row LSE).
  // v_members = 2 (dv 256): a workgroup member is a (KV head, 128-column half of the V rows) pair -- two waves share
  // K and the softmax and each accumulates and stores its own half.  v_chunk_mask = 7 (dv 64): the 16 lanes of a
  // wave row fetch the eight 16-byte chunks of a 128-byte V row twice, and only v_cols = 64 columns are stored.
  int32_t dv, v_members, v_chunk_mask, v_cols;
  int32_t park_bytes;             // LDS bytes of one parked partial: the finished one -- fp32 LSEs of the wave's head
                                  // slots, then the normalised rows [head][D] of its real heads in mid_dtype
  // Fused combine (tickets != nullptr): the workgroup that finishes a (sequence, head block) last
  // merges its S partials (+ num_extra further ones) into the final output.
  int32_t* tickets;      // one zero-initialised counter per (sequence, KV head, head block); left at zero
  void* fout;            // [batch, Hq, D(+1)] out_dtype
  float* flse;           // nullptr or [batch, Hq] fp32
  const void* extra_out; // [num_extra, batch, Hq, D] out_dtype
  const float* extra_lse;
  int64_t sfo_b, sfo_h;
  int32_t out_dtype, num_extra, lse_column;
};

struct CombineArgs {
  const void* mid_o;
  const float* mid_lse;  // nullptr: LSE at column D of the mid_o row
  void* out;
  float* lse_out;        // nullptr or [batch, Hq] fp32
  const int32_t* seqlens;
  const void* extra_out;
  const float* extra_lse;
  int64_t s_mb, s_mh, s_ms, s_ob, s_oh;
  int32_t batch, Hq, D, num_partials, num_extra, mode, mid_dtype, out_dtype;
  int32_t vec_mid;  // 1: every mid_o row starts on a multiple of four elements (128-bit loads of fp32, 64-bit loads of
                    // 16-bit partials)
  int32_t cg_shift; // log2 of the 128-bit column groups a workgroup of the general kernel covers (set by the launcher)
  int32_t per_mask;           // as SplitArgs::per_mask, for the validity of split ranges
  int32_t adapt;              // as SplitArgs::adapt
  uint32_t s_magic, s_shift;  // n / num_partials, as in SplitArgs
  int32_t all_slots_written;  // 1: the partials come from this library's split kernel in the same call, which
                              // writes every slot (empty splits as out = 0, lse = -inf)
  int64_t capacity;           // split modes: lengths are clamped to it, as the split kernels clamp them to the block
                              // table's capacity (stand-alone calls that do not know a table: 2^31 - 1 - num_partials)
  // fd_rank_merge: the extras stand for the other ranks of a sequence-parallel decode
  const int32_t* rank_lens;   // nullptr, or [num_extra + 1, batch]: extra e counts iff its rank's length is > 0
  int32_t this_rank;          // the row of rank_lens that is not an extra
  int32_t local_dtype;
  void* local_out;            // nullptr, or [batch, Hq, D + 1]: the merge of the split partials alone, LSE at column D
  int64_t s_lb, s_lh;
};

// How a decode step cuts a sequence into ranges: what the scheduler needs to know of it.
struct RangePlan {
  int32_t S;                  // ranges per sequence (grid slots)
  uint32_t s_magic, s_shift;  // n / S
  int32_t per_mask, adapt;    // as in SplitArgs
};

// Arguments of the KV-append / rotary kernel.
struct AppendArgs {
  const void* k_new;     // nullptr: no append (rotary of q only)
  const void* v_new;
  void* k_cache;
  void* v_cache;
  const int32_t* bt;
  const int32_t* kv_lens;
  int32_t* kv_lens_out;  // nullptr or [batch]
  int32_t* seq_order;    // nullptr or [2 * batch]: sequences ranked by grown length, longest first, then those lengths
  int32_t* items;        // nullptr or [2 * batch * ranges.S]: work items of the decode that follows (fd_schedule_items)
  RangePlan ranges;      // how that decode cuts a sequence into ranges (items only)
  int32_t data_blocks;   // workgroups that move data; the ones after them compute seq_order
  int32_t rank_shift;    // log2 of the lanes that share a sequence in those (fd_rank_shift)
  const float* k_scale;
  const float* v_scale;
  int64_t skn_b, skn_t, skn_h, svn_b, svn_t, svn_h, sk_t, sk_h, sv_t, sv_h, sbt;
  int32_t batch, T, Hq, Hkv, D, P, max_pages, num_pages;
  const float* cos_sin;  // nullptr: no rotation
  const void* pos;       // [batch, T] int32 or int64
  int64_t s_cs, sp_b, sp_t;
  int32_t pos_i64, max_pos;
  const void* q;         // nullptr: no query rows
  void* q_out;
  int64_t sq_b, sq_t, sq_h, sqo_b, sqo_t, sqo_h;
  const void* qn_w;      // nullptr: q is not normalised; else [D] RMS-norm weight in the activation dtype
  const void* kn_w;
  float qn_eps, kn_eps;
};

// ---------------------------------------------------------------- scalar conversions

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t lo16) { return __uint_as_float(lo16 << 16); }
__device__ __forceinline__ float f16_bits_to_f32(uint32_t lo16) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)lo16);
}

__device__ __forceinline__ float load_as_f32(const void* p, int64_t idx, int dtype) {
  switch (dtype) {
    case FD_F32: return ((const float*)p)[idx];
    case FD_F16: return (float)((const _Float16*)p)[idx];
    default: return (float)((const __bf16*)p)[idx];
  }
}

__device__ __forceinline__ void store_from_f32(void* p, int64_t idx, int dtype, float x) {
  switch (dtype) {
    case FD_F32: ((float*)p)[idx] = x; break;
    case FD_F16: ((_Float16*)p)[idx] = (_Float16)x; break;
    default: ((__bf16*)p)[idx] = (__bf16)x; break;
  }
}

// Agent-scope coherent accesses.  Each XCD has its own L2, and an ordinary store may sit there
// unseen by the other XCDs until the kernel ends; a relaxed agent-scope atomic store is written
// through, a relaxed agent-scope atomic load bypasses the local L2.  Workgroups on different
// XCDs exchange partial results through these instead of cache-wide release/acquire fences,
// which write back and invalidate a whole L2 each time.
__device__ __forceinline__ void store_f32_agent(float* p, float x) {
  __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_f32_agent(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ f32x2 load_f32x2_agent(const float* p) {  // p 8-byte aligned
  const uint64_t v = __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return __builtin_bit_cast(f32x2, v);
}

__device__ __forceinline__ float fd_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fd_log2(float x) { return __builtin_amdgcn_logf(x); }

// soft_cap * tanh(x / soft_cap), tanh(y) = 1 - 2 / (1 + e^{2y})
__device__ __forceinline__ float fd_softcap(float x, float cap, float inv_cap) {
  float e = fd_exp2(2.0f * FD_LOG2E * x * inv_cap);
  return cap * (1.0f - 2.0f / (1.0f + e));
}

// K/V rows are read exactly once per decode step: non-temporal loads keep them from being allocated in the
// caches on their way through (measured with a pure-read probe on the same access pattern: 6.97 vs 6.15 TB/s).
__device__ __forceinline__ u32x4 load_stream_b128(const void* p) { return __builtin_nontemporal_load((const u32x4*)p); }
__device__ __forceinline__ u32x2 load_stream_b64(const void* p) { return __builtin_nontemporal_load((const u32x2*)p); }

// Vectors in global memory that are only known to start on a 4-byte boundary: global loads and stores of two or four
// dwords need no more than dword alignment on this target.
typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

// Four consecutive values of a partial row that starts on a multiple of four elements (SplitArgs::vec_out): one
// 128-bit store for fp32, one 64-bit store of four packed values for fp16 / bf16.  through: written through to memory
// (sc0 sc1).  The write-through form is inline assembly, which the compiler does not count in vmcnt: only for stores
// that no vector-memory load of the same wave follows.  Nor does the compiler's hazard pass look inside it: a store of
// more than 64 bits needs wait states before a VALU instruction may overwrite its data registers, so the 128-bit
// forms carry their own s_nop.
__device__ __forceinline__ void store_partial4(void* base, int64_t off, int dtype, f32x4 o, bool through) {
  if (dtype == FD_F32) {
    float* p = (float*)base + off;
    if (through) {
      asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(o) : "memory");
    } else {
      *(f32x4_a4*)p = o;   // fp32 rows count as vector rows on any 4-byte boundary
    }
  } else {
    const f32x2 lo = {o[0], o[1]}, hi = {o[2], o[3]};
    u32x2 w;
    if (dtype == FD_F16) {
      w[0] = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, f16x2));
      w[1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, f16x2));
    } else {
      w[0] = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, bf16x2));
      w[1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, bf16x2));
    }
    uint16_t* p = (uint16_t*)base + off;
    if (through) {
      asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1" ::"v"(p), "v"(w) : "memory");
    } else {
      *(u32x2*)p = w;
    }
  }
}

// One value, with the same write-through option and the same restriction as store_partial4.
__device__ __forceinline__ void store_partial1(void* base, int64_t off, int dtype, float x, bool through) {
  if (!through) { store_from_f32(base, off, dtype, x); return; }
  if (dtype == FD_F32) {
    asm volatile("global_store_dword %0, %1, off sc0 sc1" ::"v"((float*)base + off), "v"(x) : "memory");
  } else {
    const uint32_t w = dtype == FD_F16 ? (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x)
                                       : (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)x);
    asm volatile("global_store_short %0, %1, off sc0 sc1" ::"v"((uint16_t*)base + off), "v"(w) : "memory");
  }
}
// Orders LDS accesses of one wave: lanes of a wave exchange data through LDS
// without a workgroup barrier (the LDS queue of a wave is in order); this only
// stops the compiler from moving accesses across the point.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Fetches everything a wave needs before its first K/V request from the kernel-argument segment NOW, as one
// batch of scalar loads.  Left to itself the compiler loads each field right before its first use, which puts
// half a dozen dependent scalar-load round trips in front of the first table lookup; a value pinned in an SGPR
// here has to be loaded here (input-only constraints: the values themselves, and what the compiler knows about the
// pointers, stay as they are).
__device__ __forceinline__ void fd_fetch_args_now(const SplitArgs& a) {
#define FD_PIN(f) asm volatile("" ::"s"(a.f))
  FD_PIN(q); FD_PIN(k); FD_PIN(v); FD_PIN(bt); FD_PIN(kv_lens); FD_PIN(order); FD_PIN(order_lens);
  FD_PIN(sq_b); FD_PIN(sq_h); FD_PIN(sk_t); FD_PIN(sk_h); FD_PIN(sv_t); FD_PIN(sv_h); FD_PIN(sbt);
  FD_PIN(sm_scale); FD_PIN(batch); FD_PIN(G); FD_PIN(S); FD_PIN(P); FD_PIN(max_pages); FD_PIN(num_pages);
  FD_PIN(div_magic); FD_PIN(div_shift); FD_PIN(nhb); FD_PIN(hpw); FD_PIN(nsub); FD_PIN(member_hb); FD_PIN(s_magic);
  FD_PIN(s_shift); FD_PIN(per_mask); FD_PIN(adapt); FD_PIN(skip_empty); FD_PIN(order_items); FD_PIN(chunk);
  // what the epilogue reads, so that it does not wait for the argument segment either
  FD_PIN(out); FD_PIN(lse); FD_PIN(so_b); FD_PIN(so_h); FD_PIN(so_s); FD_PIN(tickets); FD_PIN(mid_dtype);
  FD_PIN(vec_out); FD_PIN(store_through); FD_PIN(park); FD_PIN(no_lse); FD_PIN(out_dtype); FD_PIN(num_extra); FD_PIN(lse_column);
#undef FD_PIN
}

// Work item of a wave: grid = ((Hkv / hpw) * nhb, S, batch).  A workgroup owns hpw ADJACENT KV heads of
// one (sequence, split): wave w works on head kvh0 + w % hpw and on token sub-range w / hpw of the
// split.  Sibling waves therefore request neighbouring 128/256-byte pieces of the same token rows
// from the same CU at about the same time, which the memory system serves markedly better than the
// same pieces requested by workgroups on different XCDs (measured with a pure-read probe: 5.3 vs
// 5.85-6.1 TB/s for 128-byte rows).
//
// Issue order (workgroups are issued x-fastest and handed to the 8 XCDs, and within an XCD to its CUs, round-robin):
//  * every sequence uses all S ranges (the reference's rule): grid (x, S, batch), z = rank of the sequence -- with a
//    ranked batch the largest items are issued first and the smallest last;
//  * ranges by each sequence's own length, unscheduled: grid (x, batch, S) -- the split is the slowest dimension, so the
//    ranges every sequence has come first as one contiguous run and the empty ones last.  Next to x, the busy
//    workgroups of sequences that use only their first range would all fall on the same XCDs (measured: half the chip
//    idle, 73 instead of 43 us for 64 sequences of 1000 tokens with S = 2); rotating the split by the rank spreads the
//    XCDs but alternates busy and empty workgroups over the CUs of an XCD (57 us);
//  * scheduled (order_items): the issue order is a list of (sequence, range) items, non-empty ranges first, largest
//    first, empty ones last (fd_schedule_items_block).

// Most partials the small combine kernel takes (one dependent round trip, every slot must hold a partial).
constexpr int kCombineSmallMax = 16;

// Ranges by each sequence's own length (split_adapt): a range is not made shorter than this unless the
// sequence would otherwise get fewer ranges than the shape needs to fill the chip.
constexpr int kMinTokensPerRange = 1024;
// A batch gets enough splits that no range of a full-length sequence is longer than this (the split plan).
constexpr int kMaxTokensPerRange = 4096;

// Tokens per split range of a sequence of kv_len tokens.  Reference rule: ceil(kv_len / S) (flash_decode.py:193-195).
// With adapt > 0 (a power of two, the ranges every sequence needs so that the batch fills the chip) the ranges of a
// sequence follow its own length, not the table's capacity: per = max(ceil(kv_len / S), min(ceil(kv_len / adapt),
// want)) with want = ceil(kv_len / 8) kept within [1024, 4096] -- at least adapt ranges; beyond that 1024-token
// ranges up to 8 of them, 8 ranges up to 4096 tokens each, 4096-token ranges up to S of them, S ranges beyond.
// per_mask rounds the result up to the split alignment.  The split kernels and the combine kernel both call this, so they agree on
// which ranges are empty.
__device__ __forceinline__ int tokens_per_range(int kv_len, int S, uint32_t s_magic, uint32_t s_shift, int per_mask,
                                                int adapt) {
  // ceil(kv_len / S) by multiplication (kv_len + S - 1 < 2^31 is checked on the host)
  int per = (int)(((uint64_t)(uint32_t)(kv_len + S - 1) * s_magic) >> s_shift);
  if (adapt > 0) {
    const int floor_ranges = (kv_len + adapt - 1) >> (31 - __clz(adapt));   // ceil(kv_len / adapt)
    const int want = min(max((kv_len + 7) >> 3, kMinTokensPerRange), kMaxTokensPerRange);
    per = max(per, min(floor_ranges, want));
  }
  return (per + per_mask) & ~per_mask;
}

// x / d for x >= 0 and a wave-uniform d > 0 that is a power of two in almost every launch (waves per range, members
// per workgroup): a scalar test and a shift instead of the division sequence, which sits in front of the first table
// lookup of every wave.
__device__ __forceinline__ int div_uniform(int x, int d) {
  return (d & (d - 1)) == 0 ? x >> (31 - __clz(d)) : x / d;
}

struct WorkItem {
  int b, s, kvh, hb, start, end;
  bool skip;  // empty range and nothing to write: the workgroup may leave at once (uniform over the workgroup)
  int vh;     // 128-column half of the V rows this wave accumulates (SplitArgs::v_members == 2), else 0
  int kvh0;   // first KV head of the workgroup
  int hb0;    // first head block of the workgroup
  int sub;    // token sub-range index of this wave
  int nsub;   // token sub-ranges (waves per head)
  // chunked work items (SplitArgs::chunk > 1): this wave owns the splits s .. s + ns - 1 (ns may be 0) of per tokens
  // each, i.e. the tokens [start, end)
  int ns, per;
};

__device__ __forceinline__ WorkItem decode_work_item(const SplitArgs& a) {
  WorkItem w;
  w.vh = 0;
  // The sequence and its length first: these scalar loads head the chain length -> block table -> K/V rows that
  // every wave has to walk before it can stream.
  int b, s;
  int64_t len;
  if (a.order_items) {
    // scheduled: item k of the issue order names its sequence and range (grid (x, S, batch), y fastest)
    const int k = blockIdx.y + a.S * blockIdx.z;
    const uint32_t item = (uint32_t)a.order[k];
    len = a.order_lens[k];
    b = item & 0xffffu;
    s = item >> 16;
    w.b = min(b, a.batch - 1);
  } else {
    // ranges by each sequence's own length: grid (x, batch, S), else grid (x, S, batch)
    const bool slab_major = a.adapt > 0;
    const int r = slab_major ? blockIdx.y : blockIdx.z;
    s = slab_major ? blockIdx.z : blockIdx.y;
    b = a.order ? a.order[r] : r;
    w.b = min(max(b, 0), a.batch - 1);
    len = a.order && a.order_lens ? a.order_lens[r] : a.kv_lens[w.b];
  }
  const int wave = threadIdx.x >> 6;
  if (a.member_hb) {
    // workgroup = hpw head blocks of one KV head; blockIdx.x = kv head * (nhb / hpw) + block group
    const int groups = a.nhb / a.hpw;
    const int kvh = groups == 1 ? (int)blockIdx.x : (int)blockIdx.x / groups;
    const int hbg = blockIdx.x - kvh * groups;
    w.sub = div_uniform(wave, a.hpw);
    w.hb0 = hbg * a.hpw;
    w.hb = w.hb0 + (wave - w.sub * a.hpw);
    w.kvh0 = kvh;
    w.kvh = kvh;
    w.nsub = a.nsub;
  } else {
    int grp;
    if (a.nhb == 1) {
      grp = blockIdx.x;
      w.hb = 0;
    } else {
      grp = blockIdx.x / a.nhb;
      w.hb = blockIdx.x - grp * a.nhb;
    }
    w.hb0 = w.hb;
    if (a.hpw == 1) {
      w.kvh0 = grp;
      w.kvh = grp;
      w.sub = wave;
    } else if (a.v_members == 2) {   // members are (KV head, V half) pairs: hpw / 2 heads per workgroup
      const int member = wave - div_uniform(wave, a.hpw) * a.hpw;
      w.kvh0 = grp * (a.hpw >> 1);
      w.sub = div_uniform(wave, a.hpw);
      w.kvh = w.kvh0 + (member >> 1);
      w.vh = member & 1;
    } else {
      w.kvh0 = grp * a.hpw;
      w.sub = div_uniform(wave, a.hpw);
      w.kvh = w.kvh0 + (wave - w.sub * a.hpw);
    }
    w.nsub = a.nsub;
  }
  fd_fetch_args_now(a);   // issued behind the loads above: the rest of the arguments arrives together with them
  // ... and the length is pinned like them: left alone, the compiler sinks its load below the index arithmetic that
  // follows, to the block of its first use, and waits for it there -- one more dependent round trip in front of the
  // first table lookup
  {
    const int len_now = (int)len;
    asm volatile("" ::"s"(len_now));
  }

  int64_t cap = (int64_t)a.max_pages * a.P;
  len = len < 0 ? 0 : (len > cap ? cap : len);
  const int kv_len = (int)len;
  const int per = tokens_per_range(kv_len, a.S, a.s_magic, a.s_shift, a.per_mask, a.adapt);
  w.per = per;
  if (a.chunk > 1) {
    // s counts work items of a.chunk splits; the waves of a head share them out in runs of whole splits
    const int ns = div_uniform(a.chunk + w.nsub - 1, w.nsub);
    const int first = s * a.chunk + w.sub * ns;
    const int lim = min(min((s + 1) * a.chunk, a.S), first + ns);
    w.s = first;
    w.ns = max(lim - first, 0);
    const int64_t st = (int64_t)per * first, en = (int64_t)per * (first + w.ns);
    w.start = st > kv_len ? kv_len : (int)st;
    w.end = en > kv_len ? kv_len : (int)en;
    w.skip = false;
    return w;
  }
  w.s = min(s, a.S - 1);
  w.ns = 1;
  int64_t st = (int64_t)per * w.s;
  w.start = st > kv_len ? kv_len : (int)st;
  int64_t en = st + per;
  w.end = en > kv_len ? kv_len : (int)en;
  w.skip = a.skip_empty && w.start >= w.end;
  return w;
}

// n / P without a divide or a branch: P is only known at run time, and a branch in the
// streaming loop would make the compiler's wait counts conservative.
__device__ __forceinline__ int page_index(const SplitArgs& a, int n) {
  return (int)(((uint64_t)(uint32_t)n * a.div_magic) >> a.div_shift);
}

// Block-table entry and in-page slot of the token a lane looks up for tile t of its wave's run (TILE tokens per
// tile): token start + t * TILE + tok_lane, clamped to the last token of the range (the scores of the clamped
// tokens are masked).  The table entry is returned raw: its arithmetic is left to the consumer one iteration later,
// so that the load stays in flight across the tile that is being processed.
template <int TILE>
__device__ __forceinline__ int fd_tile_slot(const SplitArgs& a, const WorkItem& w, const int32_t* bt_row, int t,
                                            int tok_lane, int& slot) {
  int n = w.start + t * TILE + tok_lane;
  n = min(n, w.end - 1);
  const int pidx = page_index(a, n);
  slot = n - pidx * a.P;
  return bt_row[pidx];
}

// Flat cache row page * P + slot of a raw table entry, the page id clamped into the pool so that a corrupt table
// cannot fault the GPU.
__device__ __forceinline__ int fd_flat_row(const SplitArgs& a, int page, int slot) {
  return min(max(page, 0), a.num_pages - 1) * a.P + slot;
}

// Flat cache row of logical token n of sequence b: page*P + n%P, with the page id
// clamped into the pool so that a corrupt table entry cannot fault the GPU.
__device__ __forceinline__ int token_row(const SplitArgs& a, const int32_t* bt_row, int n) {
  const int pidx = page_index(a, n);
  return fd_flat_row(a, bt_row[pidx], n - pidx * a.P);
}

// Merges the per-wave partial states of a workgroup and stores one normalised partial (out, lse)
// per query head, for every KV head the workgroup owns.
//
// LDS layout of wave v's partial (floats): part[v*stride + h*D + d] = un-normalised accumulator,
// part[v*stride + HB*D + h] = running max (base-2 domain), part[v*stride + HB*D + HB + h] = running
// sum.  Wave v = member (v % hpw) + hpw * token sub-range; a member is a KV head or, for groups above 16 query
// heads, a head block of the one KV head.  Called by every thread of the workgroup after a __syncthreads() with
// nheads = the calling wave's head count.  fp8 caches: the waves have already multiplied their accumulators by
// v_scale[kv head] (a load here, between the stores, would cost its latency once per loop iteration).
//
// Two steps with a barrier between them.  First one thread per (member, head) row turns the row's running maxima
// into merge weights 2^(m_p - M) in place, leaves 1 / L in sub-range 0's sum slot and stores the row's LSE; then every
// thread sums its four (or, for rows that do not start on a multiple of four elements, its one) output values over
// the sub-ranges with those weights.  All of this runs once per workgroup after the last tile, with nothing left to
// overlap it: the per-row arithmetic is not repeated per value (a workgroup of 2 x 32 heads merged for 4.6 us when
// every thread derived its row's weights itself, 8 rounds of about 200 instructions), and every LDS read of a
// round is requested before the first one is used (unrolled over the sub-ranges).
template <int HB, int D>
__device__ __forceinline__ void cta_merge_store_rounds(const SplitArgs& a, float* part, int stride, const WorkItem& w,
                                                int nheads) {
  const int tid = threadIdx.x;
  const int nthreads = 64 * a.hpw * a.nsub;   // == blockDim.x, without a trip to the implicit kernel arguments
  constexpr int D4 = D / 4;
  // head blocks as members: the last block of a group may hold fewer heads than the others
  const int heads = a.member_hb ? HB : nheads;
  const int pstep = a.hpw * stride;   // floats between the partials of two sub-ranges of one member
  const bool through = a.store_through != 0;

  // ---- step 1: weights, 1 / L and the LSE of every row
  for (int row = tid; row < a.hpw * heads; row += nthreads) {
    int hm = 0;   // member of the row, without a division by a run-time value or a divergent loop (hpw <= 8)
#pragma unroll
    for (int k = 1; k < 8; ++k) hm += row >= k * heads;
    const int h = row - hm * heads;
    float* ml = part + hm * stride + HB * D + h;   // m_p at ml[p * pstep], l_p at ml[p * pstep + HB]
    float M = -INFINITY, L = 0.f;
    auto weigh = [&](auto nsub_tag, int ns) {
      constexpr int NS = decltype(nsub_tag)::value;   // 0: run-time count ns
      constexpr int CAP = NS ? NS : 1;
      float mm[CAP], ll[CAP];
      if constexpr (NS > 0) {
#pragma unroll
        for (int p = 0; p < NS; ++p) {
          mm[p] = ml[p * pstep];
          ll[p] = ml[p * pstep + HB];
        }
#pragma unroll
        for (int p = 0; p < NS; ++p) M = fmaxf(M, mm[p]);
#pragma unroll
        for (int p = 0; p < NS; ++p) {
          const float wgt = M > -INFINITY ? fd_exp2(mm[p] - M) : 0.f;   // exp2(-inf) = 0 for idle waves
          L += ll[p] * wgt;
          ml[p * pstep] = wgt;
        }
      } else {
        for (int p = 0; p < ns; ++p) M = fmaxf(M, ml[p * pstep]);
        for (int p = 0; p < ns; ++p) {
          const float wgt = M > -INFINITY ? fd_exp2(ml[p * pstep] - M) : 0.f;
          L += ml[p * pstep + HB] * wgt;
          ml[p * pstep] = wgt;
        }
      }
    };
    switch (w.nsub) {
      case 1: weigh(std::integral_constant<int, 1>{}, 1); break;
      case 2: weigh(std::integral_constant<int, 2>{}, 2); break;
      case 4: weigh(std::integral_constant<int, 4>{}, 4); break;
      case 8: weigh(std::integral_constant<int, 8>{}, 8); break;
      default: weigh(std::integral_constant<int, 0>{}, w.nsub);
    }
    ml[HB] = L > 0.f ? 1.0f / L : 0.f;
    const int kvh = a.member_hb ? w.kvh0 : w.kvh0 + (a.v_members == 2 ? hm >> 1 : hm);
    const int co = a.v_members == 2 ? (hm & 1) * 128 : 0;   // this member's half of the V columns
    const int hb = a.member_hb ? w.hb0 + hm : w.hb;
    if (h < a.G - hb * HB && co == 0 && (a.tickets || !a.no_lse)) {
      const float lse = L > 0.f ? (M + fd_log2(L)) * FD_LN2 : -INFINITY;
      const int head = kvh * a.G + hb * HB + h;
      const int64_t lse_at = ((int64_t)w.b * a.Hq + head) * a.S + w.s;
      const int64_t col_d = (int64_t)w.b * a.so_b + (int64_t)head * a.so_h + (int64_t)w.s * a.so_s + a.dv;
      if (a.tickets) {   // fused combine (fp32 partials only): another XCD's workgroup may read these
        store_f32_agent(a.lse ? a.lse + lse_at : (float*)a.out + col_d, lse);
      } else if (a.lse) {
        a.lse[lse_at] = lse;
      } else {
        store_partial1(a.out, col_d, a.mid_dtype, lse, through);
      }
    }
  }
  __syncthreads();

  // ---- step 2: the values.  V values per thread and round: 4 (one 128- or 64-bit store), or 1 where rows do not
  // start on a multiple of four elements (the reference's [B, Hq, S, D + 1] layout): consecutive threads on
  // consecutive elements, so that a store instruction still covers contiguous memory.
  // The loop is specialised on everything that is the same for all its rounds (values per thread, sub-range count):
  // a taken branch costs a wave an instruction-buffer refill, and with the decisions inside the loop a round was
  // some 25 of them -- about 1100 cycles per round for 80 instructions of work.
  auto values = [&](auto vec_tag, auto nsub_tag, int ns) {
    constexpr int V = decltype(vec_tag)::value;
    constexpr int NS = decltype(nsub_tag)::value;   // 0: run-time count ns
    constexpr int PER_ROW = D / V;
    using Val = typename std::conditional<V == 4, f32x4, float>::type;
    const int per_member = heads * PER_ROW;
    const bool fused = a.tickets != nullptr;
    for (int e = tid; e < a.hpw * per_member; e += nthreads) {
      // member of e without a division by a run-time value or a divergent loop (hpw <= 8)
      int hm = 0;
#pragma unroll
      for (int k = 1; k < 8; ++k) hm += e >= k * per_member;
      const int r = e - hm * per_member;
      const int h = r / PER_ROW;
      const int d = (r - h * PER_ROW) * V;
      const int kvh = a.member_hb ? w.kvh0 : w.kvh0 + (a.v_members == 2 ? hm >> 1 : hm);
      const int co = a.v_members == 2 ? (hm & 1) * 128 : 0;   // this member's half of the V columns
      const int hb = a.member_hb ? w.hb0 + hm : w.hb;
      if (h >= a.G - hb * HB || d >= a.v_cols) continue;
      const float* x0 = part + hm * stride + h * D + d;
      const float* w0 = part + hm * stride + HB * D + h;
      Val o{};
      const float inv = w0[HB];   // 1 / L
      if constexpr (NS > 0) {
        Val xx[NS];
        float ww[NS];
#pragma unroll
        for (int p = 0; p < NS; ++p) {
          xx[p] = *(const Val*)(x0 + p * pstep);
          ww[p] = w0[p * pstep];
        }
#pragma unroll
        for (int p = 0; p < NS; ++p) o += xx[p] * ww[p];
      } else {
        for (int p = 0; p < ns; ++p) o += *(const Val*)(x0 + p * pstep) * w0[p * pstep];
      }
      o *= inv;
      const int head = kvh * a.G + hb * HB + h;
      const int64_t off = (int64_t)w.b * a.so_b + (int64_t)head * a.so_h + (int64_t)w.s * a.so_s + d + co;
      if constexpr (V == 4) {
        if (fused) {
#pragma unroll
          for (int i = 0; i < 4; ++i) store_f32_agent((float*)a.out + off + i, o[i]);
        } else {
          store_partial4(a.out, off, a.mid_dtype, o, through);
        }
      } else {
        store_partial1(a.out, off, a.mid_dtype, o, through);
      }
    }
  };
  auto values_of = [&](auto vec_tag) {
    switch (w.nsub) {
      case 1: values(vec_tag, std::integral_constant<int, 1>{}, 1); break;
      case 2: values(vec_tag, std::integral_constant<int, 2>{}, 2); break;
      case 4: values(vec_tag, std::integral_constant<int, 4>{}, 4); break;
      case 8: values(vec_tag, std::integral_constant<int, 8>{}, 8); break;
      default: values(vec_tag, std::integral_constant<int, 0>{}, w.nsub);
    }
  };
  if (a.vec_out || a.tickets) {
    values_of(std::integral_constant<int, 4>{});
  } else {
    values_of(std::integral_constant<int, 1>{});
  }
}

template <int HB, int D>
__device__ __forceinline__ void cta_merge_store_one_round(const SplitArgs& a, const float* part, int stride,
                                                const WorkItem& w, int nheads) {
  const int tid = threadIdx.x;
  const int nthreads = 64 * a.hpw * a.nsub;   // == blockDim.x, without a trip to the implicit kernel arguments
  constexpr int D4 = D / 4;
  if (!a.vec_out && !a.tickets) {
    // Rows that do not start on a multiple of four elements -- the reference's [B, Hq, S, D + 1] layout, whose rows
    // are D + 1 elements apart: one element per thread, consecutive threads on consecutive elements, so that a store
    // instruction still covers contiguous memory (256 bytes of fp32 per wave).
    const int heads = a.member_hb ? HB : nheads;
    for (int e = tid; e < a.hpw * heads * D; e += nthreads) {
      const int hm = e / (heads * D);
      const int r = e - hm * heads * D;
      const int h = r / D;
      const int d = r - h * D;
      const int kvh = a.member_hb ? w.kvh0 : w.kvh0 + (a.v_members == 2 ? hm >> 1 : hm);
      const int co = a.v_members == 2 ? (hm & 1) * 128 : 0;   // this member's half of the V columns
      const int hb = a.member_hb ? w.hb0 + hm : w.hb;
      if (h >= a.G - hb * HB || d >= a.v_cols) continue;
      float M = -INFINITY;
      for (int p = 0; p < w.nsub; ++p) M = fmaxf(M, part[(hm + a.hpw * p) * stride + HB * D + h]);
      float L = 0.f, o = 0.f;
      if (M > -INFINITY) {
        for (int p = 0; p < w.nsub; ++p) {
          const float* pp = part + (hm + a.hpw * p) * stride;
          const float wgt = fd_exp2(pp[HB * D + h] - M);
          L += pp[HB * D + HB + h] * wgt;
          o += pp[h * D + d] * wgt;
        }
      }
      const float inv = L > 0.f ? 1.0f / L : 0.f;
      const int head = kvh * a.G + hb * HB + h;
      const int64_t row = (int64_t)w.b * a.so_b + (int64_t)head * a.so_h + (int64_t)w.s * a.so_s;
      store_partial1(a.out, row + d + co, a.mid_dtype, o * inv, a.store_through != 0);
      if (d == 0 && co == 0 && !a.no_lse) {
        const float lse = L > 0.f ? (M + fd_log2(L)) * FD_LN2 : -INFINITY;
        if (a.lse) {
          a.lse[((int64_t)w.b * a.Hq + head) * a.S + w.s] = lse;
        } else {
          store_partial1(a.out, row + a.dv, a.mid_dtype, lse, a.store_through != 0);
        }
      }
    }
    return;
  }
  // head blocks as members: the last block of a group may hold fewer heads than the others
  const int per_head = (a.member_hb ? HB : nheads) * D4;
  for (int e = tid; e < a.hpw * per_head; e += nthreads) {
    int hm = 0, r = e;
    while (r >= per_head) {   // at most hpw - 1 <= 3 rounds: cheaper than a division by a run-time value
      r -= per_head;
      ++hm;
    }
    const int h = r / D4;
    const int d = (r - h * D4) * 4;
    const int kvh = a.member_hb ? w.kvh0 : w.kvh0 + (a.v_members == 2 ? hm >> 1 : hm);
    const int co = a.v_members == 2 ? (hm & 1) * 128 : 0;   // this member's half of the V columns
    const int hb = a.member_hb ? w.hb0 + hm : w.hb;
    if (h >= a.G - hb * HB || d >= a.v_cols) continue;
    // This runs once per workgroup, after the last tile, with nothing left to overlap: every LDS read below is
    // requested before the first one is used (unrolled over the sub-ranges; a loop over a run-time count takes one
    // dependent LDS round trip per sub-range and value, about 1 us per launch in all).
    float M = -INFINITY, L = 0.f;
    f32x4 o = {0.f, 0.f, 0.f, 0.f};
    auto merge = [&](auto nsub_tag) {
      constexpr int NS = decltype(nsub_tag)::value;
      float mm[NS], ll[NS];
      f32x4 xx[NS];
#pragma unroll
      for (int p = 0; p < NS; ++p) {
        const float* pp = part + (hm + a.hpw * p) * stride;
        mm[p] = pp[HB * D + h];
        ll[p] = pp[HB * D + HB + h];
        xx[p] = *(const f32x4*)(pp + h * D + d);
      }
#pragma unroll
      for (int p = 0; p < NS; ++p) M = fmaxf(M, mm[p]);
      if (M > -INFINITY) {
#pragma unroll
        for (int p = 0; p < NS; ++p) {
          const float wgt = fd_exp2(mm[p] - M);  // exp2(-inf) = 0 for idle waves
          L += ll[p] * wgt;
          o += xx[p] * wgt;
        }
      }
    };
    switch (w.nsub) {
      case 1: merge(std::integral_constant<int, 1>{}); break;
      case 2: merge(std::integral_constant<int, 2>{}); break;
      case 4: merge(std::integral_constant<int, 4>{}); break;
      case 8: merge(std::integral_constant<int, 8>{}); break;
      default:
        for (int p = 0; p < w.nsub; ++p) M = fmaxf(M, part[(hm + a.hpw * p) * stride + HB * D + h]);
        if (M > -INFINITY) {
          for (int p = 0; p < w.nsub; ++p) {
            const float* pp = part + (hm + a.hpw * p) * stride;
            const float wgt = fd_exp2(pp[HB * D + h] - M);
            L += pp[HB * D + HB + h] * wgt;
            o += *(const f32x4*)(pp + h * D + d) * wgt;
          }
        }
    }
    float inv = L > 0.f ? 1.0f / L : 0.f;
    o *= inv;
    const int head = kvh * a.G + hb * HB + h;
    const int64_t row = (int64_t)w.b * a.so_b + (int64_t)head * a.so_h + (int64_t)w.s * a.so_s;
    const int64_t off = row + d + co;
    const float lse = L > 0.f ? (M + fd_log2(L)) * FD_LN2 : -INFINITY;
    if (a.tickets) {
      // fused combine (fp32 partials only): another XCD's workgroup may read these
#pragma unroll
      for (int i = 0; i < 4; ++i) store_f32_agent((float*)a.out + off + i, o[i]);
      if (d == 0 && co == 0)
        store_f32_agent(a.lse ? a.lse + ((int64_t)w.b * a.Hq + head) * a.S + w.s : (float*)a.out + row + a.dv, lse);
    } else {
      if (a.vec_out) {
        store_partial4(a.out, off, a.mid_dtype, o, a.store_through != 0);
      } else {
        for (int i = 0; i < 4; ++i) store_from_f32(a.out, off + i, a.mid_dtype, o[i]);
      }
      if (d == 0 && co == 0 && !a.no_lse) {
        if (a.lse) {
          a.lse[((int64_t)w.b * a.Hq + head) * a.S + w.s] = lse;
        } else {
          store_from_f32(a.out, row + a.dv, a.mid_dtype, lse);
        }
      }
    }
  }
}

// Few rows (at most two rounds of four values per thread): every thread derives its row's weights itself, no second
// barrier (config 2, 2 x 4 heads: 44.5 us per step against 44.9 us with the two steps below).  More rows: two steps.
template <int HB, int D>
__device__ __forceinline__ void cta_merge_store(const SplitArgs& a, float* part, int stride, const WorkItem& w,
                                                int nheads) {
  const int heads = a.member_hb ? HB : nheads;
  const bool by_element = !a.vec_out && !a.tickets;   // one value per thread and round: four times the rounds
  if (a.hpw * heads * (D / 4) <= 2 * 64 * a.hpw * a.nsub && !by_element) {
    cta_merge_store_one_round<HB, D>(a, part, stride, w, nheads);
  } else {
    cta_merge_store_rounds<HB, D>(a, part, stride, w, nheads);
  }
}

// Eight consecutive values of a finished partial row into a parked slot's rows (SplitArgs::park_final): two 128-bit
// LDS writes for fp32, one of eight packed values for fp16 / bf16.  elem = element offset of the first value.
__device__ __forceinline__ void park_store8(char* rows, int elem, int dtype, const float (&v)[8]) {
  if (dtype == FD_F32) {
    float* p = (float*)rows + elem;
    *(f32x4*)p = f32x4{v[0], v[1], v[2], v[3]};
    *(f32x4*)(p + 4) = f32x4{v[4], v[5], v[6], v[7]};
  } else {
    u32x4 w;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const f32x2 x = {v[2 * e], v[2 * e + 1]};
      w[e] = dtype == FD_F16 ? __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2))
                             : __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
    }
    *(u32x4*)((uint16_t*)rows + elem) = w;
  }
}

// Raw-bit stores of one dword / one 16-bit value, optionally written through (same restriction as store_partial4).
__device__ __forceinline__ void store_bits32(void* p, uint32_t w, bool through) {
  if (through) {
    asm volatile("global_store_dword %0, %1, off sc0 sc1" ::"v"(p), "v"(w) : "memory");
  } else {
    *(uint32_t*)p = w;
  }
}
__device__ __forceinline__ void store_bits16(void* p, uint32_t w, bool through) {
  if (through) {
    asm volatile("global_store_short %0, %1, off sc0 sc1" ::"v"(p), "v"(w) : "memory");
  } else {
    *(uint16_t*)p = (uint16_t)w;
  }
}
__device__ __forceinline__ uint32_t f32_to_bits16(float x, int dtype) {
  return dtype == FD_F16 ? (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x)
                         : (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)x);
}

// Chunked work items: ONE wave copies a finished partial that it parked in LDS (HB fp32 LSEs, then the normalised
// rows [head][D] of its real heads in mid_dtype) to split s of its head slots.  Called at the end of the wave's run
// only: on this target stores and loads of a wave retire in order (one vmcnt), so a store issued between two tiles
// would hold back every later K/V load until it is acknowledged.  empty: the split holds no token (out = 0,
// lse = -inf; the slot is not read).  Every form moves 128 bits per lane with whole rows per store instruction, and
// the values are the parked bits: nothing is scaled or converted here but the LSE.
//  * fp32 rows, and 16-bit rows that start on multiples of four elements (the library's own layout): straight copies.
//    fp32 rows of the reference's [B, Hq, S, D + 1] layout start on 4-byte boundaries only, which is all a 128-bit
//    store needs.
//  * 16-bit rows of that layout (D values with the LSE behind them, D + 1 elements apart, so every other row starts
//    between two 4-byte boundaries): a row that starts on a boundary goes out as it is parked and its LSE alone; one
//    that starts between two stores value 0 alone and then the 128-bit pieces (1 .. 8), (9 .. 16), .. (D - 7 .. D - 1,
//    LSE), each put together from five parked dwords with a funnel shift.  The LDS reads of all rows are independent
//    of each other, so the wave pays one LDS round trip, not one per row.
template <int HB, int D>
__device__ __forceinline__ void wave_copy_parked(const SplitArgs& a, const char* slot, int b, int head0, int nheads,
                                                 int s, bool empty) {
  const int lane = threadIdx.x & 63;
  constexpr int D4 = D / 4;
  constexpr int RPI = 64 / D4;
  static_assert(D4 <= 64 && HB % RPI == 0 && D % 64 == 0, "one wave covers whole rows");
  const float* lse_slot = (const float*)slot;
  const char* rows = slot + HB * 4;
  const bool through = a.store_through != 0;
  constexpr int LPR = D / 8;      // 16-bit rows: lanes per row, eight values each
  constexpr int RPS = 64 / LPR;   // ... and rows per store instruction
  static_assert(HB % RPS == 0, "one wave covers whole rows");
  if (a.mid_dtype == FD_F32) {
    const int d = (lane % D4) * 4;
#pragma unroll
    for (int r = 0; r < HB / RPI; ++r) {
      const int h = r * RPI + lane / D4;
      if (h >= nheads) continue;
      const int head = head0 + h;
      const int64_t off = (int64_t)b * a.so_b + (int64_t)head * a.so_h + (int64_t)s * a.so_s + d;
      const f32x4 v = empty ? f32x4{0.f, 0.f, 0.f, 0.f} : *(const f32x4*)((const float*)rows + h * D + d);
      float* p = (float*)a.out + off;
      if (through) {
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
      } else {
        *(f32x4_a4*)p = v;
      }
      if (d == 0 && !a.no_lse) {
        const float lse = empty ? -INFINITY : lse_slot[h];
        if (a.lse) {
          a.lse[((int64_t)b * a.Hq + head) * a.S + s] = lse;
        } else {
          store_partial1(a.out, off + D, a.mid_dtype, lse, through);
        }
      }
    }
    return;
  }
  if (a.vec_out) {
    const int d = (lane % LPR) * 8;
#pragma unroll
    for (int r = 0; r < HB / RPS; ++r) {
      const int h = r * RPS + lane / LPR;
      if (h >= nheads) continue;
      const int head = head0 + h;
      const int64_t off = (int64_t)b * a.so_b + (int64_t)head * a.so_h + (int64_t)s * a.so_s + d;
      const u32x4 v = empty ? u32x4{0u, 0u, 0u, 0u} : *(const u32x4*)((const uint16_t*)rows + h * D + d);
      uint16_t* p = (uint16_t*)a.out + off;
      if (through) {
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
      } else {
        *(u32x4_a4*)p = v;
      }
      if (d == 0 && !a.no_lse) {
        const float lse = empty ? -INFINITY : lse_slot[h];
        if (a.lse) {
          a.lse[((int64_t)b * a.Hq + head) * a.S + s] = lse;
        } else {
          store_partial1(a.out, off + D, a.mid_dtype, lse, through);
        }
      }
    }
    return;
  }
  const int64_t row0 = (int64_t)b * a.so_b + (int64_t)head0 * a.so_h + (int64_t)s * a.so_s;
  uint16_t* out = (uint16_t*)a.out;
  const uint16_t* r16 = (const uint16_t*)rows;
  const uint32_t* r32 = (const uint32_t*)rows;
  // lane h serves row h's single values: its LSE (and, for a row that starts between two boundaries, value 0)
  const int hl = lane < nheads ? lane : nheads - 1;
  const float lse_l = empty ? -INFINITY : lse_slot[hl];
  const bool paired = !a.lse && !a.no_lse;
  if (!paired) {
    // 16-bit rows without an LSE behind them: element by element
    constexpr int NV = D / 64;
    for (int h = 0; h < nheads; ++h) {
      uint16_t* row = out + row0 + (int64_t)h * a.so_h;
#pragma unroll
      for (int k = 0; k < NV; ++k) store_bits16(row + lane + 64 * k, empty ? 0u : r16[h * D + lane + 64 * k], through);
    }
    if (lane < nheads && !a.no_lse) a.lse[((int64_t)b * a.Hq + head0 + hl) * a.S + s] = lse_l;
    return;
  }
  // element parity of a row's start relative to a 4-byte boundary
  const uint64_t par0 = (reinterpret_cast<uintptr_t>(a.out) >> 1) + (uint64_t)row0;
  if (lane < nheads) {
    const bool first_l = ((par0 + (uint64_t)hl * (uint64_t)a.so_h) & 1) != 0;
    uint16_t* row = out + row0 + (int64_t)hl * a.so_h;
    store_bits16(row + (first_l ? 0 : D), first_l ? (empty ? 0u : (uint32_t)r16[hl * D]) : f32_to_bits16(lse_l, a.mid_dtype),
                 through);
  }
  const int j = lane % LPR;
#pragma unroll
  for (int r = 0; r < HB / RPS; ++r) {
    const int h = r * RPS + lane / LPR;
    if (h >= nheads) continue;
    const uint32_t first = (uint32_t)((par0 + (uint64_t)h * (uint64_t)a.so_h) & 1);
    u32x4 w = {0u, 0u, 0u, 0u};
    uint32_t next = 0u;
    if (!empty) {
      w = *(const u32x4*)(r32 + h * (D / 2) + 4 * j);
      next = r32[h * (D / 2) + min(4 * j + 4, D / 2 - 1)];
    }
    if (j == LPR - 1) next = f32_to_bits16(empty ? -INFINITY : lse_slot[h], a.mid_dtype);
    if (first) {
      w = u32x4{__builtin_amdgcn_alignbit(w[1], w[0], 16), __builtin_amdgcn_alignbit(w[2], w[1], 16),
                __builtin_amdgcn_alignbit(w[3], w[2], 16), __builtin_amdgcn_alignbit(next, w[3], 16)};
    }
    uint16_t* p = out + row0 + (int64_t)h * a.so_h + 8 * j + first;
    if (through) {
      asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(w) : "memory");
    } else {
      *(u32x4_a4*)p = w;
    }
  }
}

// Fused combine: called by every thread of the workgroup after cta_merge_store() (which, in this
// mode, wrote the fp32 partials with agent-scope stores).  Every wave waits for its stores to
// be acknowledged (an explicit vmcnt(0) wait), one thread takes a ticket for the (sequence, KV head, head block) group, and the
// workgroup that draws the last ticket merges the group's S partials (and the extra ones) into the
// final output with the stand-alone combine kernel's weights softmax(LSE)_s.  No workgroup ever
// waits for another one.  s_lse: LDS scratch of at least (S + num_extra) * nheads floats.
template <int D>
__device__ __forceinline__ void fused_combine(const SplitArgs& a, const WorkItem& w, int head0, int nheads,
                                              float* s_lse) {
  __shared__ int s_last;
  const int tid = threadIdx.x;
  const int nth = 64 * a.hpw * a.nsub;
  // Every wave waits here until all its partial stores have been acknowledged: they are agent-scope write-through
  // stores, so an acknowledged store has left this XCD's L2 and is what an agent-scope load from any XCD returns.  A
  // workgroup-scope release fence would not do: outside threadgroup-split mode it orders LDS traffic only (waves of a
  // workgroup share their CU's vector cache) and leaves vector-memory stores in flight.  The barrier then collects
  // "all stores of all waves acknowledged", and only after it does thread 0 take the ticket, itself an agent-scope
  // read-modify-write performed at the same memory-side point the stores went to.  The workgroup that draws the last
  // ticket therefore takes it after every other workgroup's partials have landed, and its agent-scope loads (which
  // do not hit in its own L2) are issued after the ticket has returned (s_last goes through LDS and a barrier).
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (tid == 0) {
    int32_t* t = a.tickets + ((int64_t)w.b * a.Hkv + w.kvh) * a.nhb + w.hb;
    const int old = __hip_atomic_fetch_add(t, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int last = old == a.S - 1;
    // every split of the group has arrived: leave the counter clean for the next launch
    if (last) __hip_atomic_store(t, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = last;
  }
  __syncthreads();
  if (!s_last) return;

  const int S = a.S;
  const int NP = S + a.num_extra;
  const float* mid = (const float*)a.out;
  for (int i = tid; i < NP * nheads; i += nth) {
    const int h = i / NP;
    const int s = i - h * NP;
    const int head = head0 + h;
    float L;
    if (s < S) {
      L = load_f32_agent(a.lse ? a.lse + ((int64_t)w.b * a.Hq + head) * S + s
                               : mid + (int64_t)w.b * a.so_b + (int64_t)head * a.so_h + (int64_t)s * a.so_s + D);
    } else {
      L = a.extra_lse[((int64_t)(s - S) * a.batch + w.b) * a.Hq + head];
    }
    s_lse[i] = L;
  }
  __syncthreads();
  constexpr int D4 = D / 4;
  for (int e = tid; e < nheads * D4; e += nth) {
    const int h = e / D4;
    const int d = (e - h * D4) * 4;
    const int head = head0 + h;
    const float* ls = s_lse + h * NP;
    float M = -INFINITY;
    for (int s = 0; s < NP; ++s) M = fmaxf(M, ls[s]);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float L = 0.f;
    if (M > -INFINITY) {
      const float* base = mid + (int64_t)w.b * a.so_b + (int64_t)head * a.so_h + d;
      // every split slot was written by its workgroup (empty ones hold zeros), so the rows are
      // loaded unconditionally and several loads stay in flight
      if (a.vec_out) {
#pragma unroll 8
        for (int s = 0; s < S; ++s) {
          const float wgt = __expf(ls[s] - M);
          const f32x2 lo = load_f32x2_agent(base + (int64_t)s * a.so_s);
          const f32x2 hi = load_f32x2_agent(base + (int64_t)s * a.so_s + 2);
          acc += f32x4{lo[0], lo[1], hi[0], hi[1]} * wgt;
          L += wgt;
        }
      } else {
#pragma unroll 4
        for (int s = 0; s < S; ++s) {
          const float wgt = __expf(ls[s] - M);
#pragma unroll
          for (int k = 0; k < 4; ++k) acc[k] += wgt * load_f32_agent(base + (int64_t)s * a.so_s + k);
          L += wgt;
        }
      }
      for (int x = 0; x < a.num_extra; ++x) {
        const float wgt = __expf(ls[S + x] - M);
        const int64_t off = (((int64_t)x * a.batch + w.b) * a.Hq + head) * D + d;
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[k] += wgt * load_as_f32(a.extra_out, off + k, a.out_dtype);
        L += wgt;
      }
    }
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    const int64_t ob = (int64_t)w.b * a.sfo_b + (int64_t)head * a.sfo_h;
#pragma unroll
    for (int k = 0; k < 4; ++k) store_from_f32(a.fout, ob + d + k, a.out_dtype, acc[k] * inv);
    if (d == 0) {
      const float lse = L > 0.f ? M + __logf(L) : -INFINITY;
      if (a.lse_column) store_from_f32(a.fout, ob + D, a.out_dtype, lse);
      if (a.flse) a.flse[(int64_t)w.b * a.Hq + head] = lse;
    }
  }
}

// Rank of a sequence = the number of sequences in front of it when they are sorted by length descending, ties by
// index.  T = 1 << t_shift lanes of a wave share a sequence (T is the same for the whole ranking grid, whose thread
// `gid` serves sequence gid >> t_shift): the lengths go through LDS in chunks, lane `part` of a sequence compares it with
// the groups of four lengths part, part + T, ... of every chunk (lanes of one sequence read consecutive 16-byte groups,
// lanes of different sequences the same ones), and the partial ranks are summed over the T lanes with shuffles.  With
// one thread per sequence walking all the others 1024 sequences took 51 us -- one wave per SIMD on four CUs, every
// compare a dependent step.  Every thread of the workgroup calls this (it contains barriers); the result is valid in
// all T lanes of sequences < batch.  s_len: LDS, kRankChunk entries, 16-byte aligned.  len_of(j): length of sequence j.
constexpr int kRankChunk = 2048;

template <typename LenFn>
__device__ __forceinline__ int fd_rank_sequence(int gid, int batch, int t_shift, LenFn len_of, int32_t* s_len,
                                                int* mine_out) {
  const int T = 1 << t_shift;
  const int i = gid >> t_shift;
  const int part = gid & (T - 1);
  const int mine = i < batch ? len_of(i) : 0;
  int rank = 0;
  for (int j0 = 0; j0 < batch; j0 += kRankChunk) {
    const int cnt = min(kRankChunk, batch - j0);
    const int groups = (cnt + 3) >> 2;
    __syncthreads();
    // padding entries (INT32_MIN at indices >= batch) never rank before a real sequence
    for (int j = threadIdx.x; j < 4 * groups; j += blockDim.x) s_len[j] = j < cnt ? len_of(j0 + j) : INT32_MIN;
    __syncthreads();
    for (int g = part; g < groups; g += T) {
      const i32x4 other = *(const i32x4*)&s_len[4 * g];
#pragma unroll
      for (int e = 0; e < 4; ++e) rank += (other[e] > mine) || (other[e] == mine && j0 + 4 * g + e < i);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const int up = __shfl_xor(rank, off);
    if (off < T) rank += up;
  }
  *mine_out = mine;
  return rank;
}

// Lanes per sequence for fd_rank_sequence: as many as keep the ranking grid at 512 workgroups of 256 threads or fewer
// (64 up to 2048 sequences, 2 at 65535).
inline int fd_rank_shift(int64_t batch) {
  int t_shift = 6;
  while (t_shift > 0 && (batch << t_shift) > 131072) --t_shift;
  return t_shift;
}

// Sequences one scheduling workgroup ranks (its LDS holds 12 bytes per sequence).
constexpr int kMaxItemBatch = 1024;

// Work-item order for the split kernels, computed by ONE workgroup (batch <= kMaxItemBatch, blockDim.x >= batch
// rounded up to a power of two, at least 64).  items[k], k < batch * S, = sequence | range << 16: first the non-empty
// ranges, sequence by sequence in descending order of length, ties by index -- the tokens per range never decrease
// with the length and all ranges of a sequence have the same size, so this is largest-item-first -- then the empty
// ranges.  items[batch * S + k] = the length of item k's sequence.  len_of(j) = length of sequence j as the decode
// will see it.  Up to 64 sequences are ranked by one wave with shuffles (every lane against every other); larger
// batches by a bitonic sort and a prefix sum in LDS, O(log^2 batch) steps (all pairs took 58 us for 1024 sequences,
// one workgroup being one CU).  The list is written with consecutive threads on consecutive entries.
// s_key / s_n: LDS, blockDim.x entries each.
template <typename LenFn>
__device__ __forceinline__ void fd_schedule_items_block(int tid, int batch, LenFn len_of, const RangePlan& rp,
                                                        int32_t* items, uint64_t* s_key, int32_t* s_n) {
  int np2 = 64;
  while (np2 < batch) np2 <<= 1;
  // n = non-empty ranges of a sequence of len tokens = ceil(len / per) <= S, without an integer division
  auto ranges_of = [&](int len) {
    if (len <= 0) return 0;
    const int per = tokens_per_range(len, rp.S, rp.s_magic, rp.s_shift, rp.per_mask, rp.adapt);
    int n = (int)((float)len / (float)per);
    while ((int64_t)n * per < len) ++n;
    while (n > 0 && (int64_t)(n - 1) * per >= len) --n;
    return n;
  };
  // key = length in the high word, ~index in the low word: descending keys = longest first, ties by index;
  // padding entries (0) sort behind every real one
  const uint64_t key = tid < batch ? ((uint64_t)(uint32_t)len_of(tid) << 32) | (0xffffffffu - (uint32_t)tid) : 0;
  if (np2 == 64) {
    if (tid < 64) {
      const int n = key ? ranges_of((int)(key >> 32)) : 0;
      int rank = 0, first = 0;
      for (int j = 0; j < 64; ++j) {
        const uint64_t other = ((uint64_t)(uint32_t)__shfl((int)(key >> 32), j) << 32) | (uint32_t)__shfl((int)(uint32_t)key, j);
        const int n_j = __shfl(n, j);
        const bool before = other > key;   // keys are distinct
        rank += before ? 1 : 0;
        first += before ? n_j : 0;
      }
      if (key) {
        s_key[rank] = key;        // rank = position in the sorted order
        s_n[rank] = first + n;    // inclusive prefix sum of the non-empty ranges
      }
    }
    __syncthreads();
  } else {
    if (tid < np2) s_key[tid] = key;
    __syncthreads();
    for (int k = 2; k <= np2; k <<= 1) {
      for (int j = k >> 1; j > 0; j >>= 1) {
        const int partner = tid ^ j;
        if (tid < np2 && partner > tid) {
          const uint64_t x = s_key[tid], y = s_key[partner];
          const bool descending = (tid & k) == 0;
          if (descending ? x < y : x > y) {
            s_key[tid] = y;
            s_key[partner] = x;
          }
        }
        __syncthreads();
      }
    }
    if (tid < np2) {
      const uint64_t mine = s_key[tid];
      s_n[tid] = mine ? ranges_of((int)(mine >> 32)) : 0;
    }
    __syncthreads();
    for (int off = 1; off < np2; off <<= 1) {   // inclusive prefix sum over the ranks
      const int add = tid < np2 && tid >= off ? s_n[tid - off] : 0;
      __syncthreads();
      if (tid < np2) s_n[tid] += add;
      __syncthreads();
    }
  }
  const int total = batch * rp.S;
  const int busy = s_n[batch - 1];   // non-empty ranges of the whole batch
  for (int e = tid; e < total; e += blockDim.x) {
    const int r = (int)(((uint64_t)(uint32_t)e * rp.s_magic) >> rp.s_shift);   // rank, e / S
    const int t = e - r * rp.S;                                                 // range of that sequence
    const uint64_t mine = s_key[r];
    const int incl = s_n[r];
    const int first = r ? s_n[r - 1] : 0;      // non-empty ranges of the sequences before this one
    const int n = incl - first;
    // the empty ranges of the sequences before this one come first among the empty ones
    const int k = t < n ? first + t : busy + (r * rp.S - first) + (t - n);
    items[k] = (int32_t)((0xffffffffu - (uint32_t)mine) | ((uint32_t)t << 16));
    items[total + k] = (int)(mine >> 32);
  }
}

// Launch grid of the split kernels (see decode_work_item).
inline dim3 fd_split_grid(const SplitArgs& a) {
  if (a.adapt > 0 && !a.order_items) return dim3((unsigned)a.grid_x, (unsigned)a.batch, (unsigned)a.S);
  const int items = a.chunk > 1 ? (a.S + a.chunk - 1) / a.chunk : a.S;   // work items per sequence
  return dim3((unsigned)a.grid_x, (unsigned)items, (unsigned)a.batch);
}

// Launchers implemented in the kernel translation units (host side).
int fd_launch_split_mfma(hipStream_t stream, const SplitArgs& a, int kv_dtype, int waves, bool soft_cap);
int fd_launch_split_mfma_d64(hipStream_t stream, const SplitArgs& a, int kv_dtype, int waves, bool soft_cap);
int fd_launch_split_mfma_d256(hipStream_t stream, const SplitArgs& a, int kv_dtype, int waves, bool soft_cap);
int fd_launch_split_mfma_fp8_d256(hipStream_t stream, const SplitArgs& a, int q_dtype, int waves, bool soft_cap);
int fd_launch_split_mfma_fp8(hipStream_t stream, const SplitArgs& a, int q_dtype, int waves, bool soft_cap);
int fd_launch_split_mfma_fp8_d64(hipStream_t stream, const SplitArgs& a, int q_dtype, int waves, bool soft_cap,
                                 int kv_heads_per_wave);
int fd_launch_split_valu(hipStream_t stream, const SplitArgs& a, int kv_dtype, int head_dim, int v_head_dim, int waves);
int fd_launch_combine(hipStream_t stream, const CombineArgs& a);
int fd_launch_schedule(hipStream_t stream, const int32_t* kv_lens, int batch, int32_t* order);
int fd_launch_schedule_items(hipStream_t stream, const int32_t* kv_lens, int batch, int64_t capacity,
                             const RangePlan& ranges, int32_t* items);
int fd_launch_kv_append(hipStream_t stream, const AppendArgs& a, int src_dtype, int kv_dtype);
