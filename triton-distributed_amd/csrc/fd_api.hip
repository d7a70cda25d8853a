// extern "C" entry points of libflash_decode_gfx950.so: argument validation,
// kernel selection and launch.  Declarations and the reference interfaces they
// replace are in include/flash_decode.h.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "fd_common.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int dtype_size(int dt) {
  switch (dt) {
    case FD_F32: return 4;
    case FD_F16:
    case FD_BF16: return 2;
    case FD_FP8_E4M3: return 1;
    default: return 0;
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Head dim of the V cache, of the partials and of the output.
int v_dim(const fd_params* p) { return p->v_head_dim > 0 ? p->v_head_dim : p->head_dim; }

// Magic number for n / d, exact for 0 <= n < 2^31: with l = ceil(log2 d) and k = 31 + l,
// M = floor(2^k / d) + 1 fits in 32 bits and floor(n * M / 2^k) == floor(n / d).
void div_magic(uint32_t d, uint32_t* magic, uint32_t* shift) {
  uint32_t l = 0;
  while (((uint64_t)1 << l) < d) ++l;
  const uint32_t k = 31 + l;
  *magic = (uint32_t)((((uint64_t)1 << k) / d) + 1);
  *shift = k;
}

// Shapes the MFMA split kernels are built for: head_dim 64, 128 or 256 with a 16-bit or fp8-e4m3 cache; any GQA
// group (blocks of 16 query heads, the last one padded: even with one query head per KV head the MFMA kernels stream
// faster than the VALU kernel, 46.1 vs 50.2 us on config 2's shape as MHA, 46.1 vs 78.9 us with 3 query heads per
// KV head).
bool mfma_shape_ok(int head_dim, int kv_dtype) {
  const bool kv16 = kv_dtype == FD_F16 || kv_dtype == FD_BF16;
  return (head_dim == 64 || head_dim == 128 || head_dim == 256) && (kv16 || kv_dtype == FD_FP8_E4M3);
}

// Tuning overrides for experiments, read once per process: FD_WAVES_PER_BLOCK (1, 2, 4 or 8 waves per (KV head,
// split) where the caller leaves the choice to the library), FD_HEADS_PER_BLOCK (members per workgroup),
// FD_HEAD_BLOCK (16 or 32 query heads per wave in the head_dim-128 kernels) and FD_NO_CHUNK.
int env_int(const char* name) {
  const char* e = getenv(name);
  return e ? atoi(e) : 0;
}

// Query-head slots of one head block of the MFMA kernels: 16 (one MFMA column block per wave), or 32 where the kernel
// serves two column blocks per wave from one pass over K and V and the group is large enough to use them.
int mfma_head_block(int head_dim, int group, int kv_dtype) {
  if (head_dim != 128) return 16;
  static const int forced = env_int("FD_HEAD_BLOCK");   // tuning override for experiments: 16 or 32
  if (forced == 16 || forced == 32) return forced;
  if (kv_dtype == FD_F16 || kv_dtype == FD_BF16) return group > 16 ? 32 : 16;
  // fp8: two sibling waves of 16 heads each still beat one two-block wave (G = 32: 47.3 vs 52.1 us on config 2's
  // shape); beyond that two two-block waves beat four sibling waves (G = 64: 62.5 vs 77.0 us)
  if (kv_dtype == FD_FP8_E4M3) return group > 32 ? 32 : 16;
  return 16;
}

// Whether the fp8 head_dim-64 kernel can serve two adjacent KV heads per wave (given contiguous rows).
bool fp8_d64_pairs(int group, int kv_heads) { return group <= 16 && kv_heads % 2 == 0; }

// fd_params.split_adapt: 0, or a power of two together with a split alignment and a power-of-two split count.
int check_split_adapt(const char* fn, const fd_params* p) {
  const int k = p->split_adapt;
  if (k == 0) return FD_OK;
  if (k < 0 || (k & (k - 1)) || p->split_align <= 0)
    return fail(FD_ERR_INVALID_ARG, "%s: split_adapt %d needs a power of two and split_align > 0", fn, k);
  return FD_OK;
}

// Longest sequence the launch shape is planned for: the block table's capacity, or the caller's smaller hint.
// A sequence that is longer all the same is still decoded in full (its ranges just get longer than planned).
int64_t planned_tokens(const fd_params* p) {
  const int64_t cap = (int64_t)p->max_pages_per_seq * p->page_size;
  return p->max_kv_len > 0 && p->max_kv_len < cap ? p->max_kv_len : cap;
}

// Launch-shape policy, from sweeps on one MI355X (256 CUs): the MFMA kernels stream best with about
// 1024 waves in flight (16 KB of loads each), the VALU kernel with about 2048 (8 KB each), each walking
// a long token range (every wave pays a fixed prologue / epilogue, and every split adds a partial for
// the combine), and with at least one workgroup per CU.
constexpr int64_t kTargetWaves = 1024;
constexpr int64_t kTargetWavesValu = 2048;
constexpr int64_t kMinWorkgroups = 256;
constexpr int64_t kMaxTokensPerSplit = kMaxTokensPerRange;   // keeps a ragged batch balanceable by the dispatcher
constexpr int64_t kMaxBalanceSplits = 32;                    // ... with at most this many splits for that purpose
constexpr int kPlanMinTokensPerSplit = 0;                    // fewest tokens a planned split of a full-length sequence holds
constexpr int64_t kStoreThroughBytes = 16 << 20;   // partials of a step from which on they are written through
constexpr int kMaxChunkBatch = 32;     // chunked work items: largest batch they are used for
constexpr int kMaxSplitsPerWave = 4;   // chunked work items: splits one wave walks (finished partials parked in LDS)
constexpr int kChunkLdsBytes = 80 * 1024;   // LDS a chunked workgroup may take: two of them per CU

int env_waves() {
  static const int v = env_int("FD_WAVES_PER_BLOCK");
  return v;
}
int env_heads() {
  static const int v = env_int("FD_HEADS_PER_BLOCK");
  return v;
}
// FD_NO_CHUNK=1 (experiments): one workgroup per split even where a workgroup could walk several.
// LDS of one wave's staging buffer in the head_dim-128 MFMA kernels (the larger of the 16-bit and the fp8 kernel's)
int hb_slots_lds(int hbsz) { return hbsz > 16 ? (32 * 128 + 2 * 32) * 4 : 64 * 144; }

bool env_no_chunk() {
  static const int v = env_int("FD_NO_CHUNK");
  return v != 0;
}

// Waves per (KV head, split) when the caller does not choose: the smallest power of two that reaches
// kTargetWaves, never more waves than tiles a split can have.
int choose_waves(int64_t head_splits, int64_t max_tokens_per_split, int tile, int64_t target, int max_waves) {
  int64_t tiles = (max_tokens_per_split + tile - 1) / tile;
  int w = 1;
  // (a grid a few workgroups short of one per CU -- 252 -- counts as reaching the target)
  while (w < max_waves && head_splits * w * 16 < target * 15 && w * 2 <= tiles) w *= 2;
  const int e = env_waves();
  if (e == 1 || e == 2 || e == 4 || e == 8) w = e;
  return w < max_waves ? w : max_waves;
}

// Adjacent KV heads per workgroup (one wave each): sibling waves fetch up to 512 contiguous bytes of
// every token row together.  Bounded by the waves a workgroup may have and by keeping one workgroup per CU.
int choose_heads_per_group(int kv_heads, int row_bytes, int waves, int64_t head_splits, int max_waves) {
  int h = row_bytes > 0 ? 512 / row_bytes : 1;
  if (env_heads() > 0) h = env_heads();
  if (h < 1) h = 1;
  // (a grid that misses one workgroup per CU by a few -- 12 KV heads x 42 splits / 2 = 252 -- still counts as full)
  while (h > 1 && (kv_heads % h != 0 || h * waves > max_waves || head_splits / h < kMinWorkgroups * 15 / 16)) h >>= 1;
  // Between one and one and a half workgroups per CU the busiest CUs hold two workgroups of h members; with half the
  // members they hold three of h / 2 (measured 3 - 7 % faster there: B = 5 x 5000 tokens 22.4 -> 20.8 us)
  const int64_t nwg = head_splits / h;
  if (h > 1 && nwg > kMinWorkgroups && 2 * nwg <= 3 * kMinWorkgroups) h >>= 1;
  return h;
}

}  // namespace

// Partial workspace of fd_decode_noalloc: a file-scope device array, so that the entry point never allocates.
// Every GPU the library runs on holds its own copy (FD_NOALLOC_SCRATCH_BYTES of device memory until the process
// ends) at its own address.  In host code the array's name is only a handle for the runtime, not a device
// address: the address is looked up once per device with hipGetSymbolAddress and only that pointer is handed
// to kernels.
static __device__ __align__(256) unsigned char scratch[FD_NOALLOC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];   // per device, written once (every thread that races here writes the same value)

// Device address of `scratch` on the current device, or nullptr with the error message set.
void* scratch_on_current_device(const char* fn) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fail(FD_ERR_LAUNCH, "%s: hipGetDevice: %s (device %d)", fn, hipGetErrorString(e), dev);
    return nullptr;
  }
  void* ptr = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (ptr) return ptr;
  e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !ptr) {
    fail(FD_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch): %s", fn, hipGetErrorString(e));
    return nullptr;
  }
  __atomic_store_n(&g_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
  return ptr;
}

}  // namespace

extern "C" {
const char* fd_last_error(void) { return g_err; }
int fd_abi_version(void) { return FD_ABI_VERSION; }
#ifndef FD_BUILD_ID
#define FD_BUILD_ID "unknown"
#endif
// kept with its tag so that the id can also be read from the file without loading it
static const char g_build_id[] = "FD_BUILD_ID=" FD_BUILD_ID;
const char* fd_build_id(void) { return g_build_id + sizeof("FD_BUILD_ID=") - 1; }
}

namespace {

struct FusedTail {          // what the fused combine needs on top of the split arguments
  int32_t* tickets = nullptr;
  void* out = nullptr;
  float* lse_out = nullptr;
  const void* extra_out = nullptr;
  const float* extra_lse = nullptr;
  int64_t stride_obs = 0, stride_oh = 0;
  int32_t num_extra = 0, lse_column = 0;
};

// Largest dynamic LDS a workgroup may ask for on gfx950 (160 KB per CU).
constexpr size_t kMaxLds = 160 * 1024;

// What a launch of the split kernel looks like (fd_launch_plan reports it).
struct LaunchShape {
  int mfma, tile, waves_per_head, members, chunk, head_block, store_through;
  unsigned grid[3];
};

// shape_only: the launch shape is reported there and nothing is launched (the pointers are only checked, never
// dereferenced on the host, so a planner may pass stand-ins).
int split_impl(const char* fn, void* stream, const void* q, const void* k_cache, const void* v_cache,
               void* out_split, float* lse_split, float sm_scale, const int32_t* block_table,
               const int32_t* kv_lens, int32_t batch, int64_t stride_q_bs, int64_t stride_q_h, int64_t stride_k_tok,
               int64_t stride_k_h, int64_t stride_v_tok, int64_t stride_v_h, int64_t stride_o_bs, int64_t stride_o_h,
               int64_t stride_o_split, int64_t stride_table_bs, const int32_t* seq_order, const fd_params* p,
               const FusedTail* tail, bool* fused, bool no_lse = false, bool skip_empty = false,
               LaunchShape* shape_only = nullptr) {
  if (fused) *fused = false;
  if (!p) return fail(FD_ERR_INVALID_ARG, "%s: params is NULL", fn);
  if (!q || !k_cache || !v_cache || !out_split || !block_table || !kv_lens)
    return fail(FD_ERR_INVALID_ARG, "%s: NULL tensor pointer", fn);
  if (batch < 0) return fail(FD_ERR_INVALID_ARG, "%s: batch = %d", fn, batch);
  if (batch == 0) return FD_OK;
  if (batch > 65535) return fail(FD_ERR_TOO_LARGE, "%s: batch %d > 65535 (grid z)", fn, batch);
  if (p->q_heads <= 0 || p->kv_heads <= 0 || p->q_heads % p->kv_heads != 0)
    return fail(FD_ERR_INVALID_ARG, "%s: q_heads %d must be a positive multiple of kv_heads %d", fn, p->q_heads,
                p->kv_heads);
  if (p->page_size <= 0 || p->num_splits <= 0 || p->num_pages <= 0 || p->max_pages_per_seq <= 0)
    return fail(FD_ERR_INVALID_ARG, "%s: page_size/num_splits/num_pages/max_pages_per_seq must be > 0", fn);
  if (p->num_splits > 65535) return fail(FD_ERR_TOO_LARGE, "%s: num_splits %d > 65535 (grid y)", fn, p->num_splits);
  if ((int64_t)p->num_pages * p->page_size >= (int64_t)1 << 31)
    return fail(FD_ERR_TOO_LARGE, "%s: pool of %lld token rows exceeds 2^31", fn,
                (long long)p->num_pages * p->page_size);
  if ((int64_t)p->max_pages_per_seq * p->page_size + p->num_splits >= (int64_t)1 << 31)
    return fail(FD_ERR_TOO_LARGE, "%s: block table capacity exceeds 2^31 tokens", fn);
  const int D = p->head_dim;
  if (D != 64 && D != 128 && D != 256) return fail(FD_ERR_UNSUPPORTED, "%s: head_dim %d (64/128/256)", fn, D);
  const int Dv = v_dim(p);
  if (Dv != 64 && Dv != 128 && Dv != 256) return fail(FD_ERR_UNSUPPORTED, "%s: v_head_dim %d (64/128/256)", fn, Dv);
  if (Dv != D && p->kv_dtype == FD_FP8_E4M3)
    return fail(FD_ERR_UNSUPPORTED, "%s: an fp8 cache needs equal K and V head dims (%d, %d)", fn, D, Dv);
  const int qsz = dtype_size(p->q_dtype), kvsz = dtype_size(p->kv_dtype), msz = dtype_size(p->mid_dtype);
  if (!qsz || p->q_dtype == FD_FP8_E4M3) return fail(FD_ERR_UNSUPPORTED, "%s: q_dtype %d", fn, p->q_dtype);
  if (!kvsz) return fail(FD_ERR_UNSUPPORTED, "%s: kv_dtype %d", fn, p->kv_dtype);
  if (!msz || p->mid_dtype == FD_FP8_E4M3) return fail(FD_ERR_UNSUPPORTED, "%s: mid_dtype %d", fn, p->mid_dtype);
  if (p->kv_dtype == FD_FP8_E4M3 && (!p->k_scale || !p->v_scale))
    return fail(FD_ERR_INVALID_ARG, "%s: fp8 KV cache needs k_scale and v_scale", fn);
  const int kv_elems16 = 16 / kvsz;
  if (!aligned16(k_cache) || !aligned16(v_cache) || stride_k_tok % kv_elems16 || stride_k_h % kv_elems16 ||
      stride_v_tok % kv_elems16 || stride_v_h % kv_elems16)
    return fail(FD_ERR_ALIGNMENT, "%s: K/V rows must be 16-byte aligned (pointer and token/head strides)", fn);
  if (stride_k_tok <= 0 || stride_v_tok <= 0 || stride_k_tok * kvsz >= ((int64_t)1 << 31) ||
      stride_v_tok * kvsz >= ((int64_t)1 << 31))
    return fail(FD_ERR_INVALID_ARG, "%s: token stride out of range", fn);
  const int G = p->q_heads / p->kv_heads;
  int64_t max_tok_split = (planned_tokens(p) + p->num_splits - 1) / p->num_splits;
  if (p->split_adapt > 0 && max_tok_split < kMinTokensPerRange)   // ranges by each sequence's own length
    max_tok_split = kMinTokensPerRange;

  SplitArgs a;
  memset(&a, 0, sizeof(a));
  a.q = q; a.k = k_cache; a.v = v_cache; a.out = out_split; a.lse = lse_split;
  a.bt = block_table; a.kv_lens = kv_lens; a.order = seq_order; a.order_lens = seq_order ? p->seq_order_lens : nullptr;
  if (seq_order && p->seq_order_items) {   // (sequence, range) items and, behind them, their lengths
    a.order_items = 1;
    a.order_lens = seq_order + (int64_t)batch * p->num_splits;
  }
  a.k_scale = p->k_scale; a.v_scale = p->v_scale;
  a.sq_b = stride_q_bs; a.sq_h = stride_q_h; a.sk_t = stride_k_tok; a.sk_h = stride_k_h;
  a.sv_t = stride_v_tok; a.sv_h = stride_v_h; a.so_b = stride_o_bs; a.so_h = stride_o_h; a.so_s = stride_o_split;
  a.sbt = stride_table_bs; a.no_lse = no_lse ? 1 : 0; a.skip_empty = skip_empty ? 1 : 0;
  a.sm_scale = sm_scale; a.soft_cap = p->soft_cap > 0.f ? p->soft_cap : 0.f;
  a.batch = batch; a.Hq = p->q_heads; a.Hkv = p->kv_heads; a.G = G; a.S = p->num_splits; a.P = p->page_size;
  div_magic((uint32_t)p->page_size, &a.div_magic, &a.div_shift);
  div_magic((uint32_t)p->num_splits, &a.s_magic, &a.s_shift);
  if (p->split_align < 0 || p->split_align > 4096 || (p->split_align & (p->split_align - 1)))
    return fail(FD_ERR_INVALID_ARG, "%s: split_align %d (0 or a power of two <= 4096)", fn, p->split_align);
  a.per_mask = p->split_align ? p->split_align - 1 : 0;
  if (int rc = check_split_adapt(fn, p)) return rc;
  a.adapt = p->split_adapt;
  a.max_pages = p->max_pages_per_seq; a.num_pages = p->num_pages;
  a.q_dtype = p->q_dtype; a.mid_dtype = p->mid_dtype;
  // fp32 rows, and 16-bit rows that start on a multiple of four elements, are stored four values at a time
  a.vec_out = msz == 4 ? ((reinterpret_cast<uintptr_t>(out_split) & 3) == 0 ? 1 : 0)
                       : ((reinterpret_cast<uintptr_t>(out_split) & (4u * msz - 1)) == 0 && stride_o_bs % 4 == 0 &&
                          stride_o_h % 4 == 0 && stride_o_split % 4 == 0) ? 1 : 0;

  // Tens of MB of partials left dirty in the L2s are written back when the kernel ends, with nothing to overlap;
  // written through they leave while other workgroups stream (config 5's shape, 64 splits, 67 MB of fp32 partials:
  // 204 -> 192 us; 4 MB of partials: no gain, so the plain store stays for those).
  {
    static const int forced = env_int("FD_STORE_THROUGH");   // tuning override for experiments: 1 always, 2 never
    const int64_t partial_bytes = (int64_t)batch * p->q_heads * p->num_splits * Dv * msz;
    a.store_through = forced != 2 && (forced == 1 || partial_bytes >= kStoreThroughBytes) ? 1 : 0;
  }

  const bool q16 = p->q_dtype == FD_BF16 || p->q_dtype == FD_F16;
  const bool kv_fp8 = p->kv_dtype == FD_FP8_E4M3;
  // V head dim 64 or 256 beside a K head dim of 128: the head_dim-128 16-bit kernel with its V side narrowed or split
  // into two members (groups of up to 16 query heads, two launches)
  const bool fuse_wanted = tail && tail->tickets && p->mid_dtype == FD_F32;
  const bool dv_mfma = Dv != D && D == 128 && !kv_fp8 && (Dv == 64 || Dv == 256) && G <= 16 && !fuse_wanted &&
                       stride_v_h % 8 == 0 && stride_v_tok % 8 == 0;
  const bool mfma_ok = mfma_shape_ok(D, p->kv_dtype) && (Dv == D || dv_mfma) && q16 &&
                       (kv_fp8 || p->q_dtype == p->kv_dtype) && aligned16(q) && stride_q_bs % 8 == 0 &&
                       stride_q_h % 8 == 0;
  bool use_mfma = mfma_ok;
  if (p->path == FD_PATH_VALU) use_mfma = false;
  if (p->path == FD_PATH_MFMA && !mfma_ok)
    return fail(FD_ERR_UNSUPPORTED,
                "%s: MFMA path needs a 16-bit query with a KV cache of the same dtype or fp8-e4m3, equal K and V head "
                "dims (or K 128 with V 64 / 256, 16-bit cache, up to 16 query heads per KV head, no fused combine) and "
                "16-byte aligned q rows", fn);
  if (p->waves_per_block != 0 && p->waves_per_block != 1 && p->waves_per_block != 2 && p->waves_per_block != 4 &&
      p->waves_per_block != 8)
    return fail(FD_ERR_INVALID_ARG, "%s: waves_per_block %d (0, 1, 2, 4 or 8)", fn, p->waves_per_block);

  // fp8 rows of head_dim 64 are half a cache line: where two adjacent KV heads' rows are one contiguous 128 bytes,
  // a wave of the MFMA kernel serves both, and the pair is presented to the kernel as one KV head with 2 G query heads
  const bool pair = use_mfma && kv_fp8 && D == 64 && fp8_d64_pairs(G, p->kv_heads) && stride_k_h == 64 && stride_v_h == 64;
  if (pair) {
    a.Hkv = p->kv_heads / 2;
    a.G = 2 * G;
  }
  int tile;
  if (use_mfma) {
    const int hb = pair ? 32 : mfma_head_block(D, G, p->kv_dtype);
    a.hbsz = a.G < hb ? a.G : hb;
    a.nhb = (a.G + hb - 1) / hb;
    tile = kv_fp8 ? (D == 256 ? 32 : 64) : (D == 64 ? 64 : (D == 256 ? 16 : 32));
  } else {
    a.hbsz = G >= 3 ? 4 : G;
    a.nhb = (G + a.hbsz - 1) / a.hbsz;
    tile = 4 * (64 / (D * kvsz / 16));
  }
  if ((int64_t)a.Hkv * a.nhb >= ((int64_t)1 << 31))
    return fail(FD_ERR_TOO_LARGE, "%s: %lld workgroups per split", fn, (long long)a.Hkv * a.nhb);
  const bool fuse = tail && tail->tickets && p->mid_dtype == FD_F32;
  // the two-block MFMA kernel needs the register file of a whole SIMD per wave: workgroups of at most 4 waves
  const int max_waves = use_mfma && (a.hbsz > 16 || pair) ? 4 : 8;
  // the fp8 head_dim-64 kernel keeps 8 KB in flight per wave with one KV head per wave, like the VALU kernel;
  // the other MFMA kernels 16 KB
  const int64_t wave_target = use_mfma && !(kv_fp8 && D == 64 && !pair) ? kTargetWaves : kTargetWavesValu;
  // Partials are parked finished -- normalised, in mid_dtype, the rows of the real heads only: 2 KB for 8 heads in
  // bf16 against 8.3 KB of raw state -- and a wave walks up to four splits.
  const int hb_slots = a.hbsz > 16 ? 32 : 16;
  // What a wish of `wish` consecutive splits per work item becomes: the waves of a head take whole splits,
  // kMaxSplitsPerWave at most -- a wave keeps the finished partials of all but its last split in LDS until it has
  // issued its last load (stores and loads of a wave retire in order, so a store between two tiles would hold back
  // the loads behind it) --, so the chunk is a multiple of the waves, rounded down or up.  wgs: (sequence, work item,
  // KV head, head block) units before that rounding, which the choices that follow were tuned with; grid_waves: the
  // waves the grid will hold.
  struct ChunkPlan { int chunk, waves, per_wave; int64_t wgs, grid_waves; };
  auto chunk_plan = [&](int wish, bool round_up) {
    ChunkPlan c;
    const int items = (a.S + wish - 1) / wish;   // work items per (sequence, KV head, head block)
    // Ranges that are certain to be busy per sequence: all of them, or, when the ranges follow each sequence's own
    // length, only the ones every sequence gets (the rest of the grid may be empty ranges).
    const int busy_splits = a.adapt > 0 && a.adapt < a.S ? a.adapt : items;
    c.wgs = (int64_t)batch * busy_splits * a.Hkv * a.nhb;
    c.waves = p->waves_per_block ? (p->waves_per_block < max_waves ? p->waves_per_block : max_waves)
                                 : choose_waves(c.wgs, max_tok_split * wish, tile, wave_target, max_waves);
    // A batch planned by its block table's capacity rarely fills it: the sequences of a serving batch differ in
    // length and most of their grid slots are short or empty, so the chip holds fewer waves than the count above
    // assumes.  Two waves per range then (head_dim 128: 96 ragged sequences of up to 8192 tokens 290 -> 271 us, 128
    // of them 373 -> 339 us; batches that do fill their tables lose nothing: 96 x 16384 tokens 1045 -> 929 us; the
    // other MFMA kernels alike, scheduled: head_dim 64 40 sequences of up to 16384 tokens 134 -> 116 us, fp8 head_dim
    // 256 96 of up to 8192 tokens 321 -> 280 us, fp8 head_dim 128 256 of up to 2048 tokens in one split 98 -> 87 us;
    // not the fp8 head_dim-64 kernel, whose waves serve two KV heads each).
    // Four in a small batch whose full-length ranges have 3072 tokens or more: its few longest sequences are the last
    // to finish, and their waves alone must keep the memory busy (16 ragged sequences of up to 32768 tokens 166 -> 149
    // us, on an fp8 cache with 64 query heads 108 -> 88 us; from 32 sequences on it gains nothing, and config 5's fp8
    // step lost 6 % to it: four waves per range leave room for two sibling KV heads instead of four).
    if (use_mfma && !(kv_fp8 && D == 64) && a.adapt > 0 && batch > 1 && !p->waves_per_block && env_waves() == 0) {
      const int at_least = D == 128 && a.S > 1 && batch <= 24 && max_tok_split * wish >= kMaxTokensPerRange * 3 / 4 && max_waves >= 4 ? 4 : 2;
      if (c.waves < at_least && max_tok_split * wish >= at_least * tile) c.waves = at_least;
    }
    c.per_wave = 1;
    c.chunk = wish;
    if (wish > 1) {
      while (c.waves > 1 && c.waves > wish) c.waves >>= 1;
      c.per_wave = round_up ? (wish + c.waves - 1) / c.waves : wish / c.waves;
      if (c.per_wave > kMaxSplitsPerWave) c.per_wave = kMaxSplitsPerWave;
      c.chunk = c.waves * c.per_wave;
    }
    c.grid_waves = (int64_t)batch * ((a.S + c.chunk - 1) / c.chunk) * a.Hkv * a.nhb * c.waves;
    return c;
  };
  // Chunked work items: the caller's split count and ranges are kept exactly (they are observable in out_split), but a
  // workgroup walks `chunk` consecutive splits, so that the chip sees about as many work items as the library's own
  // plan would launch: every work item pays the prologue (arguments -> length -> block table -> first rows) once, not
  // once per split.  Kernels that have this form: head_dim 128, 16-bit and fp8 caches.  (The head_dim 64 and 256
  // kernels were given it as well and measured level with one workgroup per split -- config 2's shape with 32
  // caller-visible bf16 partials: head_dim 256 91.8 against 92.4 us, head_dim 64 27.9 against 27.3 us; in the
  // library's own layout 90.4 against 89.7 and 26.6 against 26.2 us -- so they launch a workgroup per split.)
  // Not for large batches: their lengths differ in practice, and many short work items balance better over the CUs
  // than few long ones (config 4's ragged batch of 64 with exactly 32 splits: 691 us unchunked, 713 us chunked).
  ChunkPlan cp = chunk_plan(1, false);
  if (use_mfma && D == 128 && Dv == D && !fuse && a.adapt == 0 && !a.order_items && !skip_empty && !no_lse && a.S > 1 &&
      batch <= kMaxChunkBatch && !env_no_chunk()) {
    fd_params plan = *p;
    plan.split_adapt = 0;
    const int s_plan = fd_plan_splits(&plan, batch);
    if (s_plan > 0 && s_plan < a.S) {
      // Splits per work item: the split count over the plan's, rounded up -- few long work items -- unless that
      // leaves the grid short of the waves that keep the memory system busy (a split count the plan does not divide:
      // 12 splits against a plan of 8 as 6 items of two are 768 waves on config 2's shape, 55 us; as 12 items 48 us;
      // one sequence of 131072 tokens with 24 splits 148 against 95 us), then rounded down: at least as many items as
      // the plan has.
      cp = chunk_plan((a.S + s_plan - 1) / s_plan, true);
      if (cp.grid_waves < wave_target * 7 / 8) cp = chunk_plan(a.S / s_plan, false);
    }
  }
  a.chunk = cp.chunk;
  const int64_t wgs = cp.wgs;
  int waves = cp.waves;
  int chunk_per_wave = cp.per_wave;
  if (a.chunk > 1) {
    a.park_bytes = hb_slots * 4 + a.hbsz * D * msz;
    a.park = chunk_per_wave - 1;
  }
  // Heads per workgroup: only the MFMA kernels, and not with the fused combine (its tickets are per KV head).
  a.hpw = 1;
  if (use_mfma && !fuse && a.nhb > 1) {
    // more query heads per KV head than one wave serves: the head blocks of a KV head share a workgroup (largest divisor of
    // nhb that keeps the workgroup at 8 waves and the grid at one workgroup per CU), so that they read their
    // common K/V rows in step
    int h = max_waves / waves;
    if (env_heads() > 0 && env_heads() < h) h = env_heads();   // same tuning override as for sibling KV heads
    while (h > 1 && (a.nhb % h != 0 || wgs / h < kMinWorkgroups)) --h;
    if (h > 1) {
      a.hpw = h;
      a.member_hb = 1;
    }
  } else if (use_mfma && !fuse) {
    a.hpw = choose_heads_per_group(a.Hkv, D * kvsz * (pair ? 2 : 1), waves, wgs, max_waves);
  }
  // V head dim: the column of an in-row LSE; on the head_dim-128 MFMA kernel a V head dim of 256 makes every KV head
  // two workgroup members (one per 128-column half), one of 64 narrows the V fetch and the stored columns
  a.dv = Dv;
  a.v_members = 1;
  a.v_chunk_mask = 15;
  a.v_cols = 1 << 30;
  if (use_mfma && Dv != D) {
    if (Dv == 256) {
      while (waves * 2 > max_waves) waves >>= 1;
      const int heads = choose_heads_per_group(a.Hkv, D * kvsz, waves * 2, wgs, max_waves);
      a.v_members = 2;
      a.hpw = 2 * heads;
    } else {
      a.v_chunk_mask = 7;
      a.v_cols = 64;
    }
  }
  if (a.chunk > 1) {
    // two chunked workgroups per CU: fewer parked splits per wave if their LDS would not allow it
    const int wave_lds = hb_slots_lds(a.hbsz);
    while (chunk_per_wave > 1 &&
           (int64_t)a.hpw * waves * (wave_lds + (int64_t)(chunk_per_wave - 1) * a.park_bytes) > kChunkLdsBytes)
      --chunk_per_wave;
    a.chunk = waves * chunk_per_wave;
    a.park = chunk_per_wave - 1;
  }
  a.grid_x = a.member_hb ? a.Hkv * (a.nhb / a.hpw) : a.Hkv / (a.hpw / a.v_members) * a.nhb;
  a.nsub = waves;
  waves *= a.hpw;   // total waves of a workgroup

  // fuse the combine into the split kernel's tail when a ticket buffer is there and the LSEs fit in LDS
  if (fuse) {  // the fused tail exchanges fp32 partials only
    const size_t lse_lds = (size_t)(a.S + tail->num_extra) * (pair ? 32 : use_mfma && a.hbsz < 16 ? 16 : a.hbsz) * 4;
    if (lse_lds <= kMaxLds / 2) {
      a.tickets = tail->tickets; a.fout = tail->out; a.flse = tail->lse_out;
      a.extra_out = tail->extra_out; a.extra_lse = tail->extra_lse;
      a.sfo_b = tail->stride_obs; a.sfo_h = tail->stride_oh;
      a.out_dtype = p->out_dtype; a.num_extra = tail->num_extra; a.lse_column = tail->lse_column;
      if (fused) *fused = true;
    }
  }

  if (shape_only) {
    shape_only->mfma = use_mfma ? 1 : 0;
    shape_only->tile = tile;
    shape_only->waves_per_head = a.nsub;
    shape_only->members = a.hpw;
    shape_only->chunk = a.chunk;
    shape_only->head_block = a.hbsz;
    shape_only->store_through = a.store_through;
    const dim3 grid = fd_split_grid(a);
    shape_only->grid[0] = grid.x; shape_only->grid[1] = grid.y; shape_only->grid[2] = grid.z;
    return FD_OK;
  }
  int rc;
  if (use_mfma && kv_fp8 && D == 256) {
    rc = fd_launch_split_mfma_fp8_d256((hipStream_t)stream, a, p->q_dtype, waves, a.soft_cap > 0.f);
  } else if (use_mfma && kv_fp8 && D == 64) {
    rc = fd_launch_split_mfma_fp8_d64((hipStream_t)stream, a, p->q_dtype, waves, a.soft_cap > 0.f, pair ? 2 : 1);
  } else if (use_mfma && kv_fp8) {
    rc = fd_launch_split_mfma_fp8((hipStream_t)stream, a, p->q_dtype, waves, a.soft_cap > 0.f);
  } else if (use_mfma && D == 64) {
    rc = fd_launch_split_mfma_d64((hipStream_t)stream, a, p->kv_dtype, waves, a.soft_cap > 0.f);
  } else if (use_mfma && D == 256) {
    rc = fd_launch_split_mfma_d256((hipStream_t)stream, a, p->kv_dtype, waves, a.soft_cap > 0.f);
  } else if (use_mfma) {
    rc = fd_launch_split_mfma((hipStream_t)stream, a, p->kv_dtype, waves, a.soft_cap > 0.f);
  } else {
    rc = fd_launch_split_valu((hipStream_t)stream, a, p->kv_dtype, D, Dv, waves);
  }
  if (rc == FD_ERR_LAUNCH) return fail(rc, "%s: launch failed: %s", fn, hipGetErrorString(hipGetLastError()));
  if (rc != FD_OK) return fail(rc, "%s: no kernel for kv_dtype %d, head_dim %d, group %d", fn, p->kv_dtype, D, G);
  return FD_OK;
}

}  // namespace

extern "C" {

// The ranges of a decode step with these parameters, for the schedulers.
static int range_plan(const char* fn, const fd_params* p, RangePlan* rp) {
  if (p->num_splits <= 0 || p->num_splits > 65535)
    return fail(FD_ERR_INVALID_ARG, "%s: num_splits %d", fn, p->num_splits);
  if (p->split_align < 0 || p->split_align > 4096 || (p->split_align & (p->split_align - 1)))
    return fail(FD_ERR_INVALID_ARG, "%s: split_align %d (0 or a power of two <= 4096)", fn, p->split_align);
  if (int rc = check_split_adapt(fn, p)) return rc;
  rp->S = p->num_splits;
  div_magic((uint32_t)p->num_splits, &rp->s_magic, &rp->s_shift);
  rp->per_mask = p->split_align ? p->split_align - 1 : 0;
  rp->adapt = p->split_adapt;
  return FD_OK;
}

static int combine_impl(void* stream, const void* mid_o, const float* mid_lse, void* out, float* lse_out,
                        const int32_t* seqlens, int32_t batch, int32_t q_heads, int32_t num_partials,
                        int64_t stride_mid_ob, int64_t stride_mid_oh, int64_t stride_mid_os, int64_t stride_obs,
                        int64_t stride_oh, int32_t mode, const void* extra_out, const float* extra_lse,
                        int32_t num_extra, const fd_params* p, bool all_slots_written);

int fd_split_kv(void* stream, const void* q, const void* k_cache, const void* v_cache, void* out_split,
                float* lse_split, float sm_scale, const int32_t* block_table, const int32_t* kv_lens, int32_t batch,
                int64_t stride_q_bs, int64_t stride_q_h, int64_t stride_k_tok, int64_t stride_k_h,
                int64_t stride_v_tok, int64_t stride_v_h, int64_t stride_o_bs, int64_t stride_o_h,
                int64_t stride_o_split, int64_t stride_table_bs, const int32_t* seq_order, const fd_params* p) {
  return split_impl("fd_split_kv", stream, q, k_cache, v_cache, out_split, lse_split, sm_scale, block_table, kv_lens,
                    batch, stride_q_bs, stride_q_h, stride_k_tok, stride_k_h, stride_v_tok, stride_v_h, stride_o_bs,
                    stride_o_h, stride_o_split, stride_table_bs, seq_order, p, nullptr, nullptr);
}

int fd_decode(void* stream, const void* q, const void* k_cache, const void* v_cache, void* out_split,
              float* lse_split, void* out, float* lse_out, float sm_scale, const int32_t* block_table,
              const int32_t* kv_lens, int32_t batch, int64_t stride_q_bs, int64_t stride_q_h, int64_t stride_k_tok,
              int64_t stride_k_h, int64_t stride_v_tok, int64_t stride_v_h, int64_t stride_o_bs, int64_t stride_o_h,
              int64_t stride_o_split, int64_t stride_table_bs, int64_t stride_obs, int64_t stride_oh,
              const int32_t* seq_order, int32_t combine_mode, const void* extra_out, const float* extra_lse,
              int32_t num_extra, int32_t* tickets, const fd_params* p) {
  if (!out) return fail(FD_ERR_INVALID_ARG, "fd_decode: out is NULL");
  if (combine_mode != FD_COMBINE_SPLIT && combine_mode != FD_COMBINE_SPLIT_LSE)
    return fail(FD_ERR_INVALID_ARG, "fd_decode: combine_mode %d (FD_COMBINE_SPLIT or FD_COMBINE_SPLIT_LSE)",
                combine_mode);
  if (num_extra < 0 || (num_extra > 0 && (!extra_out || !extra_lse)))
    return fail(FD_ERR_INVALID_ARG, "fd_decode: num_extra %d needs extra_out and extra_lse", num_extra);
  if (p && (!dtype_size(p->out_dtype) || p->out_dtype == FD_FP8_E4M3))
    return fail(FD_ERR_UNSUPPORTED, "fd_decode: out_dtype %d", p->out_dtype);
  if (p && p->rank_merge && tickets)
    return fail(FD_ERR_INVALID_ARG, "fd_decode: rank_merge is not available with a ticket buffer (fused combine)");
  if (!out_split) {
    // One split and nothing else to merge: its normalised partial IS the result.  The split kernel writes
    // it (and the LSE) in the output's place and dtype; no combine launch.
    if (!p) return fail(FD_ERR_INVALID_ARG, "fd_decode: params is NULL");
    if (p->num_splits != 1 || num_extra != 0)
      return fail(FD_ERR_INVALID_ARG, "fd_decode: out_split may be NULL only with num_splits == 1 and no extra partials");
    if (combine_mode == FD_COMBINE_SPLIT_LSE && lse_out)
      return fail(FD_ERR_INVALID_ARG, "fd_decode: without out_split the LSE goes to lse_out or to the output column, not both");
    fd_params direct = *p;
    direct.mid_dtype = p->out_dtype;
    return split_impl("fd_decode", stream, q, k_cache, v_cache, out, lse_out, sm_scale, block_table, kv_lens, batch,
                      stride_q_bs, stride_q_h, stride_k_tok, stride_k_h, stride_v_tok, stride_v_h, stride_obs, stride_oh,
                      0, stride_table_bs, seq_order, &direct, nullptr, nullptr,
                      combine_mode == FD_COMBINE_SPLIT && !lse_out);
  }
  FusedTail tail;
  tail.tickets = tickets; tail.out = out; tail.lse_out = lse_out; tail.extra_out = extra_out;
  tail.extra_lse = extra_lse; tail.stride_obs = stride_obs; tail.stride_oh = stride_oh; tail.num_extra = num_extra;
  tail.lse_column = combine_mode == FD_COMBINE_SPLIT_LSE;
  bool fused = false;
  // Ranges that follow each sequence's own length leave most slots of a long split list empty: beyond what the
  // small combine kernel takes in one gulp, the empty ranges' workgroups write nothing and the combine derives
  // from kv_lens which slots hold a partial (one more dependent load there, no traffic for the empty ones).
  const bool skip_empty = p && p->split_adapt > 0 && p->split_adapt < p->num_splits &&
                          p->num_splits > kCombineSmallMax && !tickets;
  int rc = split_impl("fd_decode", stream, q, k_cache, v_cache, out_split, lse_split, sm_scale, block_table, kv_lens,
                      batch, stride_q_bs, stride_q_h, stride_k_tok, stride_k_h, stride_v_tok, stride_v_h, stride_o_bs,
                      stride_o_h, stride_o_split, stride_table_bs, seq_order, p, &tail, &fused, false, skip_empty);
  if (rc != FD_OK || fused || batch == 0) return rc;
  return combine_impl(stream, out_split, lse_split, out, lse_out, kv_lens, batch, p->q_heads, p->num_splits,
                      stride_o_bs, stride_o_h, stride_o_split, stride_obs, stride_oh, combine_mode, extra_out,
                      extra_lse, num_extra, p, !skip_empty);
}

int fd_decode_noalloc(void* stream, const void* q, const void* k_cache, const void* v_cache, void* out, float* lse_out,
                      float sm_scale, const int32_t* block_table, const int32_t* kv_lens, int32_t batch,
                      int64_t stride_q_bs, int64_t stride_q_h, int64_t stride_k_tok, int64_t stride_k_h,
                      int64_t stride_v_tok, int64_t stride_v_h, int64_t stride_table_bs, int64_t stride_obs,
                      int64_t stride_oh, const int32_t* seq_order, int32_t combine_mode, const void* extra_out,
                      const float* extra_lse, int32_t num_extra, const fd_params* p) {
  const char* fn = "fd_decode_noalloc";
  if (!p) return fail(FD_ERR_INVALID_ARG, "%s: params is NULL", fn);
  if (batch < 0 || p->q_heads <= 0 || p->num_splits <= 0 || p->head_dim <= 0)
    return fail(FD_ERR_INVALID_ARG, "%s: batch %d, q_heads %d, num_splits %d, head_dim %d", fn, batch, p->q_heads,
                p->num_splits, p->head_dim);
  const bool lse_twice = combine_mode == FD_COMBINE_SPLIT_LSE && lse_out;
  if (p->num_splits == 1 && num_extra == 0 && !lse_twice)   // one split: written straight to `out`, no partials at all
    return fd_decode(stream, q, k_cache, v_cache, nullptr, nullptr, out, lse_out, sm_scale, block_table, kv_lens, batch,
                     stride_q_bs, stride_q_h, stride_k_tok, stride_k_h, stride_v_tok, stride_v_h, 0, 0, 0,
                     stride_table_bs, stride_obs, stride_oh, seq_order, combine_mode, extra_out, extra_lse, num_extra,
                     nullptr, p);
  // fp32 partials [batch, Hq, S, D] followed by their fp32 LSEs [batch, Hq, S]
  const int64_t rows = (int64_t)batch * p->q_heads * p->num_splits;
  const int64_t need = rows * (v_dim(p) + 1) * 4;
  if (need > (int64_t)FD_NOALLOC_SCRATCH_BYTES)
    return fail(FD_ERR_TOO_LARGE,
                "%s: batch %d x q_heads %d x num_splits %d x (head_dim %d + 1) fp32 partials = %lld bytes exceed the "
                "static workspace of %lld bytes; use fewer splits (fd_plan_splits) or fd_decode with a workspace of "
                "your own", fn, batch, p->q_heads, p->num_splits, v_dim(p), (long long)need,
                (long long)FD_NOALLOC_SCRATCH_BYTES);
  if (batch == 0) return FD_OK;
  void* ws = scratch_on_current_device(fn);
  if (!ws) return FD_ERR_LAUNCH;
  fd_params own = *p;
  own.mid_dtype = FD_F32;
  const int64_t D = v_dim(p), S = p->num_splits;
  float* lse_split = (float*)ws + rows * D;
  return fd_decode(stream, q, k_cache, v_cache, ws, lse_split, out, lse_out, sm_scale, block_table, kv_lens, batch,
                   stride_q_bs, stride_q_h, stride_k_tok, stride_k_h, stride_v_tok, stride_v_h,
                   (int64_t)p->q_heads * S * D, S * D, D, stride_table_bs, stride_obs, stride_oh, seq_order,
                   combine_mode, extra_out, extra_lse, num_extra, nullptr, &own);
}

// Splits a shape needs to fill the chip, regardless of how long its sequences are (a power of two >= 1), or a
// negative fd_status.  fd_plan_splits adds the bound on the length of a split and the caller's limit.
static int64_t plan_fill_splits(const char* fn, const fd_params* p, int32_t batch) {
  if (!p) return fail(FD_ERR_INVALID_ARG, "%s: params is NULL", fn);
  if (batch <= 0 || p->q_heads <= 0 || p->kv_heads <= 0 || p->q_heads % p->kv_heads != 0 || p->num_splits <= 0 ||
      p->page_size <= 0 || p->max_pages_per_seq <= 0)
    return fail(FD_ERR_INVALID_ARG, "%s: batch, heads, num_splits, page_size, max_pages_per_seq must be > 0", fn);
  const int G = p->q_heads / p->kv_heads;
  const bool dv_mfma = p->head_dim == 128 && p->kv_dtype != FD_FP8_E4M3 && (v_dim(p) == 64 || v_dim(p) == 256) && G <= 16;
  const bool mfma = mfma_shape_ok(p->head_dim, p->kv_dtype) && (v_dim(p) == p->head_dim || dv_mfma) &&
                    p->path != FD_PATH_VALU;
  const int hb = mfma ? mfma_head_block(p->head_dim, G, p->kv_dtype) : (G >= 3 ? 4 : G);
  const int64_t nhb = (G + hb - 1) / hb;
  // fp8 rows of head_dim 64: two KV heads per wave (the usual cache layout has their rows side by side)
  const bool pair = mfma && p->kv_dtype == FD_FP8_E4M3 && p->head_dim == 64 && fp8_d64_pairs(G, p->kv_heads);
  const int kv_units = pair ? p->kv_heads / 2 : p->kv_heads;
  const int64_t groups = (int64_t)batch * kv_units * nhb;        // (KV head, head block) pairs per split
  const int64_t max_tokens = planned_tokens(p);
  int64_t s = 1;
  if (mfma) {
    // (1) one workgroup per CU at the full member width (sibling KV heads, or head blocks of one KV head): measured
    // over head dims, cache dtypes and batch sizes, 256 workgroups x 4 waves beats 512 x 2 and 128 x 8 ...
    int members = 1;
    if (nhb > 1) {
      for (int h = 4; h > 1; --h)
        if (nhb % h == 0) { members = h; break; }
    } else {
      const int row_bytes = p->head_dim * dtype_size(p->kv_dtype) * (pair ? 2 : 1);
      members = row_bytes > 0 && row_bytes < 512 ? 512 / row_bytes : 1;
      while (members > 1 && kv_units % members != 0) members >>= 1;
    }
    while (s * groups < kMinWorkgroups * members) s <<= 1;
    if (s * groups != kMinWorkgroups * members) {
      // (1b) The groups do not divide the CU count (12 KV heads): no power of two gives one workgroup per CU.  The
      // count just under it does -- 12 x 42 / 2 = 252 workgroups in one round -- with far fewer partials than the
      // power of two that reaches a whole number per CU (128 splits, 768 workgroups): one query, 96 / 12 heads,
      // 65536 tokens 72.2 -> 68.2 us, 1048576 tokens 953.6 -> 949.0 us.  Where a split would hold fewer than 512
      // tokens the sibling members are given up for half as many splits (16384 tokens: 25.5 -> 23.3 us with 21).
      int64_t m = members;
      int64_t exact = kMinWorkgroups * m / groups;
      while (m > 1 && exact > 0 && max_tokens / exact < 512) {
        m >>= 1;
        exact = kMinWorkgroups * m / groups;
      }
      if (exact >= 2 && exact * groups * 10 >= kMinWorkgroups * m * 9) return exact;
    }
    // (2) ... and a whole number of workgroups per CU, or at least four, while a split of a full-length sequence
    // keeps 512 tokens: equal work items run in one round, and 1.5 workgroups per CU take as long as 2
    while (s < p->num_splits && (s * groups / members) % kMinWorkgroups != 0 &&
           s * groups / members < 4 * kMinWorkgroups && 2 * s * 512 <= max_tokens)
      s <<= 1;
  } else {
    // the VALU kernel keeps half as many bytes in flight per wave: twice the waves, four per (KV head, split)
    while (s * 4 * groups < kTargetWavesValu) s <<= 1;
  }
  return s;
}

int fd_plan_min_splits(const fd_params* p, int32_t batch) {
  const int64_t s = plan_fill_splits("fd_plan_min_splits", p, batch);
  if (s < 0) return (int)s;
  int64_t pow2 = 1;   // fd_params.split_adapt is a power of two: the next one
  while (pow2 < s && pow2 < 65536) pow2 <<= 1;
  return (int)pow2;
}

int fd_plan_splits(const fd_params* p, int32_t batch) {
  int64_t s = plan_fill_splits("fd_plan_splits", p, batch);
  if (s < 0) return (int)s;
  // (3) in a batch, enough splits that no split of a full-length sequence is longer than kMaxTokensPerSplit: the
  // dispatcher evens out ragged lengths with them
  const int64_t max_tokens = planned_tokens(p);
  // -- up to kMaxBalanceSplits: the grid has that many slots for EVERY sequence of the batch, and the ones a shorter
  // sequence leaves empty still cost an issue slot each (a table sized for 1 M tokens would put 256 x batch x KV heads
  // mostly empty workgroups in front of the chip); sequences beyond 32 x 4096 tokens get longer ranges instead.
  if (batch > 1) {
    while (s * kMaxTokensPerSplit < max_tokens && s < kMaxBalanceSplits) s <<= 1;
  }
  // No floor on the tokens of a split by default: cutting a short table into one- and two-tile splits was measured
  // against fewer, longer ones (FD_PLAN_MIN_TOKENS = 64 ... 512; graph replays) and the many short splits are level or
  // ahead -- 3 sequences of 512 tokens on 8 KV heads 7.5 us with 10 splits against 8.4 / 9.3 us with 4 / 2, of 1024
  // tokens 7.8 against 8.5 / 9.3 / 10.5 us with 8 / 4 / 2, one query on 12 KV heads over 2048 tokens 9.0 us with 21
  // splits against 9.9 / 12.2 us with 8 / 4: such steps are latency, and more workgroups hide more of it.
  {
    static const int min_tokens = env_int("FD_PLAN_MIN_TOKENS") > 0 ? env_int("FD_PLAN_MIN_TOKENS") : kPlanMinTokensPerSplit;
    if (min_tokens > 0) {
      int64_t most = max_tokens / min_tokens;
      if (most < 1) most = 1;
      if (s > most) {
        const bool was_pow2 = (s & (s - 1)) == 0;
        s = most;
        if (was_pow2) while (s & (s - 1)) s &= s - 1;   // stay a power of two
      }
    }
  }
  // Powers of two where the shape allows: with sequence lengths that are powers of two (or multiples of large ones)
  // every split then starts on a tile boundary and the waves of a workgroup get equal runs.
  const bool pow2 = (s & (s - 1)) == 0;
  while (pow2 && s > p->num_splits) s >>= 1;
  if (s > p->num_splits) s = p->num_splits;
  if (s < 1) s = 1;
  return (int)s;
}

static int combine_impl(void* stream, const void* mid_o, const float* mid_lse, void* out, float* lse_out,
                        const int32_t* seqlens, int32_t batch, int32_t q_heads, int32_t num_partials,
                        int64_t stride_mid_ob, int64_t stride_mid_oh, int64_t stride_mid_os, int64_t stride_obs,
                        int64_t stride_oh, int32_t mode, const void* extra_out, const float* extra_lse,
                        int32_t num_extra, const fd_params* p, bool all_slots_written) {
  if (!p) return fail(FD_ERR_INVALID_ARG, "fd_combine: params is NULL");
  if (!mid_o || !out || !seqlens) return fail(FD_ERR_INVALID_ARG, "fd_combine: NULL tensor pointer");
  if (batch < 0 || q_heads <= 0 || num_partials <= 0 || num_extra < 0)
    return fail(FD_ERR_INVALID_ARG, "fd_combine: batch %d, q_heads %d, num_partials %d, num_extra %d", batch, q_heads,
                num_partials, num_extra);
  if (batch == 0) return FD_OK;
  if (mode != FD_COMBINE_SPLIT && mode != FD_COMBINE_SPLIT_LSE && mode != FD_COMBINE_RANK)
    return fail(FD_ERR_INVALID_ARG, "fd_combine: mode %d", mode);
  if (num_extra > 0 && (!extra_out || !extra_lse))
    return fail(FD_ERR_INVALID_ARG, "fd_combine: num_extra > 0 needs extra_out and extra_lse");
  if (v_dim(p) != 64 && v_dim(p) != 128 && v_dim(p) != 256)
    return fail(FD_ERR_UNSUPPORTED, "fd_combine: head dim of the partials %d (64/128/256)", v_dim(p));
  if (!dtype_size(p->mid_dtype) || p->mid_dtype == FD_FP8_E4M3 || !dtype_size(p->out_dtype) ||
      p->out_dtype == FD_FP8_E4M3)
    return fail(FD_ERR_UNSUPPORTED, "fd_combine: mid_dtype %d / out_dtype %d", p->mid_dtype, p->out_dtype);
  if ((int64_t)batch * q_heads >= ((int64_t)1 << 31)) return fail(FD_ERR_TOO_LARGE, "fd_combine: batch * q_heads");
  CombineArgs a;
  memset(&a, 0, sizeof(a));
  a.mid_o = mid_o; a.mid_lse = mid_lse; a.out = out; a.lse_out = lse_out; a.seqlens = seqlens;
  a.extra_out = extra_out; a.extra_lse = extra_lse;
  a.s_mb = stride_mid_ob; a.s_mh = stride_mid_oh; a.s_ms = stride_mid_os; a.s_ob = stride_obs; a.s_oh = stride_oh;
  a.batch = batch; a.Hq = q_heads; a.D = v_dim(p); a.num_partials = num_partials; a.num_extra = num_extra;
  a.mode = mode; a.mid_dtype = p->mid_dtype; a.out_dtype = p->out_dtype;
  // Rows that start on a multiple of four elements are read four values at a time.  (A 128-bit load would do with a
  // 4-byte boundary, but reading the reference's fp32 [.., D + 1] rows that way is slower than one element per thread
  // and load, consecutive threads on consecutive elements: config 2 with 32 such partials 4.3 against 3.7 us.)
  a.vec_mid = ((reinterpret_cast<uintptr_t>(mid_o) & (4u * dtype_size(p->mid_dtype) - 1)) == 0 && stride_mid_ob % 4 == 0 &&
               stride_mid_oh % 4 == 0 && stride_mid_os % 4 == 0) ? 1 : 0;
  a.all_slots_written = all_slots_written ? 1 : 0;
  if (p->split_align < 0 || p->split_align > 4096 || (p->split_align & (p->split_align - 1)))
    return fail(FD_ERR_INVALID_ARG, "fd_combine: split_align %d (0 or a power of two <= 4096)", p->split_align);
  a.per_mask = p->split_align ? p->split_align - 1 : 0;
  if (mode != FD_COMBINE_RANK) {
    a.adapt = p->split_adapt;
    if (a.adapt < 0 || (a.adapt & (a.adapt - 1)) || (a.adapt > 0 && p->split_align <= 0))
      return fail(FD_ERR_INVALID_ARG, "fd_combine: split_adapt %d needs a power of two and split_align > 0", a.adapt);
  }
  div_magic((uint32_t)num_partials, &a.s_magic, &a.s_shift);
  // Lengths beyond the block table's capacity are clamped exactly as the split kernels clamp them, so that both
  // agree on which ranges exist; a caller that names no table still gets kv_len + num_partials - 1 < 2^31.
  a.capacity = ((int64_t)1 << 31) - 1 - num_partials;
  if (p->max_pages_per_seq > 0 && p->page_size > 0) {
    const int64_t cap = (int64_t)p->max_pages_per_seq * p->page_size;
    if (cap < a.capacity) a.capacity = cap;
  }
  if (const fd_rank_merge* rm = p->rank_merge) {
    if (mode == FD_COMBINE_RANK) return fail(FD_ERR_INVALID_ARG, "fd_combine: rank_merge goes with the split modes");
    if (!rm->rank_lens || rm->this_rank < 0 || rm->this_rank > num_extra)
      return fail(FD_ERR_INVALID_ARG, "fd_combine: rank_merge needs rank_lens and 0 <= this_rank %d <= num_extra %d",
                  rm->this_rank, num_extra);
    a.rank_lens = rm->rank_lens;
    a.this_rank = rm->this_rank;
    if (rm->local_out) {
      if (!dtype_size(rm->local_dtype) || rm->local_dtype == FD_FP8_E4M3)
        return fail(FD_ERR_UNSUPPORTED, "fd_combine: rank_merge.local_dtype %d", rm->local_dtype);
      if ((int64_t)num_partials + num_extra > 1024)
        return fail(FD_ERR_TOO_LARGE, "fd_combine: rank_merge.local_out with more than 1024 partials");
      a.local_out = rm->local_out;
      a.local_dtype = rm->local_dtype;
      a.s_lb = rm->stride_lb;
      a.s_lh = rm->stride_lh;
    }
  }
  int rc = fd_launch_combine((hipStream_t)stream, a);
  if (rc != FD_OK) return fail(rc, "fd_combine: launch failed: %s", hipGetErrorString(hipGetLastError()));
  return FD_OK;
}

int fd_combine(void* stream, const void* mid_o, const float* mid_lse, void* out, float* lse_out,
               const int32_t* seqlens, int32_t batch, int32_t q_heads, int32_t num_partials, int64_t stride_mid_ob,
               int64_t stride_mid_oh, int64_t stride_mid_os, int64_t stride_obs, int64_t stride_oh, int32_t mode,
               const void* extra_out, const float* extra_lse, int32_t num_extra, const fd_params* p) {
  return combine_impl(stream, mid_o, mid_lse, out, lse_out, seqlens, batch, q_heads, num_partials, stride_mid_ob,
                      stride_mid_oh, stride_mid_os, stride_obs, stride_oh, mode, extra_out, extra_lse, num_extra, p,
                      false);
}

int fd_kv_append(void* stream, const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                 const int32_t* block_table, const int32_t* kv_lens, int32_t* kv_lens_out, int32_t* seq_order_out,
                 int32_t batch, int32_t new_tokens, int64_t stride_kn_b, int64_t stride_kn_t, int64_t stride_kn_h,
                 int64_t stride_vn_b, int64_t stride_vn_t, int64_t stride_vn_h, int64_t stride_k_tok,
                 int64_t stride_k_h, int64_t stride_v_tok, int64_t stride_v_h, int64_t stride_table_bs,
                 const fd_qk_prep* prep, const fd_params* p) {
  const char* fn = "fd_kv_append";
  if (!p) return fail(FD_ERR_INVALID_ARG, "%s: params is NULL", fn);
  if (batch < 0 || new_tokens < 0) return fail(FD_ERR_INVALID_ARG, "%s: batch %d, new_tokens %d", fn, batch, new_tokens);
  if (batch == 0 || new_tokens == 0) return FD_OK;
  const bool append = k_new || v_new;
  const bool with_q = prep && prep->q;
  if (seq_order_out && !append) return fail(FD_ERR_INVALID_ARG, "%s: seq_order_out needs k_new / v_new and kv_lens", fn);
  if (seq_order_out && batch > 4096)
    return fail(FD_ERR_TOO_LARGE, "%s: seq_order_out with batch %d > 4096 (use fd_schedule)", fn, batch);
  if (!append && !with_q) return fail(FD_ERR_INVALID_ARG, "%s: nothing to do (no k_new / v_new and no prep->q)", fn);
  const int D = p->head_dim;
  if (D != 64 && D != 128 && D != 256) return fail(FD_ERR_UNSUPPORTED, "%s: head_dim %d (64/128/256)", fn, D);
  if (v_dim(p) != D) return fail(FD_ERR_UNSUPPORTED, "%s: K and V head dims must be equal (%d, %d)", fn, D, v_dim(p));
  const int ssz = dtype_size(p->q_dtype);
  if (!ssz || p->q_dtype == FD_FP8_E4M3) return fail(FD_ERR_UNSUPPORTED, "%s: q_dtype %d", fn, p->q_dtype);
  const int src16 = 16 / ssz;
  if (p->q_heads <= 0 || p->kv_heads <= 0)
    return fail(FD_ERR_INVALID_ARG, "%s: q_heads %d, kv_heads %d", fn, p->q_heads, p->kv_heads);

  AppendArgs a;
  memset(&a, 0, sizeof(a));
  a.batch = batch; a.T = new_tokens; a.Hq = p->q_heads; a.Hkv = p->kv_heads; a.D = D;
  int kv_dtype = p->q_dtype;
  if (append) {
    if (!k_new || !v_new || !k_cache || !v_cache || !block_table || !kv_lens)
      return fail(FD_ERR_INVALID_ARG, "%s: NULL tensor pointer", fn);
    if (kv_lens_out == kv_lens) return fail(FD_ERR_INVALID_ARG, "%s: kv_lens_out must not be kv_lens", fn);
    if (p->page_size <= 0 || p->num_pages <= 0 || p->max_pages_per_seq <= 0)
      return fail(FD_ERR_INVALID_ARG, "%s: page_size/num_pages/max_pages_per_seq must be > 0", fn);
    if ((int64_t)p->num_pages * p->page_size >= (int64_t)1 << 31)
      return fail(FD_ERR_TOO_LARGE, "%s: pool of %lld token rows exceeds 2^31", fn,
                  (long long)p->num_pages * p->page_size);
    if ((int64_t)p->max_pages_per_seq * p->page_size >= (int64_t)1 << 31)
      return fail(FD_ERR_TOO_LARGE, "%s: block table capacity exceeds 2^31 tokens", fn);
    kv_dtype = p->kv_dtype;
    const int kvsz = dtype_size(kv_dtype);
    if (!kvsz) return fail(FD_ERR_UNSUPPORTED, "%s: kv_dtype %d", fn, kv_dtype);
    if (kv_dtype == FD_FP8_E4M3 && (!p->k_scale || !p->v_scale))
      return fail(FD_ERR_INVALID_ARG, "%s: fp8 KV cache needs k_scale and v_scale", fn);
    const int kv16 = 16 / kvsz;
    if (!aligned16(k_cache) || !aligned16(v_cache) || stride_k_tok % kv16 || stride_k_h % kv16 ||
        stride_v_tok % kv16 || stride_v_h % kv16)
      return fail(FD_ERR_ALIGNMENT, "%s: K/V cache rows must be 16-byte aligned (pointer and token/head strides)", fn);
    if (!aligned16(k_new) || !aligned16(v_new) || stride_kn_b % src16 || stride_kn_t % src16 || stride_kn_h % src16 ||
        stride_vn_b % src16 || stride_vn_t % src16 || stride_vn_h % src16)
      return fail(FD_ERR_ALIGNMENT, "%s: k_new / v_new rows must be 16-byte aligned (pointer and strides)", fn);
    if (stride_k_tok <= 0 || stride_v_tok <= 0) return fail(FD_ERR_INVALID_ARG, "%s: token stride out of range", fn);
    a.k_new = k_new; a.v_new = v_new; a.k_cache = k_cache; a.v_cache = v_cache;
    a.bt = block_table; a.kv_lens = kv_lens; a.kv_lens_out = kv_lens_out;
    if (seq_order_out && p->seq_order_items) {
      if (batch > 256) return fail(FD_ERR_TOO_LARGE, "%s: work-item order with batch %d > 256 (use fd_schedule_items)", fn, batch);
      if (int rc = range_plan(fn, p, &a.ranges)) return rc;
      a.items = seq_order_out;
    } else {
      a.seq_order = seq_order_out;
    }
    a.k_scale = p->k_scale; a.v_scale = p->v_scale;
    a.skn_b = stride_kn_b; a.skn_t = stride_kn_t; a.skn_h = stride_kn_h;
    a.svn_b = stride_vn_b; a.svn_t = stride_vn_t; a.svn_h = stride_vn_h;
    a.sk_t = stride_k_tok; a.sk_h = stride_k_h; a.sv_t = stride_v_tok; a.sv_h = stride_v_h;
    a.sbt = stride_table_bs; a.P = p->page_size; a.max_pages = p->max_pages_per_seq; a.num_pages = p->num_pages;
  }
  if (prep) {
    if (!prep->cos_sin && !prep->q_norm_weight && !prep->k_norm_weight)
      return fail(FD_ERR_INVALID_ARG, "%s: prep without cos_sin and without a norm weight", fn);
    if (prep->cos_sin) {
      if (!prep->position_ids) return fail(FD_ERR_INVALID_ARG, "%s: cos_sin needs position_ids", fn);
      if (prep->max_positions <= 0) return fail(FD_ERR_INVALID_ARG, "%s: prep->max_positions %d", fn, prep->max_positions);
      if (prep->position_dtype != 0 && prep->position_dtype != 1)
        return fail(FD_ERR_INVALID_ARG, "%s: prep->position_dtype %d (0: int32, 1: int64)", fn, prep->position_dtype);
      if (!aligned16(prep->cos_sin) || prep->stride_cos_sin % 4 || prep->stride_cos_sin < D)
        return fail(FD_ERR_ALIGNMENT, "%s: cos_sin rows must hold head_dim floats and be 16-byte aligned", fn);
      a.cos_sin = prep->cos_sin; a.s_cs = prep->stride_cos_sin; a.pos = prep->position_ids;
      a.pos_i64 = prep->position_dtype; a.max_pos = prep->max_positions;
      a.sp_b = prep->stride_pos_b; a.sp_t = prep->stride_pos_t;
    }
    if (!aligned16(prep->q_norm_weight) || !aligned16(prep->k_norm_weight))
      return fail(FD_ERR_ALIGNMENT, "%s: norm weights must be 16-byte aligned", fn);
    if (prep->q_norm_weight && !with_q) return fail(FD_ERR_INVALID_ARG, "%s: q_norm_weight without prep->q", fn);
    if (prep->k_norm_weight && !append) return fail(FD_ERR_INVALID_ARG, "%s: k_norm_weight without k_new", fn);
    a.qn_w = prep->q_norm_weight; a.kn_w = prep->k_norm_weight;
    a.qn_eps = prep->q_norm_eps; a.kn_eps = prep->k_norm_eps;
    if (with_q) {
      if (!prep->q_out) return fail(FD_ERR_INVALID_ARG, "%s: prep->q without prep->q_out", fn);
      if (!aligned16(prep->q) || !aligned16(prep->q_out) || prep->stride_q_b % src16 || prep->stride_q_t % src16 ||
          prep->stride_q_h % src16 || prep->stride_qo_b % src16 || prep->stride_qo_t % src16 ||
          prep->stride_qo_h % src16)
        return fail(FD_ERR_ALIGNMENT, "%s: q / q_out rows must be 16-byte aligned (pointer and strides)", fn);
      a.q = prep->q; a.q_out = prep->q_out;
      a.sq_b = prep->stride_q_b; a.sq_t = prep->stride_q_t; a.sq_h = prep->stride_q_h;
      a.sqo_b = prep->stride_qo_b; a.sqo_t = prep->stride_qo_t; a.sqo_h = prep->stride_qo_h;
    }
  }
  int rc = fd_launch_kv_append((hipStream_t)stream, a, p->q_dtype, kv_dtype);
  if (rc == FD_ERR_LAUNCH) return fail(rc, "%s: launch failed: %s", fn, hipGetErrorString(hipGetLastError()));
  if (rc == FD_ERR_TOO_LARGE) return fail(rc, "%s: batch * new_tokens * heads too large for one launch", fn);
  if (rc != FD_OK) return fail(rc, "%s: no kernel for q_dtype %d -> kv_dtype %d", fn, p->q_dtype, kv_dtype);
  return FD_OK;
}

int fd_schedule_items(void* stream, const int32_t* kv_lens, int32_t batch, int32_t* item_order, const fd_params* p) {
  const char* fn = "fd_schedule_items";
  if (!p) return fail(FD_ERR_INVALID_ARG, "%s: params is NULL", fn);
  if (!kv_lens || !item_order) return fail(FD_ERR_INVALID_ARG, "%s: NULL pointer", fn);
  if (batch < 0) return fail(FD_ERR_INVALID_ARG, "%s: batch = %d", fn, batch);
  if (batch == 0) return FD_OK;
  if (batch > kMaxItemBatch) return fail(FD_ERR_TOO_LARGE, "%s: batch %d > %d (use fd_schedule)", fn, batch, kMaxItemBatch);
  if (p->page_size <= 0 || p->max_pages_per_seq <= 0)
    return fail(FD_ERR_INVALID_ARG, "%s: page_size / max_pages_per_seq must be > 0", fn);
  RangePlan rp;
  if (int rc = range_plan(fn, p, &rp)) return rc;
  int rc = fd_launch_schedule_items((hipStream_t)stream, kv_lens, batch, (int64_t)p->max_pages_per_seq * p->page_size, rp,
                                    item_order);
  if (rc != FD_OK) return fail(rc, "%s: launch failed: %s", fn, hipGetErrorString(hipGetLastError()));
  return FD_OK;
}

int fd_schedule(void* stream, const int32_t* kv_lens, int32_t batch, int32_t* seq_order) {
  if (!kv_lens || !seq_order) return fail(FD_ERR_INVALID_ARG, "fd_schedule: NULL pointer");
  if (batch < 0) return fail(FD_ERR_INVALID_ARG, "fd_schedule: batch = %d", batch);
  if (batch == 0) return FD_OK;
  int rc = fd_launch_schedule((hipStream_t)stream, kv_lens, batch, seq_order);
  if (rc != FD_OK) return fail(rc, "fd_schedule: launch failed: %s", hipGetErrorString(hipGetLastError()));
  return FD_OK;
}

// ---------------------------------------------------------------------------------------------------------------
// The launch policy of a decode step whose partials the caller does not see (fd_plan_decode / fd_decode_planned).

namespace {

constexpr int kDefaultSplits = 32;        // flash_decode.py:779
constexpr int kPlannedSplitAlign = 64;    // tokens: the largest tile of the split kernels
constexpr int kMaxAutoSplits = 256;       // upper bound of the library's own choice
constexpr int64_t kPartials16BitFromBytes = 4 << 20;   // fp32 partials of a planned step from which on they take the output's 16-bit type
// Largest batch the step schedules as (sequence, range) items of its own accord; beyond it the item list costs more
// than it gains over the per-sequence order (256 ragged sequences of up to 8192 tokens: 650 against 640 us, 160 of
// them: 426 against 435 us)
constexpr int kItemsUpToBatch = 192;
// From this batch size on a step that was not asked to schedule ranks its sequences all the same (one launch of
// 3.5 us): a batch that large is ragged in practice and runs 4 - 15 % faster longest first (256 sequences of up to 2048
// tokens: 187 against 159 us, 72 of up to 8192 tokens 213 against 196 us); a uniform one loses the launch.
constexpr int kAutoOrderFromBatch = 64;
constexpr int kAutoOrderMinCapacity = 1024;   // ... unless no sequence can be longer than a range
constexpr int kMaxSeqOrderBatch = 4096;       // sequences fd_schedule ranks for a step
constexpr int kAppendOrderFromBatch = 16;     // an order that costs no launch (the append computes it) pays earlier

int64_t align256(int64_t n) { return (n + 255) & ~(int64_t)255; }

// Upper bound of the split count when the partials stay inside the library.  The caller's count is a hint there, not a
// limit -- the result does not depend on it, and the reference's 32 were chosen for contexts of a few thousand tokens:
// a single sequence of 131072 tokens on 8 KV heads runs 5 % faster with 64.
int split_bound(int hint, int64_t tokens) {
  int64_t own = tokens / 512;
  if (own > kMaxAutoSplits) own = kMaxAutoSplits;
  if (own < kDefaultSplits) own = kDefaultSplits;
  return hint > own ? hint : (int)own;
}

struct StepPlan {
  fd_params p;          // the parameters fd_decode / fd_split_kv / fd_combine / fd_schedule_items run the step with
  int direct, order_kind;
  int64_t partial_bytes, lse_bytes, order_bytes, lse_off, order_off, total;
  int64_t so_b, so_h, so_s;   // element strides of the partials in the workspace
};

int plan_step(const char* fn, const fd_params* in, int32_t batch, int32_t num_extra, int32_t flags,
              bool caller_order, StepPlan* sp) {
  if (!in) return fail(FD_ERR_INVALID_ARG, "%s: params is NULL", fn);
  if (batch <= 0 || num_extra < 0) return fail(FD_ERR_INVALID_ARG, "%s: batch %d, num_extra %d", fn, batch, num_extra);
  if (in->q_heads <= 0 || in->kv_heads <= 0 || in->q_heads % in->kv_heads != 0 || in->page_size <= 0 ||
      in->max_pages_per_seq <= 0)
    return fail(FD_ERR_INVALID_ARG, "%s: q_heads %d, kv_heads %d, page_size %d, max_pages_per_seq %d", fn, in->q_heads,
                in->kv_heads, in->page_size, in->max_pages_per_seq);
  const int Dv = v_dim(in);
  if (Dv != 64 && Dv != 128 && Dv != 256) return fail(FD_ERR_UNSUPPORTED, "%s: v_head_dim %d (64/128/256)", fn, Dv);
  const bool exact = (flags & (FD_STEP_EXACT_SPLITS | FD_STEP_CALLER_PARTIALS)) != 0;
  const bool caller_partials = (flags & FD_STEP_CALLER_PARTIALS) != 0;
  const bool fused = (flags & FD_STEP_FUSED) != 0;
  StepPlan& r = *sp;
  memset(&r, 0, sizeof(r));
  r.p = *in;
  const int64_t capacity = (int64_t)in->max_pages_per_seq * in->page_size;
  // the host-side length hint: rounded up to 1024 tokens, so that a growing batch does not re-plan at every step
  int64_t hint = 0;
  if (in->max_kv_len > 0 && in->max_kv_len < capacity) {
    hint = ((int64_t)in->max_kv_len + 1023) / 1024 * 1024;
    if (hint >= capacity) hint = 0;
  }
  r.p.max_kv_len = (int32_t)hint;
  r.p.seq_order_items = caller_order ? in->seq_order_items : 0;
  if (!caller_order) r.p.seq_order_lens = nullptr;
  if (exact) {
    r.p.num_splits = in->num_splits > 0 ? in->num_splits : kDefaultSplits;
    r.p.split_adapt = 0;
    r.p.split_align = caller_partials ? 0 : kPlannedSplitAlign;
  } else {
    // nobody looks at the partials: the library chooses the split count.  The grid has num_splits slots per
    // sequence; a sequence uses as many as its own length asks for (split_adapt).
    r.p.num_splits = split_bound(in->num_splits, hint ? hint : capacity);
    r.p.split_adapt = 0;
    r.p.split_align = kPlannedSplitAlign;
    const int s = fd_plan_splits(&r.p, batch);
    if (s < 0) return s;
    const int k = fd_plan_min_splits(&r.p, batch);
    if (k < 0) return k;
    r.p.num_splits = s;
    r.p.split_adapt = k;
  }
  const int S = r.p.num_splits;
  const int64_t rows = (int64_t)batch * in->q_heads * S;
  r.direct = S == 1 && num_extra == 0 && !fused && !caller_partials && !(flags & FD_STEP_LSE_TWICE);
  // Element type of the partials (the LSEs are always fp32, in their own buffer).  Planned splits are few and long:
  // fp32, unless there are kPartials16BitFromBytes of them or more (many query heads per KV head, large batches).
  // Those, and the partials of a caller who insists on an exact count, take the output's precision when that is
  // 16-bit -- what the reference's intra-rank wrapper allocates (flash_decode.py:867-868; the plain one fp16 whatever
  // the inputs, :783-784): megabytes that the split kernel writes at its very end and the combine reads back.
  if (!caller_partials) {
    static const int64_t from_bytes = env_int("FD_PARTIALS_16BIT_FROM_BYTES") > 0 ? env_int("FD_PARTIALS_16BIT_FROM_BYTES")
                                                                                   : kPartials16BitFromBytes;
    const bool out16 = in->out_dtype == FD_F16 || in->out_dtype == FD_BF16;
    r.p.mid_dtype = !fused && out16 && (exact || rows * Dv * 4 >= from_bytes) ? in->out_dtype : FD_F32;
  }
  // The issue order the step computes itself.
  r.order_kind = FD_ORDER_NONE;
  if (!caller_order && !(flags & FD_STEP_NO_ORDER) && batch > 1) {
    const bool free_order = (flags & FD_STEP_ORDER_FROM_APPEND) && batch >= kAppendOrderFromBatch;
    const bool scheduled = (flags & FD_STEP_SCHEDULE) || free_order;
    const bool ranked = scheduled || (batch >= kAutoOrderFromBatch && capacity >= kAutoOrderMinCapacity);
    // (a step that ranks of its own accord takes the item list as well where it applies: over ragged batches of 72 ...
    // 160 sequences it ran 1 - 4 % ahead of the per-sequence order, on config 4 650 against 687 us)
    const bool items = ranked && S > 1 && !fused && batch <= kItemsUpToBatch;
    if (items) {
      r.order_kind = FD_ORDER_ITEMS;
      r.p.seq_order_items = 1;
    } else if (ranked && batch <= kMaxSeqOrderBatch) {
      r.order_kind = FD_ORDER_SEQUENCES;
    }
  }
  const int msz = dtype_size(r.p.mid_dtype);
  if (!msz || r.p.mid_dtype == FD_FP8_E4M3) return fail(FD_ERR_UNSUPPORTED, "%s: mid_dtype %d", fn, r.p.mid_dtype);
  r.so_s = caller_partials ? Dv + 1 : Dv;
  r.so_h = (int64_t)S * r.so_s;
  r.so_b = (int64_t)in->q_heads * r.so_h;
  r.partial_bytes = caller_partials ? 0 : rows * Dv * msz;
  r.lse_bytes = caller_partials ? 0 : rows * 4;
  r.order_bytes = r.order_kind == FD_ORDER_ITEMS ? 2 * (int64_t)batch * S * 4
                  : r.order_kind == FD_ORDER_SEQUENCES ? (int64_t)batch * 4 : 0;
  r.lse_off = align256(r.partial_bytes);
  r.order_off = r.lse_off + align256(r.lse_bytes);
  r.total = r.order_off + align256(r.order_bytes);
  return FD_OK;
}

}  // namespace

int fd_plan_decode(const fd_params* params, int32_t batch, int32_t num_extra, int32_t flags, fd_launch_plan* plan) {
  const char* fn = "fd_plan_decode";
  if (!plan) return fail(FD_ERR_INVALID_ARG, "%s: plan is NULL", fn);
  StepPlan sp;
  if (int rc = plan_step(fn, params, batch, num_extra, flags, false, &sp)) return rc;
  memset(plan, 0, sizeof(*plan));
  plan->num_splits = sp.p.num_splits;
  plan->split_adapt = sp.p.split_adapt;
  plan->split_align = sp.p.split_align;
  plan->mid_dtype = sp.p.mid_dtype;
  plan->direct = sp.direct;
  plan->order_kind = sp.order_kind;
  plan->partial_bytes = sp.partial_bytes;
  plan->lse_bytes = sp.lse_bytes;
  plan->order_bytes = sp.order_bytes;
  plan->workspace_bytes = sp.total;
  plan->max_kv_len = sp.p.max_kv_len;
  // The launch shape, for contiguous caches and a contiguous query; the pointers below are stand-ins that are
  // checked for alignment only.
  void* const fake = reinterpret_cast<void*>((uintptr_t)1 << 20);
  fd_params p = sp.p;
  float one = 1.f;   // stand-in for fp8 scales (checked for presence only)
  if (p.kv_dtype == FD_FP8_E4M3) {
    if (!p.k_scale) p.k_scale = &one;
    if (!p.v_scale) p.v_scale = &one;
  }
  if (p.num_pages <= 0) p.num_pages = p.max_pages_per_seq;
  const int Dv = v_dim(&p);
  const bool caller_partials = (flags & FD_STEP_CALLER_PARTIALS) != 0;
  const bool skip_empty = !sp.direct && p.split_adapt > 0 && p.split_adapt < p.num_splits &&
                          p.num_splits > kCombineSmallMax && !(flags & FD_STEP_FUSED);
  int32_t ticket = 0;
  FusedTail tail;
  tail.tickets = (flags & FD_STEP_FUSED) ? &ticket : nullptr;
  tail.num_extra = num_extra;
  bool fused = false;
  if (sp.direct) p.mid_dtype = p.out_dtype;
  LaunchShape ls;
  memset(&ls, 0, sizeof(ls));
  const int32_t* order = sp.order_kind != FD_ORDER_NONE ? (const int32_t*)fake : nullptr;
  int rc = split_impl(fn, nullptr, fake, fake, fake, fake, caller_partials ? nullptr : (float*)fake, 1.f,
                      (const int32_t*)fake, (const int32_t*)fake, batch, (int64_t)p.q_heads * p.head_dim, p.head_dim,
                      (int64_t)p.kv_heads * p.head_dim, p.head_dim, (int64_t)p.kv_heads * Dv, Dv,
                      sp.direct ? (int64_t)p.q_heads * Dv : sp.so_b, sp.direct ? Dv : sp.so_h, sp.direct ? 0 : sp.so_s,
                      p.max_pages_per_seq, order, &p, &tail, &fused, false, skip_empty, &ls);
  if (rc != FD_OK) return rc;
  plan->mfma = ls.mfma;
  plan->tile = ls.tile;
  plan->waves_per_head = ls.waves_per_head;
  plan->members = ls.members;
  plan->chunk = ls.chunk;
  plan->head_block = ls.head_block;
  plan->store_through = ls.store_through;
  for (int i = 0; i < 3; ++i) plan->grid[i] = (int32_t)ls.grid[i];
  return FD_OK;
}

int64_t fd_workspace_bytes(const fd_params* params, int32_t batch, int32_t num_extra, int32_t flags) {
  StepPlan sp;
  if (int rc = plan_step("fd_workspace_bytes", params, batch, num_extra, flags, false, &sp)) return rc;
  return sp.total;
}

int fd_decode_planned(void* stream, const fd_decode_args* a) {
  const char* fn = "fd_decode_planned";
  if (!a) return fail(FD_ERR_INVALID_ARG, "%s: args is NULL", fn);
  if (a->batch == 0) return FD_OK;
  if (a->flags & ~(FD_STEP_EXACT_SPLITS | FD_STEP_SCHEDULE | FD_STEP_NO_ORDER))
    return fail(FD_ERR_INVALID_ARG, "%s: flags 0x%x (FD_STEP_EXACT_SPLITS | FD_STEP_SCHEDULE | FD_STEP_NO_ORDER)", fn,
                a->flags);
  if (a->combine_mode != FD_COMBINE_SPLIT && a->combine_mode != FD_COMBINE_SPLIT_LSE)
    return fail(FD_ERR_INVALID_ARG, "%s: combine_mode %d (FD_COMBINE_SPLIT or FD_COMBINE_SPLIT_LSE)", fn, a->combine_mode);
  if (!a->kv_lens) return fail(FD_ERR_INVALID_ARG, "%s: NULL tensor pointer", fn);
  const int lse_twice = a->combine_mode == FD_COMBINE_SPLIT_LSE && a->lse_out ? FD_STEP_LSE_TWICE : 0;
  StepPlan sp;
  if (int rc = plan_step(fn, &a->params, a->batch, a->num_extra, a->flags | lse_twice, a->seq_order != nullptr, &sp))
    return rc;
  const bool need_ws = !sp.direct || sp.order_kind != FD_ORDER_NONE;
  char* ws = (char*)a->workspace;
  if (need_ws) {
    if (!ws || (reinterpret_cast<uintptr_t>(ws) & 255u) || a->workspace_bytes < sp.total)
      return fail(FD_ERR_INVALID_ARG,
                  "%s: the step needs a 256-byte aligned workspace of %lld bytes (fd_workspace_bytes), got %p with %lld",
                  fn, (long long)sp.total, (void*)ws, (long long)a->workspace_bytes);
  }
  const int32_t* order = a->seq_order;
  if (sp.order_kind == FD_ORDER_ITEMS) {
    int32_t* items = (int32_t*)(ws + sp.order_off);
    if (int rc = fd_schedule_items(stream, a->kv_lens, a->batch, items, &sp.p)) return rc;
    order = items;
  } else if (sp.order_kind == FD_ORDER_SEQUENCES) {
    int32_t* seq = (int32_t*)(ws + sp.order_off);
    if (int rc = fd_schedule(stream, a->kv_lens, a->batch, seq)) return rc;
    order = seq;
  }
  return fd_decode(stream, a->q, a->k_cache, a->v_cache, sp.direct ? nullptr : ws,
                   sp.direct ? nullptr : (float*)(ws + sp.lse_off), a->out, a->lse_out, a->sm_scale, a->block_table,
                   a->kv_lens, a->batch, a->stride_q_bs, a->stride_q_h, a->stride_k_tok, a->stride_k_h, a->stride_v_tok,
                   a->stride_v_h, sp.so_b, sp.so_h, sp.so_s, a->stride_table_bs, a->stride_obs, a->stride_oh, order,
                   a->combine_mode, a->extra_out, a->extra_lse, a->num_extra, nullptr, &sp.p);
}

}  // extern "C"
