// Write side of the paged KV cache: per-head RMS norm and rotary embedding of the new tokens' Q and
// K, and the append of K / V into the page pool (with conversion to the cache's dtype, fp8-e4m3
// quantisation included).  One launch covers all of it.
//
// A thread owns 8 consecutive elements of the first half of one head row and the matching 8
// of the second half (the pair the rotation mixes), so every access is 128 bits wide for
// 16-bit data and a row of D elements takes D/16 threads.
#include "fd_common.h"

namespace {

struct Fp8 {};   // tag: OCP e4m3fn bit patterns, one byte each

template <typename T> struct ElemBytes { static constexpr int v = sizeof(T); };
template <> struct ElemBytes<Fp8> { static constexpr int v = 1; };

// STREAM: the data is read once (activations) -- non-temporal; otherwise (norm weights, shared by every row) cached.
template <typename T, bool STREAM = true>
__device__ __forceinline__ void load8(const void* base, int64_t idx, float* x) {
  if constexpr (sizeof(T) == 4) {
    const f32x4* p = (const f32x4*)((const float*)base + idx);
    const f32x4 a = STREAM ? __builtin_nontemporal_load(p) : p[0];
    const f32x4 b = STREAM ? __builtin_nontemporal_load(p + 1) : p[1];
#pragma unroll
    for (int i = 0; i < 4; ++i) { x[i] = a[i]; x[4 + i] = b[i]; }
  } else {
    typedef T vec8 __attribute__((ext_vector_type(8)));
    const vec8* p = (const vec8*)((const T*)base + idx);
    const vec8 v = STREAM ? __builtin_nontemporal_load(p) : *p;
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = (float)v[i];
  }
}

// Rounds to T (round to nearest even) and back: what a store to a T tensor followed by a load does.
template <typename T>
__device__ __forceinline__ float round_through(float x) {
  if constexpr (sizeof(T) == 4) return x;
  else return (float)(T)x;
}

// q = clamp(x / scale, +-448) rounded to e4m3fn (nearest even); 448 is the largest finite e4m3fn.
__device__ __forceinline__ uint32_t quant2_fp8(float a, float b, float scale, uint32_t old, bool hi) {
  float qa = a / scale, qb = b / scale;
  qa = fminf(fmaxf(qa, -448.f), 448.f);
  qb = fminf(fmaxf(qb, -448.f), 448.f);
  return hi ? (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(qa, qb, (int)old, true)
            : (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(qa, qb, (int)old, false);
}

template <typename T>
__device__ __forceinline__ void store8(void* base, int64_t idx, const float* x, float scale) {
  if constexpr (sizeof(T) == 4) {
    f32x4* p = (f32x4*)((float*)base + idx);
    f32x4 a, b;
#pragma unroll
    for (int i = 0; i < 4; ++i) { a[i] = x[i]; b[i] = x[4 + i]; }
    __builtin_nontemporal_store(a, p);
    __builtin_nontemporal_store(b, p + 1);
  } else if constexpr (sizeof(T) == 2) {
    typedef T vec8 __attribute__((ext_vector_type(8)));
    vec8 v;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (T)x[i];
    __builtin_nontemporal_store(v, (vec8*)((T*)base + idx));
  } else {
    u32x2 w;
    uint32_t lo = 0, hi = 0;
    lo = quant2_fp8(x[0], x[1], scale, lo, false);
    lo = quant2_fp8(x[2], x[3], scale, lo, true);
    hi = quant2_fp8(x[4], x[5], scale, hi, false);
    hi = quant2_fp8(x[6], x[7], scale, hi, true);
    w[0] = lo; w[1] = hi;
    __builtin_nontemporal_store(w, (u32x2*)((uint8_t*)base + idx));
  }
}

// out1 = x1*cos - x2*sin, out2 = x2*cos + x1*sin, every product and sum rounded on its own
// (no fused multiply-add), then rounded to the activation dtype as the stand-alone rotary
// kernel's store would.
template <typename SRC>
__device__ __forceinline__ void rotate8(float* x1, float* x2, const float* cs_row, int e0, int half) {
#pragma clang fp contract(off)
  const f32x4* pc = (const f32x4*)(cs_row + e0);
  const f32x4* ps = (const f32x4*)(cs_row + half + e0);
  const f32x4 c0 = pc[0], c1 = pc[1], s0 = ps[0], s1 = ps[1];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float c = i < 4 ? c0[i] : c1[i - 4];
    const float s = i < 4 ? s0[i] : s1[i - 4];
    const float a = x1[i], b = x2[i];
    const float ac = a * c, bs = b * s, bc = b * c, as = a * s;
    x1[i] = round_through<SRC>(ac - bs);
    x2[i] = round_through<SRC>(bc + as);
  }
}

// RMS norm of one head row held by `cpr` consecutive lanes (8 + 8 elements each):
// y = (x * rsqrt(mean(x^2) + eps)) * w in fp32, rounded to the activation dtype.
template <typename SRC>
__device__ __forceinline__ void rms_norm_row(float* x1, float* x2, const void* w, float eps, int e0, int half,
                                             int cpr) {
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) ss += x1[i] * x1[i] + x2[i] * x2[i];
  for (int off = 1; off < cpr; off <<= 1) ss += __shfl_xor(ss, off);   // the row's lanes are aligned to cpr
  const float rstd = 1.0f / sqrtf(ss / (float)(2 * half) + eps);
  float w1[8], w2[8];
  load8<SRC, false>(w, e0, w1);
  load8<SRC, false>(w, half + e0, w2);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    x1[i] = round_through<SRC>(x1[i] * rstd * w1[i]);
    x2[i] = round_through<SRC>(x2[i] * rstd * w2[i]);
  }
}

template <typename SRC, typename DST>
__global__ __launch_bounds__(256) void fd_kv_append_kernel(const AppendArgs a) {
  const int cpr = a.D >> 4;                     // threads per head row
  const int half = a.D >> 1;
  const int hq = a.q ? a.Hq : 0;
  const int hkv = a.k_new ? a.Hkv : 0;
  const int heads = hq + 2 * hkv;               // rows per (sequence, token): K heads, V heads, Q heads
  if ((int)blockIdx.x >= a.data_blocks) {
    // Trailing workgroups: issue order for the decode that follows (same ranking as the stand-alone
    // schedulers), so that it costs no launch of its own.
    const int64_t cap = (int64_t)a.max_pages * a.P;
    auto grown = [&](int b) {
      int64_t len = a.kv_lens[b];
      len = (len < 0 ? 0 : len) + a.T;
      return len > cap ? cap : len;
    };
    if (a.items) {   // one workgroup: (sequence, range) items, batch <= 256
      __shared__ uint64_t s_key[256];
      __shared__ int32_t s_n[256];
      fd_schedule_items_block(threadIdx.x, a.batch, [&](int b) { return (int)grown(b); }, a.ranges, a.items, s_key,
                              s_n);
      return;
    }
    // per-sequence order: grown length descending, ties by index
    __shared__ __align__(16) int32_t s_len[kRankChunk];
    const int gid = ((int)blockIdx.x - a.data_blocks) * blockDim.x + threadIdx.x;
    int mine;
    const int rank = fd_rank_sequence(gid, a.batch, a.rank_shift, [&](int b) { return (int)grown(b); }, s_len, &mine);
    const int i = gid >> a.rank_shift;
    if ((gid & ((1 << a.rank_shift) - 1)) == 0 && i < a.batch) {
      a.seq_order[rank] = i;
      a.seq_order[a.batch + rank] = mine;   // the lengths in issue order, for the decode's prologue
    }
    return;
  }
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t row = g / cpr;
  if (row >= (int64_t)a.batch * a.T * heads) return;
  const int c = (int)(g - row * cpr);
  const int64_t bt_idx = row / heads;
  const int hh = (int)(row - bt_idx * heads);
  const int b = (int)(bt_idx / a.T);
  const int t = (int)(bt_idx - (int64_t)b * a.T);
  const int e0 = c * 8;

  const float* cs_row = nullptr;
  if (a.cos_sin) {
    int64_t pos = a.pos_i64 ? ((const int64_t*)a.pos)[b * a.sp_b + t * a.sp_t]
                            : (int64_t)((const int32_t*)a.pos)[b * a.sp_b + t * a.sp_t];
    pos = pos < 0 ? 0 : (pos >= a.max_pos ? a.max_pos - 1 : pos);
    cs_row = a.cos_sin + pos * a.s_cs;
  }

  float x1[8], x2[8];
  if (hh >= 2 * hkv) {                          // a query head: rotate into q_out
    const int h = hh - 2 * hkv;
    const int64_t src = b * a.sq_b + t * a.sq_t + h * a.sq_h;
    load8<SRC>(a.q, src + e0, x1);
    load8<SRC>(a.q, src + half + e0, x2);
    if (a.qn_w) rms_norm_row<SRC>(x1, x2, a.qn_w, a.qn_eps, e0, half, cpr);
    if (cs_row) rotate8<SRC>(x1, x2, cs_row, e0, half);
    const int64_t dst = b * a.sqo_b + t * a.sqo_t + h * a.sqo_h;
    store8<SRC>(a.q_out, dst + e0, x1, 1.f);
    store8<SRC>(a.q_out, dst + half + e0, x2, 1.f);
    return;
  }

  const bool is_v = hh >= hkv;
  const int h = is_v ? hh - hkv : hh;
  int64_t len = a.kv_lens[b];
  const int64_t cap = (int64_t)a.max_pages * a.P;
  len = len < 0 ? 0 : len;
  if (hh == 0 && c == 0 && t == 0 && a.kv_lens_out) {
    const int64_t grown = len + a.T;
    a.kv_lens_out[b] = (int32_t)(grown > cap ? cap : grown);
  }
  const int64_t n = len + t;
  if (n >= cap) return;                         // no page for this token: nothing is written
  const int pidx = (int)(n / a.P);
  int page = a.bt[b * a.sbt + pidx];
  page = min(max(page, 0), a.num_pages - 1);
  const int64_t trow = (int64_t)page * a.P + (n - (int64_t)pidx * a.P);

  if (is_v) {
    const int64_t src = b * a.svn_b + t * a.svn_t + h * a.svn_h;
    load8<SRC>(a.v_new, src + e0, x1);
    load8<SRC>(a.v_new, src + half + e0, x2);
    const float scale = ElemBytes<DST>::v == 1 ? a.v_scale[h] : 1.f;
    const int64_t dst = trow * a.sv_t + h * a.sv_h;
    store8<DST>(a.v_cache, dst + e0, x1, scale);
    store8<DST>(a.v_cache, dst + half + e0, x2, scale);
  } else {
    const int64_t src = b * a.skn_b + t * a.skn_t + h * a.skn_h;
    load8<SRC>(a.k_new, src + e0, x1);
    load8<SRC>(a.k_new, src + half + e0, x2);
    if (a.kn_w) rms_norm_row<SRC>(x1, x2, a.kn_w, a.kn_eps, e0, half, cpr);
    if (cs_row) rotate8<SRC>(x1, x2, cs_row, e0, half);
    const float scale = ElemBytes<DST>::v == 1 ? a.k_scale[h] : 1.f;
    const int64_t dst = trow * a.sk_t + h * a.sk_h;
    store8<DST>(a.k_cache, dst + e0, x1, scale);
    store8<DST>(a.k_cache, dst + half + e0, x2, scale);
  }
}

template <typename SRC>
int launch_src(hipStream_t stream, const AppendArgs& a, int kv_dtype, dim3 grid) {
  switch (kv_dtype) {
    case FD_F32: hipLaunchKernelGGL((fd_kv_append_kernel<SRC, float>), grid, dim3(256), 0, stream, a); break;
    case FD_F16: hipLaunchKernelGGL((fd_kv_append_kernel<SRC, _Float16>), grid, dim3(256), 0, stream, a); break;
    case FD_BF16: hipLaunchKernelGGL((fd_kv_append_kernel<SRC, __bf16>), grid, dim3(256), 0, stream, a); break;
    case FD_FP8_E4M3: hipLaunchKernelGGL((fd_kv_append_kernel<SRC, Fp8>), grid, dim3(256), 0, stream, a); break;
    default: return FD_ERR_UNSUPPORTED;
  }
  return hipGetLastError() == hipSuccess ? FD_OK : FD_ERR_LAUNCH;
}

}  // namespace

int fd_launch_kv_append(hipStream_t stream, const AppendArgs& args, int src_dtype, int kv_dtype) {
  AppendArgs a = args;
  const int heads = (a.q ? a.Hq : 0) + (a.k_new ? 2 * a.Hkv : 0);
  const int64_t threads = (int64_t)a.batch * a.T * heads * (a.D >> 4);
  if (threads == 0) return FD_OK;
  int64_t blocks = (threads + 255) / 256;
  if (blocks > 0x7fff0000LL) return FD_ERR_TOO_LARGE;
  a.data_blocks = (int32_t)blocks;
  if (a.items) {
    if (a.batch > 256) return FD_ERR_TOO_LARGE;
    blocks += 1;
  } else if (a.seq_order) {
    a.rank_shift = fd_rank_shift(a.batch);
    blocks += (((int64_t)a.batch << a.rank_shift) + 255) / 256;
  }
  const dim3 grid((unsigned)blocks);
  switch (src_dtype) {
    case FD_F32: return launch_src<float>(stream, a, kv_dtype, grid);
    case FD_F16: return launch_src<_Float16>(stream, a, kv_dtype, grid);
    case FD_BF16: return launch_src<__bf16>(stream, a, kv_dtype, grid);
    default: return FD_ERR_UNSUPPORTED;
  }
}
