// Shared device-side types and helpers for the gfx950 flash-decode kernels.
//
// Everything here is written for CDNA4 wave64: "lane" is 0..63, a "row" of a
// wave is 16 consecutive lanes (the granularity of the 16x16 MFMA operand
// layouts), cross-lane traffic uses ds_bpermute via __shfl*.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/flash_decode.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
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
  const float* k_scale;
  const float* v_scale;
  int64_t sq_b, sq_h, sk_t, sk_h, sv_t, sv_h, so_b, so_h, so_s, sbt;
  float sm_scale, soft_cap;
  int32_t batch, Hq, Hkv, G, S, P, log2P, max_pages, num_pages;
  int32_t q_dtype, mid_dtype;
  int32_t nhb;      // head blocks per KV head
  int32_t hbsz;     // query heads per head block
  int32_t vec_out;  // 1: every out row start is 16-byte aligned (128-bit stores allowed)
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
};

// ---------------------------------------------------------------- scalar conversions

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t lo16) { return __uint_as_float(lo16 << 16); }

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

__device__ __forceinline__ float fd_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fd_log2(float x) { return __builtin_amdgcn_logf(x); }

// soft_cap * tanh(x / soft_cap), tanh(y) = 1 - 2 / (1 + e^{2y})
__device__ __forceinline__ float fd_softcap(float x, float cap, float inv_cap) {
  float e = fd_exp2(2.0f * FD_LOG2E * x * inv_cap);
  return cap * (1.0f - 2.0f / (1.0f + e));
}

// Orders LDS accesses of one wave: lanes of a wave exchange data through LDS
// without a workgroup barrier (the LDS queue of a wave is in order); this only
// stops the compiler from moving accesses across the point.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Decodes blockIdx.x into (sequence, split, kv head, head block) and the split's
// token range.  Work items are ordered sequence-rank major, then split, then KV
// head, so workgroups that are dispatched together read neighbouring 16-byte
// chunks of the same pages.
struct WorkItem {
  int b, s, kvh, hb, start, end;
};

__device__ __forceinline__ WorkItem decode_work_item(const SplitArgs& a) {
  WorkItem w;
  int bid = blockIdx.x;
  w.hb = bid % a.nhb;
  bid /= a.nhb;
  w.kvh = bid % a.Hkv;
  bid /= a.Hkv;
  w.s = bid % a.S;
  int r = bid / a.S;
  int b = a.order ? a.order[r] : r;
  w.b = min(max(b, 0), a.batch - 1);
  int64_t cap = (int64_t)a.max_pages * a.P;
  int64_t len = a.kv_lens[w.b];
  len = len < 0 ? 0 : (len > cap ? cap : len);
  int kv_len = (int)len;
  int per = (kv_len + a.S - 1) / a.S;  // ceil(kv_len / S)
  int64_t st = (int64_t)per * w.s;
  w.start = st > kv_len ? kv_len : (int)st;
  int64_t en = st + per;
  w.end = en > kv_len ? kv_len : (int)en;
  return w;
}

// Flat cache row of logical token n of sequence b: page*P + n%P, with the page id
// clamped into the pool so that a corrupt table entry cannot fault the GPU.
__device__ __forceinline__ int token_row(const SplitArgs& a, const int32_t* bt_row, int n) {
  int pidx = a.log2P >= 0 ? (n >> a.log2P) : (n / a.P);
  int page = bt_row[pidx];
  page = min(max(page, 0), a.num_pages - 1);
  return page * a.P + (n - pidx * a.P);
}

// Merges the per-wave partial states of a workgroup and stores one normalised
// partial (out, lse) per query head.
//
// LDS layout of partial w (floats): part[w*stride + h*D + d] = un-normalised
// accumulator, part[w*stride + HB*D + h] = running max (base-2 domain),
// part[w*stride + HB*D + HB + h] = running sum.  Called by every thread of the
// workgroup after a __syncthreads().
template <int HB, int D>
__device__ __forceinline__ void cta_merge_store(const SplitArgs& a, const float* part, int stride, int nparts,
                                                const WorkItem& w, int head0, int nheads, float out_scale) {
  const int tid = threadIdx.x;
  const int nthreads = blockDim.x;
  constexpr int D4 = D / 4;
  for (int e = tid; e < nheads * D4; e += nthreads) {
    const int h = e / D4;
    const int d = (e - h * D4) * 4;
    float M = -INFINITY;
    for (int p = 0; p < nparts; ++p) M = fmaxf(M, part[p * stride + HB * D + h]);
    float L = 0.f;
    f32x4 o = {0.f, 0.f, 0.f, 0.f};
    if (M > -INFINITY) {
      for (int p = 0; p < nparts; ++p) {
        const float* pp = part + p * stride;
        float wgt = fd_exp2(pp[HB * D + h] - M);  // exp2(-inf) = 0 for idle waves
        L += pp[HB * D + HB + h] * wgt;
        f32x4 x = *(const f32x4*)(pp + h * D + d);
        o += x * wgt;
      }
    }
    float inv = L > 0.f ? out_scale / L : 0.f;
    o *= inv;
    const int head = head0 + h;
    const int64_t off = (int64_t)w.b * a.so_b + (int64_t)head * a.so_h + (int64_t)w.s * a.so_s + d;
    if (a.mid_dtype == FD_F32 && a.vec_out) {
      *(f32x4*)((float*)a.out + off) = o;
    } else {
      for (int i = 0; i < 4; ++i) store_from_f32(a.out, off + i, a.mid_dtype, o[i]);
    }
    if (d == 0) {
      float lse = L > 0.f ? (M + fd_log2(L)) * FD_LN2 : -INFINITY;
      if (a.lse) {
        a.lse[((int64_t)w.b * a.Hq + head) * a.S + w.s] = lse;
      } else {
        store_from_f32(a.out, off + D, a.mid_dtype, lse);
      }
    }
  }
}

// Launchers implemented in the kernel translation units (host side).
int fd_launch_split_mfma(hipStream_t stream, const SplitArgs& a, int kv_dtype, int waves, bool soft_cap);
int fd_launch_split_valu(hipStream_t stream, const SplitArgs& a, int kv_dtype, int head_dim, int waves);
int fd_launch_combine(hipStream_t stream, const CombineArgs& a);
int fd_launch_schedule(hipStream_t stream, const int32_t* kv_lens, int batch, int32_t* order);
