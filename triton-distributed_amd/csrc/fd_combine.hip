// LSE-weighted combine of split / rank partials, and the sequence scheduler (gfx950).
//
// fd_combine_kernel replaces the reference's three combine kernels
// (python/triton_dist/kernels/nvidia/flash_decode.py:308-360 plain, :393-449
// intra-rank with merged LSE, :482-532 inter-rank).  The reference walks the
// partials sequentially with a running max; here one wave per (sequence, head)
// first reduces the LSEs (max, then sum of weights) and then accumulates
// sum_s w_s * O_s with all row loads independent of each other -- the same
// value, out = sum_s softmax(LSE)_s * O_s and LSE = logsumexp_s(LSE_s), with two
// dependent memory round trips instead of S.
#include "fd_common.h"

namespace {

constexpr int kMaxDPerLane = 4;  // head_dim <= 256

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) x = fmaxf(x, __shfl_xor(x, o));
  return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) x += __shfl_xor(x, o);
  return x;
}

__global__ void __launch_bounds__(64) fd_combine_kernel(const CombineArgs a) {
  const int lane = threadIdx.x;
  const int b = blockIdx.x / a.Hq;
  const int h = blockIdx.x - b * a.Hq;
  const int S = a.num_partials;
  const int NP = S + a.num_extra;
  const int D = a.D;
  const int64_t mid_base = (int64_t)b * a.s_mb + (int64_t)h * a.s_mh;

  int kv_len = 0, per = 0;
  if (a.mode != FD_COMBINE_RANK) {
    kv_len = max(a.seqlens[b], 0);
    per = (kv_len + S - 1) / S;
  }
  auto partial_valid = [&](int s) -> bool {
    if (s >= S) return true;                                   // extra partials are always valid
    if (a.mode == FD_COMBINE_RANK) return a.seqlens[(int64_t)s * a.batch + b] > 0;
    int64_t st = (int64_t)per * s;                             // split range non-empty
    return st < kv_len;
  };
  auto partial_lse = [&](int s) -> float {
    if (s >= S) return a.extra_lse[((int64_t)(s - S) * a.batch + b) * a.Hq + h];
    if (a.mid_lse) return a.mid_lse[((int64_t)b * a.Hq + h) * S + s];
    return load_as_f32(a.mid_o, mid_base + (int64_t)s * a.s_ms + D, a.mid_dtype);
  };

  // pass 1: M = max LSE over valid partials
  float M = -INFINITY;
  for (int s0 = 0; s0 < NP; s0 += 64) {
    const int s = s0 + lane;
    float L = -INFINITY;
    if (s < NP && partial_valid(s)) L = partial_lse(s);
    M = fmaxf(M, L);
  }
  M = wave_max(M);

  float acc[kMaxDPerLane] = {0.f, 0.f, 0.f, 0.f};
  float Lsum = 0.f;
  if (M > -INFINITY) {
    for (int s0 = 0; s0 < NP; s0 += 64) {
      const int s = s0 + lane;
      float wgt = 0.f;
      if (s < NP && partial_valid(s)) wgt = __expf(partial_lse(s) - M);
      Lsum += wgt;
      const int cnt = min(64, NP - s0);
      for (int j = 0; j < cnt; ++j) {
        const float wj = __shfl(wgt, j);
        if (wj == 0.f) continue;  // wave-uniform
        const int sj = s0 + j;
#pragma unroll
        for (int k = 0; k < kMaxDPerLane; ++k) {
          const int d = lane + 64 * k;
          if (d < D) {
            float o;
            if (sj < S) {
              o = load_as_f32(a.mid_o, mid_base + (int64_t)sj * a.s_ms + d, a.mid_dtype);
            } else {
              o = load_as_f32(a.extra_out, (((int64_t)(sj - S) * a.batch + b) * a.Hq + h) * D + d, a.out_dtype);
            }
            acc[k] = fmaf(wj, o, acc[k]);
          }
        }
      }
    }
    Lsum = wave_sum(Lsum);
  }
  const float inv = Lsum > 0.f ? 1.0f / Lsum : 0.f;
  const int64_t out_base = (int64_t)b * a.s_ob + (int64_t)h * a.s_oh;
#pragma unroll
  for (int k = 0; k < kMaxDPerLane; ++k) {
    const int d = lane + 64 * k;
    if (d < D) store_from_f32(a.out, out_base + d, a.out_dtype, acc[k] * inv);
  }
  if (lane == 0) {
    const float lse = Lsum > 0.f ? M + __logf(Lsum) : -INFINITY;
    if (a.mode == FD_COMBINE_SPLIT_LSE) store_from_f32(a.out, out_base + D, a.out_dtype, lse);
    if (a.lse_out) a.lse_out[(int64_t)b * a.Hq + h] = lse;
  }
}

// order[rank] = sequence index, sequences ranked by kv_len descending, ties by index.
__global__ void __launch_bounds__(256) fd_schedule_kernel(const int32_t* __restrict__ kv_lens, int batch,
                                                          int32_t* __restrict__ order) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= batch) return;
  const int mine = kv_lens[i];
  int rank = 0;
  for (int j = 0; j < batch; ++j) {
    const int other = kv_lens[j];
    rank += (other > mine) || (other == mine && j < i);
  }
  order[rank] = i;
}

}  // namespace

int fd_launch_combine(hipStream_t stream, const CombineArgs& a) {
  const unsigned grid = (unsigned)a.batch * a.Hq;
  hipLaunchKernelGGL(fd_combine_kernel, dim3(grid), dim3(64), 0, stream, a);
  return hipGetLastError() == hipSuccess ? FD_OK : FD_ERR_LAUNCH;
}

int fd_launch_schedule(hipStream_t stream, const int32_t* kv_lens, int batch, int32_t* order) {
  const unsigned grid = (unsigned)((batch + 255) / 256);
  hipLaunchKernelGGL(fd_schedule_kernel, dim3(grid), dim3(256), 0, stream, kv_lens, batch, order);
  return hipGetLastError() == hipSuccess ? FD_OK : FD_ERR_LAUNCH;
}
