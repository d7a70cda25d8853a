// MFMA wrappers shared by the 16-bit and the fp8 split kernels (gfx950).
//
// v_mfma_f32_16x16x32_{bf16,f16}: D[16x16] += A[16x32] * B[32x16].  Lane l = 16*g + r supplies
// A[row r][k = 8g..8g+7] and B[k = 8g..8g+7][col r] (8 packed 16-bit values = 4 dwords each) and
// receives D[row 4g+i][col r], i = 0..3.
#pragma once

#include "fd_common.h"

template <typename T>
struct Mma;
template <>
struct Mma<__bf16> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
  }
  // two OCP e4m3 bytes (low or high half of w) -> two packed bf16, exact
  static __device__ __forceinline__ uint32_t from_fp8(uint32_t w, bool hi) {
    return hi ? __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true))
              : __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false));
  }
};
template <>
struct Mma<_Float16> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                  0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
  }
  static __device__ __forceinline__ uint32_t from_fp8(uint32_t w, bool hi) {
    return hi ? __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true))
              : __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false));
  }
};

// One online-softmax step of the "lane c = head c" layout shared by the MFMA split kernels.  x[0..N) are this lane's
// scores of head c for N tokens of the tile, in the base-2 domain, masked tokens = -inf; the four wave rows hold
// different tokens of the same head.  Updates the reference point m (identical in the four rows; at most 8 below the
// running maximum) and the lane's share l of the running sum, replaces x by the weights 2^(x - m), and returns the
// factor the accumulators of head c have to be multiplied by; moved = some lane's reference point moved
// (wave-uniform), i.e. whether that rescale is needed at all.  Every tile holds at least one valid token, so the
// new reference point is finite.
template <int N>
__device__ __forceinline__ float fd_softmax_step(float (&x)[N], float& m, float& l, bool& moved) {
  float t[N];   // pairwise tree: a short dependency chain
#pragma unroll
  for (int i = 0; i < N; ++i) t[i] = x[i];
#pragma unroll
  for (int stride = 1; stride < N; stride *= 2) {
#pragma unroll
    for (int i = 0; i + stride < N; i += 2 * stride) t[i] = fmaxf(t[i], t[i + stride]);
  }
  float mx = t[0];
  mx = fmaxf(mx, __shfl_xor(mx, 16));
  mx = fmaxf(mx, __shfl_xor(mx, 32));
  // The reference point only moves when the maximum has grown by more than kLazyMax (base-2): until then the
  // probabilities are taken relative to the older, smaller reference (they stay below 2^kLazyMax, exact powers of two
  // away from what the true maximum would give), and the accumulators need no rescale.  m is -inf before the first tile.
  constexpr float kLazyMax = 8.0f;
  const float m_top = fmaxf(m, mx);
  const float m_new = m_top - m > kLazyMax ? m_top : m;
  const float alpha = fd_exp2(m - m_new);
  float psum = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    x[i] = fd_exp2(x[i] - m_new);
    psum += x[i];
  }
  l = l * alpha + psum;
  moved = __any(m_new > m);
  m = m_new;
  return alpha;
}
