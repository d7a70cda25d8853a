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

