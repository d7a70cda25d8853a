// Split-KV GQA paged decode on MFMA with an fp8-e4m3 (OCP) KV cache (gfx950), head_dim 256.
//
// A token row is 256 bytes -- the byte geometry of the 16-bit kernel's 128-dim rows
// (fd_split_mfma.hip) -- so tiles and loads are those: 32-token tiles, 8 + 8
// global_load_dwordx4 per lane, load i fetching for every wave row g the whole row of token
// tau(g, i) = 4g + (i & 3) + 16 (i >> 2); lane (g, c) holds the 16 bytes = dims 16c .. 16c+15
// of its 8 tokens.  The bytes are dequantised in registers with
// v_cvt_scalef32_pk_{bf16,f16}_fp8 (exact) on their way into the 16x16x32 MFMA:
//   * K: staged in LDS (row pitch 272 B), read back with ds_read_b64 as the A operand of
//     S^T = K . Q^T (lane (g, m) <- token m's bytes 32 ks + 8g .. +7, ks = 0..7).
//   * V: the lane's 8 tokens x 16 dims are converted and transposed with v_perm_b32, 8 dims at
//     a time, into the A operands of O^T[dim][head] += V^T . P^T; 16 accumulator blocks,
//     block j holding dims 16 (4g + i) + j.
// The per-KV-head K scale is folded into the softmax scale, the V scale multiplies a wave's
// finished accumulators once.
#include <type_traits>

#include "fd_common.h"
#include "fd_mma.h"

namespace {

constexpr int kD = 256;
constexpr int kTile = 32;         // tokens per tile
constexpr int kKRow = 272;        // LDS pitch of a staged K row in bytes (256 + 16 pad)
constexpr int kHB = 16;
constexpr int kWaveLds = (kHB * kD + 2 * kHB) * 4;   // 16512 B: the wave's partial result; the K tile (8704 B) fits
static_assert(kWaveLds >= kTile * kKRow, "K staging buffer must fit");

template <typename T, bool SOFTCAP>
__global__ void __launch_bounds__(512) fd_split_mfma_fp8_d256_kernel(const SplitArgs a) {
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 4;
  const int c = lane & 15;

  const WorkItem w = decode_work_item(a);
  if (w.skip) return;   // empty range, and the combine does not expect a partial from it
  const int ntok = w.end - w.start;
  const int ntiles = ntok > 0 ? (ntok + kTile - 1) / kTile : 0;
  const int tpw = div_uniform(ntiles + w.nsub - 1, w.nsub);
  const int t0 = w.sub * tpw;
  const int t1 = min(t0 + tpw, ntiles);

  const int head_in_group = w.hb * kHB + c;
  const bool head_ok = head_in_group < a.G;
  const int head = w.kvh * a.G + head_in_group;

  u32x4 qop[8];  // Q as the MFMA B operand: lane (g, c) holds Q[head c][32*ks + 8g .. +7]
  {
    const char* qp = (const char*)a.q + ((int64_t)w.b * a.sq_b + (int64_t)head * a.sq_h) * 2;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      u32x4 z = {0u, 0u, 0u, 0u};
      qop[ks] = head_ok ? *(const u32x4*)(qp + (32 * ks + 8 * g) * 2) : z;
    }
  }

  const int32_t* bt_row = a.bt + (int64_t)w.b * a.sbt;
  const char* kbase = (const char*)a.k + (int64_t)w.kvh * a.sk_h + c * 16;
  const char* vbase = (const char*)a.v + (int64_t)w.kvh * a.sv_h + c * 16;
  const int k_pitch = (int)a.sk_t;
  const int v_pitch = (int)a.sv_t;
  char* kb = smem + wave * kWaveLds;

  const float kq_scale = a.sm_scale * a.k_scale[w.kvh];  // K dequantisation folded into the softmax scale
  const float v_scale = a.v_scale[w.kvh];                // V dequantisation: once, on the finished accumulators
  const float scale2 = kq_scale * FD_LOG2E;
  const float inv_cap = SOFTCAP ? 1.0f / a.soft_cap : 0.f;

  auto tile_slot = [&](int t, int& slot) -> int { return fd_tile_slot<kTile>(a, w, bt_row, t, lane & 31, slot); };

  u32x4 kraw[8], vraw[8];
  int rows[8];
  auto fetch_rows = [&](int page, int slot) {
    const int rv = fd_flat_row(a, page, slot);
#pragma unroll
    for (int i = 0; i < 8; ++i) rows[i] = __shfl(rv, 4 * g + (i & 3) + 16 * (i >> 2));
  };
  auto issue_k = [&]() {
#pragma unroll
    for (int i = 0; i < 8; ++i) kraw[i] = load_stream_b128(kbase + (int64_t)rows[i] * k_pitch);
  };
  auto issue_v = [&]() {
#pragma unroll
    for (int i = 0; i < 8; ++i) vraw[i] = load_stream_b128(vbase + (int64_t)rows[i] * v_pitch);
  };

  float m = -INFINITY;
  float l = 0.f;
  f32x4 acc[16];  // acc[j][i] = O[head c][dim 16*(4g + i) + j]
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

  int pg_next = 0, slot_next = 0;

  auto tile = [&](int t, auto has_next_tag) {
    constexpr bool HAS_NEXT = decltype(has_next_tag)::value;
    // ---- K tile -> LDS, then request the next tile's K
    wave_lds_fence();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int tau = 4 * g + (i & 3) + 16 * (i >> 2);
      *(u32x4*)(kb + tau * kKRow + c * 16) = kraw[i];
    }
    wave_lds_fence();
    if constexpr (HAS_NEXT) {
      __builtin_amdgcn_sched_barrier(0);
      fetch_rows(pg_next, slot_next);
      issue_k();
      pg_next = tile_slot(min(t + 2, t1 - 1), slot_next);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- S^T = K . Q^T, two 16-token sub-tiles
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const u32x2 k0 = *(const u32x2*)(kb + c * kKRow + 32 * ks + 8 * g);
      const u32x2 k1 = *(const u32x2*)(kb + (16 + c) * kKRow + 32 * ks + 8 * g);
      const uint32_t a00 = k0[0], a01 = k0[1], a10 = k1[0], a11 = k1[1];
      u32x4 a0 = {Mma<T>::from_fp8(a00, false), Mma<T>::from_fp8(a00, true), Mma<T>::from_fp8(a01, false),
                  Mma<T>::from_fp8(a01, true)};
      u32x4 a1 = {Mma<T>::from_fp8(a10, false), Mma<T>::from_fp8(a10, true), Mma<T>::from_fp8(a11, false),
                  Mma<T>::from_fp8(a11, true)};
      s0 = Mma<T>::run(a0, qop[ks], s0);
      s1 = Mma<T>::run(a1, qop[ks], s1);
    }
    // ---- online softmax (head c, tokens tau(g, 0..7))
    float x[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[i] = s0[i];
      x[4 + i] = s1[i];
    }
    const int n0 = w.start + t * kTile;
    const bool full = n0 + kTile <= w.end;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float v = x[i];
      if (SOFTCAP) {
        v = fd_softcap(v * kq_scale, a.soft_cap, inv_cap) * FD_LOG2E;
      } else {
        v *= scale2;
      }
      x[i] = v;
    }
    if (!full) {   // only the last tile of a range has tokens to mask (wave-uniform branch)
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (n0 + 4 * g + (i & 3) + 16 * (i >> 2) >= w.end) x[i] = -INFINITY;
    }
    bool moved;
    const float alpha = fd_softmax_step(x, m, l, moved);
    if (moved) {
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[j] *= alpha;
    }
    u32x4 pop;  // P^T as the B operand: element e <-> token tau(g, e)
#pragma unroll
    for (int e = 0; e < 4; ++e) pop[e] = Mma<T>::pack(x[2 * e], x[2 * e + 1]);

    // ---- V: dequantise and transpose 8 tokens x 8 dims at a time, O^T += V^T . P^T
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      uint32_t cv[8][4];  // cv[e][jp] = dims (8hh + 2jp, 8hh + 2jp + 1) of token e as packed 16-bit
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t v0 = vraw[e][2 * hh], v1 = vraw[e][2 * hh + 1];
        cv[e][0] = Mma<T>::from_fp8(v0, false);
        cv[e][1] = Mma<T>::from_fp8(v0, true);
        cv[e][2] = Mma<T>::from_fp8(v1, false);
        cv[e][3] = Mma<T>::from_fp8(v1, true);
      }
      if constexpr (HAS_NEXT) {
        if (hh == 1) {   // every byte of this tile's V has been converted: refill the registers in place
          __builtin_amdgcn_sched_barrier(0);
          issue_v();
          __builtin_amdgcn_sched_barrier(0);
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
        u32x4 vop;
#pragma unroll
        for (int q2 = 0; q2 < 4; ++q2) vop[q2] = __builtin_amdgcn_perm(cv[2 * q2 + 1][j >> 1], cv[2 * q2][j >> 1], sel);
        acc[8 * hh + j] = Mma<T>::run(vop, pop, acc[8 * hh + j]);
      }
    }
  };

  if (t0 < t1) {
    int slot0;
    const int pg0 = tile_slot(t0, slot0);
    pg_next = tile_slot(min(t0 + 1, t1 - 1), slot_next);
    __builtin_amdgcn_sched_barrier(0);
    fetch_rows(pg0, slot0);
    issue_k();
    issue_v();
    __builtin_amdgcn_sched_barrier(0);
    for (int t = t0; t < t1 - 1; ++t) tile(t, std::true_type{});
    tile(t1 - 1, std::false_type{});
  }

  // ---- wave result -> LDS, then workgroup merge
  l += __shfl_xor(l, 16);
  l += __shfl_xor(l, 32);
  wave_lds_fence();
  float* part = (float*)kb;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j4 = 0; j4 < 4; ++j4) {
      f32x4 o = {acc[4 * j4][i], acc[4 * j4 + 1][i], acc[4 * j4 + 2][i], acc[4 * j4 + 3][i]};
      *(f32x4*)(part + c * kD + 16 * (4 * g + i) + 4 * j4) = o * v_scale;
    }
  }
  if (g == 0) {
    part[kHB * kD + c] = m;
    part[kHB * kD + kHB + c] = l;
  }
  __syncthreads();
  const int nheads = min(kHB, a.G - w.hb * kHB);
  cta_merge_store<kHB, kD>(a, (float*)smem, kWaveLds / 4, w, nheads);
  if (a.tickets) fused_combine<kD>(a, w, w.kvh * a.G + w.hb * kHB, nheads, (float*)smem);
}

}  // namespace

int fd_launch_split_mfma_fp8_d256(hipStream_t stream, const SplitArgs& a, int q_dtype, int waves, bool soft_cap) {
  const dim3 grid = fd_split_grid(a);
  const unsigned block = 64u * waves;
  size_t lds = (size_t)waves * kWaveLds;
  if (a.tickets) {
    const size_t need = (size_t)(a.S + a.num_extra) * kHB * 4;
    if (need > lds) lds = need;
  }
  void (*kern)(const SplitArgs) = nullptr;
  if (q_dtype == FD_BF16) {
    kern = soft_cap ? fd_split_mfma_fp8_d256_kernel<__bf16, true> : fd_split_mfma_fp8_d256_kernel<__bf16, false>;
  } else if (q_dtype == FD_F16) {
    kern = soft_cap ? fd_split_mfma_fp8_d256_kernel<_Float16, true> : fd_split_mfma_fp8_d256_kernel<_Float16, false>;
  } else {
    return FD_ERR_UNSUPPORTED;
  }
  if (lds > 64 * 1024) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return FD_ERR_LAUNCH;
  }
  hipLaunchKernelGGL(kern, grid, dim3(block), lds, stream, a);
  return hipGetLastError() == hipSuccess ? FD_OK : FD_ERR_LAUNCH;
}
