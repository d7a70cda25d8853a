// Split-KV GQA paged decode on MFMA (gfx950), head_dim 256, 16-bit KV cache.
//
// Same role and decomposition as the head_dim-128 kernel (fd_split_mfma.hip); what changes is
// the tile.  A token row is 512 bytes, so a tile is 16 tokens (8 KB of K + 8 KB of V in flight
// per wave, as there) and a lane (g, c) of the wave holds, for each of its 4 tokens 4g..4g+3,
// chunk c of the LOW half of the row (dims 8c..8c+7) and chunk c of the HIGH half (dims
// 128+8c..): 8 + 8 global_load_dwordx4 per tile, every instruction covering four half rows.
//   * S^T[token][head] = K . Q^T: 8 k-steps of v_mfma_f32_16x16x32 over the staged K tile
//     (LDS pitch 528 B), one 16-token block; lane (g, c) ends up with head c's scores of the
//     tokens 4g..4g+3 whose V rows it holds.
//   * O^T[dim][head] += V^T . P^T on v_mfma_f32_16x16x16 (k = 16 tokens: lane (g, .) supplies
//     k = 4g..4g+3), 16 accumulator blocks: block (h, j) holds dims 128h + 32g + 8i + j.
#include <type_traits>

#include "fd_common.h"
#include "fd_mma.h"

namespace {

constexpr int kD = 256;
constexpr int kTile = 16;         // tokens per tile
constexpr int kKRow = 528;        // LDS pitch of a staged K row in bytes (512 + 16 pad)
constexpr int kHB = 16;           // head slots per workgroup (MFMA N)
constexpr int kWaveLds = (kHB * kD + 2 * kHB) * 4;   // 16512 B: the wave's partial result; the K tile (8448 B) fits
static_assert(kWaveLds >= kTile * kKRow, "K staging buffer must fit");

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

// v_mfma_f32_16x16x16_{bf16,f16}: lane l = 16g + r supplies A[row r][k = 4g..4g+3] and B[k = 4g..4g+3][col r]
// (4 packed 16-bit values = 2 dwords each) and receives D[row 4g+i][col r].
template <typename T>
__device__ __forceinline__ f32x4 mma16(u32x2 a, u32x2 b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 mma16<__bf16>(u32x2 a, u32x2 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mma16<_Float16>(u32x2 a, u32x2 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
}

template <typename T, bool SOFTCAP>
__global__ void __launch_bounds__(512) fd_split_mfma16_d256_kernel(const SplitArgs a) {
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

  // Q as the MFMA B operand: lane (g, c) holds Q[head c][32*ks + 8g .. +7], ks = 0..7.
  u32x4 qop[8];
  {
    const char* qp = (const char*)a.q + ((int64_t)w.b * a.sq_b + (int64_t)head * a.sq_h) * 2;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      u32x4 z = {0u, 0u, 0u, 0u};
      qop[ks] = head_ok ? *(const u32x4*)(qp + (32 * ks + 8 * g) * 2) : z;
    }
  }

  const int32_t* bt_row = a.bt + (int64_t)w.b * a.sbt;
  const char* kbase = (const char*)a.k + ((int64_t)w.kvh * a.sk_h) * 2 + c * 16;
  const char* vbase = (const char*)a.v + ((int64_t)w.kvh * a.sv_h) * 2 + c * 16;
  const int k_pitch = (int)(a.sk_t * 2);
  const int v_pitch = (int)(a.sv_t * 2);
  char* kb = smem + wave * kWaveLds;

  float scale2 = a.sm_scale * FD_LOG2E;
  const float inv_cap = SOFTCAP ? 1.0f / a.soft_cap : 0.f;

  // lane (l & 15) owns token start + 16t + (l & 15) of tile t; the raw table entry is returned and turned
  // into a row by the consumer one iteration later (the load stays in flight across a tile)
  auto tile_slot = [&](int t, int& slot) -> int { return fd_tile_slot<kTile>(a, w, bt_row, t, c, slot); };

  u32x4 kraw[8], vraw[8];   // [2 * i + h]: token 4g + i, half h
  int rows[4];
  auto fetch_rows = [&](int page, int slot) {
    const int rv = fd_flat_row(a, page, slot);
#pragma unroll
    for (int i = 0; i < 4; ++i) rows[i] = __shfl(rv, 4 * g + i);
  };
  auto issue_k = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const char* p = kbase + (int64_t)rows[i] * k_pitch;
      kraw[2 * i] = load_stream_b128(p);
      kraw[2 * i + 1] = load_stream_b128(p + 256);
    }
  };
  auto issue_v = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const char* p = vbase + (int64_t)rows[i] * v_pitch;
      vraw[2 * i] = load_stream_b128(p);
      vraw[2 * i + 1] = load_stream_b128(p + 256);
    }
  };

  float m = -INFINITY;
  float l = 0.f;
  f32x4 acc[2][8];   // acc[h][j][i] = O[head c][dim 128h + 32g + 8i + j]
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[h][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  int pg_next = 0, slot_next = 0;

  auto tile = [&](int t, auto has_next_tag) {
    constexpr bool HAS_NEXT = decltype(has_next_tag)::value;
    wave_lds_fence();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *(u32x4*)(kb + (4 * g + i) * kKRow + c * 16) = kraw[2 * i];
      *(u32x4*)(kb + (4 * g + i) * kKRow + 256 + c * 16) = kraw[2 * i + 1];
    }
    wave_lds_fence();
    if constexpr (HAS_NEXT) {
      __builtin_amdgcn_sched_barrier(0);
      fetch_rows(pg_next, slot_next);
      issue_k();
      pg_next = tile_slot(min(t + 2, t1 - 1), slot_next);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- S^T = K . Q^T (16 tokens x 16 heads)
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      u32x4 a0 = *(const u32x4*)(kb + c * kKRow + (4 * ks + g) * 16);
      s0 = Mma<T>::run(a0, qop[ks], s0);
    }
    // ---- online softmax (head c, tokens 4g..4g+3)
    float x[4];
    const int n0 = w.start + t * kTile;
    const bool full = n0 + kTile <= w.end;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = s0[i];
      if (SOFTCAP) {
        v = fd_softcap(v * a.sm_scale, a.soft_cap, inv_cap) * FD_LOG2E;
      } else {
        v *= scale2;
      }
      x[i] = v;
    }
    if (!full) {   // only the last tile of a range has tokens to mask (wave-uniform branch)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n0 + 4 * g + i >= w.end) x[i] = -INFINITY;
    }
    bool moved;
    const float alpha = fd_softmax_step(x, m, l, moved);
    if (moved) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[h][j] *= alpha;
    }
    u32x2 pop;  // P^T as the B operand: k = 4g + e <-> token 4g + e
    pop[0] = Mma<T>::pack(x[0], x[1]);
    pop[1] = Mma<T>::pack(x[2], x[3]);

    // ---- V: transpose the lane's 4 tokens x (8 + 8) dims into 16 A operands
    u32x2 vop[2][8];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
        vop[h][j][0] = __builtin_amdgcn_perm(vraw[2 + h][j >> 1], vraw[h][j >> 1], sel);
        vop[h][j][1] = __builtin_amdgcn_perm(vraw[6 + h][j >> 1], vraw[4 + h][j >> 1], sel);
      }
    if constexpr (HAS_NEXT) {
      __builtin_amdgcn_sched_barrier(0);
      issue_v();
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- O^T += V^T . P^T
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[h][j] = mma16<T>(vop[h][j], pop, acc[h][j]);
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
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f32x4 lo = {acc[h][0][i], acc[h][1][i], acc[h][2][i], acc[h][3][i]};
      f32x4 hi = {acc[h][4][i], acc[h][5][i], acc[h][6][i], acc[h][7][i]};
      *(f32x4*)(part + c * kD + 128 * h + 32 * g + 8 * i) = lo;
      *(f32x4*)(part + c * kD + 128 * h + 32 * g + 8 * i + 4) = hi;
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

int fd_launch_split_mfma_d256(hipStream_t stream, const SplitArgs& a, int kv_dtype, int waves, bool soft_cap) {
  const dim3 grid = fd_split_grid(a);
  const unsigned block = 64u * waves;
  size_t lds = (size_t)waves * kWaveLds;
  if (a.tickets) {
    const size_t need = (size_t)(a.S + a.num_extra) * kHB * 4;
    if (need > lds) lds = need;
  }
  void (*kern)(const SplitArgs) = nullptr;
  if (kv_dtype == FD_BF16) {
    kern = soft_cap ? fd_split_mfma16_d256_kernel<__bf16, true> : fd_split_mfma16_d256_kernel<__bf16, false>;
  } else if (kv_dtype == FD_F16) {
    kern = soft_cap ? fd_split_mfma16_d256_kernel<_Float16, true> : fd_split_mfma16_d256_kernel<_Float16, false>;
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
