// Split-KV GQA paged decode on MFMA (gfx950), head_dim 64, 16-bit KV cache.
//
// A token row is 128 bytes -- the byte geometry of the fp8 kernel's 128-dim rows
// (fd_split_mfma_fp8.hip) -- so the tile and the load pattern are the same, without the
// conversions.  Per wave (lane = 16*g + c): 64-token tiles (8 KB of K and 8 KB of V).
//   * K: 8 x global_load_dwordx4, eight whole 128-byte rows per instruction; staged in LDS
//     (row pitch 144 B) and read back with ds_read_b128 as the MFMA A operand (lane (g, m) <-
//     token m's dims 32*ks + 8g .. +7, ks = 0, 1).
//   * Scores S^T[token][head]: four 16-token sub-tiles; lane (g, c) ends up with head c's
//     scores for tokens 16*tt + 4g + i.
//   * V: 16 x global_load_dwordx2.  The 64 tokens form two K=32 MFMA blocks for P.V; block kb
//     takes tokens 16*(2kb + e/4) + 4g + e%4, the tokens whose probabilities lane (g, .) holds.
//     Lane (g, c = 8u + cc) loads the 8 bytes 16*cc + 8u .. +7 of those rows = dims 8cc + 4u .. +3
//     and transposes its 8 tokens x 4 dims with v_perm_b32 into 4 A operands of
//     O^T[dim][head] += V^T . P^T.
#include <type_traits>

#include "fd_common.h"
#include "fd_mma.h"

namespace {

constexpr int kD = 64;
constexpr int kTile = 64;         // tokens per tile
constexpr int kKRow = 144;        // LDS pitch of a staged K row in bytes (128 + 16 pad)
constexpr int kWaveLds = kTile * kKRow;  // 9216 B per wave, reused for the wave's partial result
constexpr int kHB = 16;
static_assert(kWaveLds >= (kHB * kD + 2 * kHB) * 4, "partial result must fit in the K staging buffer");

template <typename T, bool SOFTCAP>
__global__ void __launch_bounds__(512) fd_split_mfma16_d64_kernel(const SplitArgs a) {
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

  u32x4 qop[2];  // Q as the MFMA B operand: lane (g, c) holds Q[head c][32*ks + 8g .. +7]
  {
    const char* qp = (const char*)a.q + ((int64_t)w.b * a.sq_b + (int64_t)head * a.sq_h) * 2;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      u32x4 z = {0u, 0u, 0u, 0u};
      qop[ks] = head_ok ? *(const u32x4*)(qp + (32 * ks + 8 * g) * 2) : z;
    }
  }

  const int32_t* bt_row = a.bt + (int64_t)w.b * a.sbt;
  // K: lane reads the 16-byte chunk (lane & 7) of token 8i + (lane >> 3); V: 8 bytes at 16*cc + 8u
  const char* kbase = (const char*)a.k + (int64_t)w.kvh * a.sk_h * 2 + (lane & 7) * 16;
  const char* vbase = (const char*)a.v + (int64_t)w.kvh * a.sv_h * 2 + (c & 7) * 16 + (c >> 3) * 8;
  const int k_pitch = (int)(a.sk_t * 2);
  const int v_pitch = (int)(a.sv_t * 2);
  char* kb = smem + wave * kWaveLds;

  const float scale2 = a.sm_scale * FD_LOG2E;
  const float inv_cap = SOFTCAP ? 1.0f / a.soft_cap : 0.f;

  // lane l owns token start + 64t + l of tile t (clamped to the last valid token of the split)
  auto tile_slot = [&](int t, int& slot) -> int { return fd_tile_slot<kTile>(a, w, bt_row, t, lane, slot); };
  auto flat_row = [&](int page, int slot) -> int {
    return fd_flat_row(a, page, slot);
  };

  u32x4 kraw[8];
  u32x2 vraw[16];
  auto issue_k = [&](int rv) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = __shfl(rv, 8 * i + (lane >> 3));
      kraw[i] = load_stream_b128(kbase + (int64_t)row * k_pitch);
    }
  };
  auto issue_v = [&](int rv, int kblk) {  // the 8 rows of P.V block kblk
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int row = __shfl(rv, 16 * (2 * kblk + (e >> 2)) + 4 * g + (e & 3));
      vraw[8 * kblk + e] = load_stream_b64(vbase + (int64_t)row * v_pitch);
    }
  };

  float m = -INFINITY;
  float l = 0.f;
  f32x4 acc[4];  // acc[j][i] = O[head c][dim 8*(r & 7) + 4*(r >> 3) + j], r = 4g + i
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

  int pg_next = 0, slot_next = 0;
  int rv_cur = 0;  // flat rows of the tile whose V is still to be requested

  auto tile = [&](int t, auto has_next_tag) {
    constexpr bool HAS_NEXT = decltype(has_next_tag)::value;
    // ---- K tile -> LDS, then request the next tile's K
    wave_lds_fence();
#pragma unroll
    for (int i = 0; i < 8; ++i) *(u32x4*)(kb + (8 * i + (lane >> 3)) * kKRow + (lane & 7) * 16) = kraw[i];
    wave_lds_fence();
    if constexpr (HAS_NEXT) {
      __builtin_amdgcn_sched_barrier(0);
      rv_cur = flat_row(pg_next, slot_next);
      issue_k(rv_cur);
      pg_next = tile_slot(min(t + 2, t1 - 1), slot_next);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- S^T = K . Q^T, four 16-token sub-tiles
    f32x4 s[4];
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) s[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
        const u32x4 ak = *(const u32x4*)(kb + (16 * tt + c) * kKRow + (4 * ks + g) * 16);
        s[tt] = Mma<T>::run(ak, qop[ks], s[tt]);
      }
    }
    // ---- online softmax: x[4*tt + i] <-> token 16*tt + 4g + i, head c
    float x[16];
    const int n0 = w.start + t * kTile;
    const bool full = n0 + kTile <= w.end;
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = s[tt][i];
        if (SOFTCAP) {
          v = fd_softcap(v * a.sm_scale, a.soft_cap, inv_cap) * FD_LOG2E;
        } else {
          v *= scale2;
        }
        x[4 * tt + i] = v;
      }
    }
    if (!full) {   // only the last tile of a range has tokens to mask (wave-uniform branch)
#pragma unroll
      for (int e = 0; e < 16; ++e)
        if (n0 + 16 * (e >> 2) + 4 * g + (e & 3) >= w.end) x[e] = -INFINITY;
    }
    bool moved;
    const float alpha = fd_softmax_step(x, m, l, moved);
    if (moved) {
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] *= alpha;
    }
    u32x4 pop[2];  // P^T B operands: block kblk, element e <-> token 16*(2kblk + e/4) + 4g + e%4
#pragma unroll
    for (int kblk = 0; kblk < 2; ++kblk)
#pragma unroll
      for (int q2 = 0; q2 < 4; ++q2) pop[kblk][q2] = Mma<T>::pack(x[8 * kblk + 2 * q2], x[8 * kblk + 2 * q2 + 1]);

    // ---- V: transpose 8 tokens x 4 dims per block, O^T += V^T . P^T
#pragma unroll
    for (int kblk = 0; kblk < 2; ++kblk) {
      u32x4 vop[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
        for (int q2 = 0; q2 < 4; ++q2)
          vop[j][q2] = __builtin_amdgcn_perm(vraw[8 * kblk + 2 * q2 + 1][j >> 1], vraw[8 * kblk + 2 * q2][j >> 1], sel);
      }
      if constexpr (HAS_NEXT) {
        // this block's V registers have just been consumed: refill them in place with the next tile's rows
        __builtin_amdgcn_sched_barrier(0);
        issue_v(rv_cur, kblk);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = Mma<T>::run(vop[j], pop[kblk], acc[j]);
    }
  };

  if (t0 < t1) {
    int slot0;
    const int pg0 = tile_slot(t0, slot0);
    pg_next = tile_slot(min(t0 + 1, t1 - 1), slot_next);
    __builtin_amdgcn_sched_barrier(0);
    rv_cur = flat_row(pg0, slot0);
    issue_k(rv_cur);
    issue_v(rv_cur, 0);
    issue_v(rv_cur, 1);
    __builtin_amdgcn_sched_barrier(0);
    for (int t = t0; t < t1 - 1; ++t) tile(t, std::true_type{});
    tile(t1 - 1, std::false_type{});
  }

  // ---- wave result -> LDS (the wave's own staging buffer), then workgroup merge
  l += __shfl_xor(l, 16);
  l += __shfl_xor(l, 32);
  wave_lds_fence();
  float* part = (float*)kb;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * g + i;
    const int dim0 = 8 * (r & 7) + 4 * (r >> 3);
    f32x4 o = {acc[0][i], acc[1][i], acc[2][i], acc[3][i]};
    *(f32x4*)(part + c * kD + dim0) = o;
  }
  if (g == 0) {
    part[kHB * kD + c] = m;
    part[kHB * kD + kHB + c] = l;
  }
  __syncthreads();
  const int nheads = min(kHB, a.G - w.hb * kHB);
  cta_merge_store<kHB, kD>(a, (float*)smem, kWaveLds / 4, w, nheads);
  if (a.tickets) fused_combine<kD>(a, w, w.kvh * a.G + w.hb * kHB, nheads, (float*)smem);  // hpw == 1 when fused
}

}  // namespace

int fd_launch_split_mfma_d64(hipStream_t stream, const SplitArgs& a, int kv_dtype, int waves, bool soft_cap) {
  const dim3 grid = fd_split_grid(a);
  const unsigned block = 64u * waves;
  size_t lds = (size_t)waves * kWaveLds;
  if (a.tickets) {
    const size_t need = (size_t)(a.S + a.num_extra) * kHB * 4;
    if (need > lds) lds = need;
  }
  void (*kern)(const SplitArgs) = nullptr;
  if (kv_dtype == FD_BF16) {
    kern = soft_cap ? fd_split_mfma16_d64_kernel<__bf16, true> : fd_split_mfma16_d64_kernel<__bf16, false>;
  } else if (kv_dtype == FD_F16) {
    kern = soft_cap ? fd_split_mfma16_d64_kernel<_Float16, true> : fd_split_mfma16_d64_kernel<_Float16, false>;
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
