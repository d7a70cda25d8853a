// Split-KV GQA paged decode on MFMA with an fp8-e4m3 (OCP) KV cache (gfx950), head_dim 64.
//
// New functionality relative to the reference (python/triton_dist/kernels/nvidia/flash_decode.py:130-239 knows
// no scaled fp8 cache); the arithmetic is that of the head_dim-128 fp8 kernel (fd_split_mfma_fp8.hip): K and V
// bytes are dequantised exactly in registers, the K scale is folded into the softmax scale and the V scale is
// applied once to a wave's finished accumulators.
//
// A token row of one KV head is only 64 bytes -- half a cache line, and too short to fetch K or V in the MFMA
// operand layout with wide loads -- so both go through LDS, and where the layout allows it a wave serves KH = 2
// adjacent KV heads (groups of at most 16 query heads, an even number of KV heads, the two rows contiguous): it
// then reads whole 128-byte lines, 16 KB per tile, and computes two independent attention problems from them.
// The host presents such a pair as one KV head with twice the query heads (SplitArgs.Hkv, .G); with KH = 1 a wave
// reads 64-byte half lines, and the sibling KV head's wave of the same workgroup the other halves.
//
// Per wave (lane = 16*g + c): 64-token tiles of RB = 64*KH byte rows.
//   * K and V: global_load_dwordx4, 1 KB per instruction (lane <- 16-byte chunk of a row; the same row indices
//     serve K and V), staged in LDS with a row pitch of RB + 16 bytes.
//   * Scores S^T[token][head] per KV head: four 16-token sub-tiles x two K=32 steps; the A operand is a ds_read_b64
//     of token c's bytes 32*ks + 8g .. +7, converted; lane (g, c) ends up with head c's scores for tokens
//     16*tt + 4g + i.
//   * P.V per KV head: two K=32 blocks; block kb takes tokens 16*(2kb + e/4) + 4g + e%4, the tokens whose
//     probabilities lane (g, .) holds.  Lane (g, c) reads the dword of dims 4c .. 4c+3 of each of those eight rows
//     (both pitches spread the 64 lanes over all 64 banks), converts it and transposes 8 tokens x 4 dims with
//     v_perm_b32 into 4 A operands of O^T[dim][head] += V^T . P^T.
#include <type_traits>

#include "fd_common.h"
#include "fd_mma.h"

namespace {

constexpr int kD = 64;
constexpr int kTile = 64;              // tokens per tile
constexpr int row_bytes(int kh) { return 64 * kh; }
constexpr int row_pitch(int kh) { return row_bytes(kh) + 16; }          // LDS pitch of a staged row: 80 or 144 B
constexpr int stage_bytes(int kh) { return kTile * row_pitch(kh); }     // one staged K or V tile
constexpr int wave_lds(int kh) { return 2 * stage_bytes(kh); }          // K and V; the K half is reused for the partial
static_assert(stage_bytes(1) >= (16 * kD + 2 * 16) * 4 && stage_bytes(2) >= (32 * kD + 2 * 32) * 4,
              "partial result must fit in the K staging buffer");

template <typename T, bool SOFTCAP, int KH>
__global__ void __launch_bounds__(KH == 2 ? 256 : 512) __attribute__((amdgpu_waves_per_eu(KH == 2 ? 2 : 3))) fd_split_mfma_fp8_d64_kernel(const SplitArgs a) {
  constexpr int kRow = row_pitch(KH);
  constexpr int kStage = stage_bytes(KH);
  constexpr int kWaveLds = wave_lds(KH);
  constexpr int kChunks = row_bytes(KH) / 16;    // 16-byte chunks per row: 4 or 8
  constexpr int kRowsPerLoad = 64 / kChunks;     // rows one wave-wide dwordx4 load covers: 16 or 8
  constexpr int kLoads = kTile / kRowsPerLoad;   // loads per tile and tensor: 4 or 8
  constexpr int kHB = 16 * KH;                   // head slots of the wave's partial result
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 4;
  const int c = lane & 15;

  // KH == 2: w.kvh counts pairs of KV heads, a.G is the query heads of a pair, and there is one head block
  const WorkItem w = decode_work_item(a);
  if (w.skip) return;   // empty range, and the combine does not expect a partial from it
  const int ntok = w.end - w.start;
  const int ntiles = ntok > 0 ? (ntok + kTile - 1) / kTile : 0;
  const int tpw = div_uniform(ntiles + w.nsub - 1, w.nsub);
  const int t0 = w.sub * tpw;
  const int t1 = min(t0 + tpw, ntiles);

  const int group = KH == 2 ? a.G >> 1 : a.G;            // query heads per KV head
  const int head_in_group = KH == 2 ? c : w.hb * 16 + c;
  const bool head_ok = head_in_group < group;

  u32x4 qop[KH][2];  // Q as the MFMA B operand: lane (g, c) holds Q[head c of KV head h2][32*ks + 8g .. +7]
  float kq_scale[KH], scale2[KH], v_scale[KH];
#pragma unroll
  for (int h2 = 0; h2 < KH; ++h2) {
    const int kvh = KH * w.kvh + h2;
    const int head = kvh * group + head_in_group;
    const char* qp = (const char*)a.q + ((int64_t)w.b * a.sq_b + (int64_t)head * a.sq_h) * 2;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      u32x4 z = {0u, 0u, 0u, 0u};
      qop[h2][ks] = head_ok ? *(const u32x4*)(qp + (32 * ks + 8 * g) * 2) : z;
    }
    kq_scale[h2] = a.sm_scale * a.k_scale[kvh];  // K dequantisation folded into the softmax scale
    scale2[h2] = kq_scale[h2] * FD_LOG2E;
    v_scale[h2] = a.v_scale[kvh];                // V dequantisation: once, on the finished accumulators
  }

  const int32_t* bt_row = a.bt + (int64_t)w.b * a.sbt;
  // lane reads the 16-byte chunk lane % kChunks of token kRowsPerLoad * i + lane / kChunks
  const char* kbase = (const char*)a.k + (int64_t)(KH * w.kvh) * a.sk_h + (lane % kChunks) * 16;
  const char* vbase = (const char*)a.v + (int64_t)(KH * w.kvh) * a.sv_h + (lane % kChunks) * 16;
  const int k_pitch = (int)a.sk_t;
  const int v_pitch = (int)a.sv_t;
  char* kb = smem + wave * kWaveLds;
  char* vb = kb + kStage;
  const int stage_off = (lane / kChunks) * kRow + (lane % kChunks) * 16;

  const float inv_cap = SOFTCAP ? 1.0f / a.soft_cap : 0.f;

  // lane l owns token start + 64t + l of tile t (clamped to the last valid token of the split)
  auto tile_slot = [&](int t, int& slot) -> int { return fd_tile_slot<kTile>(a, w, bt_row, t, lane, slot); };

  u32x4 kraw[kLoads], vraw[kLoads];
  auto issue = [&](int rv) {
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int row = __shfl(rv, kRowsPerLoad * i + lane / kChunks);
      kraw[i] = load_stream_b128(kbase + (int64_t)row * k_pitch);
      vraw[i] = load_stream_b128(vbase + (int64_t)row * v_pitch);
    }
  };

  float m[KH], l[KH];
  f32x4 acc[KH][4];  // acc[h2][j][i] = O[head c of KV head h2][dim 4*(4g + i) + j]
#pragma unroll
  for (int h2 = 0; h2 < KH; ++h2) {
    m[h2] = -INFINITY;
    l[h2] = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[h2][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  int pg_next = 0, slot_next = 0;

  auto tile = [&](int t, auto has_next_tag) {
    constexpr bool HAS_NEXT = decltype(has_next_tag)::value;
    // ---- K and V tiles -> LDS, then request the next tile
    wave_lds_fence();
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      *(u32x4*)(kb + kRowsPerLoad * i * kRow + stage_off) = kraw[i];
      *(u32x4*)(vb + kRowsPerLoad * i * kRow + stage_off) = vraw[i];
    }
    wave_lds_fence();
    if constexpr (HAS_NEXT) {
      __builtin_amdgcn_sched_barrier(0);
      issue(fd_flat_row(a, pg_next, slot_next));
      pg_next = tile_slot(min(t + 2, t1 - 1), slot_next);
      __builtin_amdgcn_sched_barrier(0);
    }
    const int n0 = w.start + t * kTile;
    const bool full = n0 + kTile <= w.end;
#pragma unroll
    for (int h2 = 0; h2 < KH; ++h2) {
      // ---- S^T = K . Q^T, four 16-token sub-tiles
      f32x4 s[4];
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) s[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
          const u32x2 kk = *(const u32x2*)(kb + (16 * tt + c) * kRow + 64 * h2 + (4 * ks + g) * 8);
          const uint32_t k0 = kk[0], k1 = kk[1];
          u32x4 ak = {Mma<T>::from_fp8(k0, false), Mma<T>::from_fp8(k0, true), Mma<T>::from_fp8(k1, false),
                      Mma<T>::from_fp8(k1, true)};
          s[tt] = Mma<T>::run(ak, qop[h2][ks], s[tt]);
        }
      }
      // ---- online softmax: x[4*tt + i] <-> token 16*tt + 4g + i, head c
      float x[16];
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v = s[tt][i];
          if (SOFTCAP) {
            v = fd_softcap(v * kq_scale[h2], a.soft_cap, inv_cap) * FD_LOG2E;
          } else {
            v *= scale2[h2];
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
      const float alpha = fd_softmax_step(x, m[h2], l[h2], moved);
      if (moved) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[h2][j] *= alpha;
      }
      // ---- V: dequantise, transpose 8 tokens x 4 dims per block, O^T += V^T . P^T
#pragma unroll
      for (int kblk = 0; kblk < 2; ++kblk) {
        u32x4 pop;  // P^T B operand: element e <-> token 16*(2kblk + e/4) + 4g + e%4
#pragma unroll
        for (int q2 = 0; q2 < 4; ++q2) pop[q2] = Mma<T>::pack(x[8 * kblk + 2 * q2], x[8 * kblk + 2 * q2 + 1]);
        uint32_t cv[8][2];  // cv[e][jp] = dims 4c + (2jp, 2jp+1) of token e as packed 16-bit
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int tok = 16 * (2 * kblk + (e >> 2)) + 4 * g + (e & 3);
          const uint32_t v = *(const uint32_t*)(vb + tok * kRow + 64 * h2 + c * 4);
          cv[e][0] = Mma<T>::from_fp8(v, false);
          cv[e][1] = Mma<T>::from_fp8(v, true);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
          u32x4 vop;
#pragma unroll
          for (int q2 = 0; q2 < 4; ++q2) vop[q2] = __builtin_amdgcn_perm(cv[2 * q2 + 1][j >> 1], cv[2 * q2][j >> 1], sel);
          acc[h2][j] = Mma<T>::run(vop, pop, acc[h2][j]);
        }
      }
    }
  };

  if (t0 < t1) {
    int slot0;
    const int pg0 = tile_slot(t0, slot0);
    pg_next = tile_slot(min(t0 + 1, t1 - 1), slot_next);
    __builtin_amdgcn_sched_barrier(0);
    issue(fd_flat_row(a, pg0, slot0));
    __builtin_amdgcn_sched_barrier(0);
    for (int t = t0; t < t1 - 1; ++t) tile(t, std::true_type{});
    tile(t1 - 1, std::false_type{});
  }

  // ---- wave result -> LDS (the wave's own staging buffer), then workgroup merge.  KH == 2: the heads of the two
  // KV heads are stored back to back (slot h2 * group + c) as the heads of the pair.
  wave_lds_fence();
  float* part = (float*)kb;
#pragma unroll
  for (int h2 = 0; h2 < KH; ++h2) {
    float lsum = l[h2];
    lsum += __shfl_xor(lsum, 16);
    lsum += __shfl_xor(lsum, 32);
    if (KH == 2 && !head_ok) continue;   // (after the shuffles: every lane takes part in them)
    const int h = KH == 2 ? h2 * group + c : c;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f32x4 o = {acc[h2][0][i], acc[h2][1][i], acc[h2][2][i], acc[h2][3][i]};
      *(f32x4*)(part + h * kD + 4 * (4 * g + i)) = o * v_scale[h2];
    }
    if (g == 0) {
      part[kHB * kD + h] = m[h2];
      part[kHB * kD + kHB + h] = lsum;
    }
  }
  __syncthreads();
  const int nheads = KH == 2 ? a.G : min(16, a.G - w.hb * 16);
  cta_merge_store<kHB, kD>(a, (float*)smem, kWaveLds / 4, w, nheads);
  if (a.tickets) fused_combine<kD>(a, w, w.kvh * a.G + w.hb * kHB, nheads, (float*)smem);  // hpw == 1 when fused
}

}  // namespace

template <typename T>
static auto pick_kernel(bool soft_cap, int kh) -> void (*)(const SplitArgs) {
  if (kh == 2) return soft_cap ? fd_split_mfma_fp8_d64_kernel<T, true, 2> : fd_split_mfma_fp8_d64_kernel<T, false, 2>;
  return soft_cap ? fd_split_mfma_fp8_d64_kernel<T, true, 1> : fd_split_mfma_fp8_d64_kernel<T, false, 1>;
}

// kv_heads_per_wave == 2: a.Hkv counts pairs of adjacent KV heads and a.G the query heads of a pair (the caller has
// checked that the two 64-byte rows of a pair are contiguous and that a.G <= 32).
int fd_launch_split_mfma_fp8_d64(hipStream_t stream, const SplitArgs& a, int q_dtype, int waves, bool soft_cap,
                                 int kv_heads_per_wave) {
  const int kh = kv_heads_per_wave == 2 ? 2 : 1;
  const dim3 grid = fd_split_grid(a);
  const unsigned block = 64u * waves;
  if (kh == 2 && waves > 4) return FD_ERR_UNSUPPORTED;
  size_t lds = (size_t)waves * wave_lds(kh);
  if (a.tickets) {  // the fused combine stages (S + num_extra) LSEs per head in LDS
    const size_t need = (size_t)(a.S + a.num_extra) * 16 * kh * 4;
    if (need > lds) lds = need;
  }
  void (*kern)(const SplitArgs) = nullptr;
  if (q_dtype == FD_BF16) {
    kern = pick_kernel<__bf16>(soft_cap, kh);
  } else if (q_dtype == FD_F16) {
    kern = pick_kernel<_Float16>(soft_cap, kh);
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
