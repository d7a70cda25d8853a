// Split-KV GQA paged decode on MFMA with an fp8-e4m3 (OCP) KV cache (gfx950), head_dim 128.
//
// New functionality relative to the reference, whose split kernel
// (python/triton_dist/kernels/nvidia/flash_decode.py:130-239) would cast an fp8
// cache with `k.to(q.dtype)` and no scales (:208) and round P to fp8 (:230).
// Here K and V bytes are dequantised in registers -- v_cvt_scalef32_pk_{bf16,f16}_fp8
// turns two e4m3 bytes into two packed 16-bit values exactly -- and fed to the same
// 16x16x32 MFMA as the 16-bit kernel; the per-KV-head K scale is folded into the
// softmax scale and the V scale is applied once to a wave's finished accumulators.
//
// Geometry per wave (lane = 16*g + m): 64-token tiles (8 KB of K and 8 KB of V).
//   * K: 8 x global_load_dwordx4, eight whole 128-byte rows per instruction; staged
//     in LDS (row pitch 144 B) and read back as the MFMA A operand with ds_read_b64
//     (lane (g, m) <- token m's bytes 32*ks + 8g .. +7), converted, multiplied with Q.
//   * Scores S^T[token][head]: four 16-token sub-tiles; lane (g, c) ends up with head
//     c's scores for tokens 16*tt + 4g + i.
//   * V: 16 x global_load_dwordx2.  For P.V the 64 tokens form two K=32 MFMA blocks;
//     block kb takes tokens tau(g,e,kb) = 16*(2kb + e/4) + 4g + e%4, which are exactly
//     the tokens whose probabilities lane (g, .) holds.  Lane (g, m = 8u + cc) loads the
//     8 bytes 16*cc + 8u .. +7 of those rows (the two u-halves of a wave row read one
//     contiguous 16 bytes, the eight cc a whole row), converts them and transposes the
//     8x8 block with v_perm_b32 into 8 A operands of O^T[dim][head] += V^T . P^T.
#include <type_traits>

#include "fd_common.h"
#include "fd_mma.h"

namespace {

constexpr int kD = 128;
constexpr int kTile = 64;         // tokens per tile
constexpr int kKRow = 144;        // LDS pitch of a staged fp8 K row in bytes (128 + 16 pad)
constexpr int kKTile = kTile * kKRow;   // 9216 B of staged K per wave
// LDS per wave: the K staging buffer, reused for the wave's partial result (16*NB heads x (128 + 2) floats)
constexpr int wave_lds(int nb) { return nb == 1 ? kKTile : (16 * nb * kD + 2 * 16 * nb) * 4; }
static_assert(wave_lds(1) >= (16 * kD + 2 * 16) * 4 && wave_lds(2) >= kKTile, "partial result and K tile share the buffer");
static_assert(wave_lds(1) >= 16 * 4 + 16 * kD * 4 && wave_lds(2) >= 32 * 4 + 32 * kD * 4, "a finished fp32 partial fits the staging buffer");

// NB = 2 (groups above 16 query heads): a wave serves two 16-head blocks from the same converted K operands and the
// same converted, transposed V operands; only the MFMAs and the softmax are done per block.
// CHUNK: a workgroup walks SplitArgs::chunk consecutive splits; every wave owns whole splits, streams their tiles as
// one run and stores one partial per split itself (see the 16-bit kernel).
template <typename T, bool SOFTCAP, int NB, bool CHUNK>
__global__ void __launch_bounds__(NB == 2 ? 256 : 512) fd_split_mfma_fp8_kernel(const SplitArgs a) {
  constexpr int kHB = 16 * NB;            // head slots per wave
  constexpr int kWaveLds = wave_lds(NB);
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 4;
  const int c = lane & 15;

  const WorkItem w = decode_work_item(a);   // this wave: KV head w.kvh, token sub-range w.sub of w.nsub
  if (w.skip) return;   // empty range, and the combine does not expect a partial from it
  if (CHUNK && w.ns <= 0) return;   // more waves than splits in the last work item of a sequence (no barrier follows)
  const int ntok = w.end - w.start;
  const int ntiles = ntok > 0 ? (ntok + kTile - 1) / kTile : 0;
  const int tpw = div_uniform(ntiles + w.nsub - 1, w.nsub);
  const int t0 = w.sub * tpw;
  const int t1 = min(t0 + tpw, ntiles);

  u32x4 qop[NB][4];  // Q as the MFMA B operand: lane (g, c) holds Q[head 16*nb + c][32*ks + 8g .. +7]
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int head_in_group = w.hb * kHB + 16 * nb + c;
    const bool head_ok = head_in_group < a.G;
    const int head = w.kvh * a.G + head_in_group;
    const char* qp = (const char*)a.q + ((int64_t)w.b * a.sq_b + (int64_t)head * a.sq_h) * 2;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      u32x4 z = {0u, 0u, 0u, 0u};
      qop[nb][ks] = head_ok ? *(const u32x4*)(qp + (32 * ks + 8 * g) * 2) : z;
    }
  }

  const int32_t* bt_row = a.bt + (int64_t)w.b * a.sbt;
  // K: lane reads the 16-byte chunk (lane & 7) of token 8i + (lane >> 3); V: 8 bytes at 16*cc + 8u
  const char* kbase = (const char*)a.k + (int64_t)w.kvh * a.sk_h + (lane & 7) * 16;
  const char* vbase = (const char*)a.v + (int64_t)w.kvh * a.sv_h + (c & 7) * 16 + (c >> 3) * 8;
  const int k_pitch = (int)a.sk_t;
  const int v_pitch = (int)a.sv_t;
  char* kb = smem + wave * kWaveLds;

  const float kq_scale = a.sm_scale * a.k_scale[w.kvh];  // K dequantisation folded into the softmax scale
  const float v_scale = a.v_scale[w.kvh];                // V dequantisation: once, on the finished accumulators
  const float scale2 = kq_scale * FD_LOG2E;
  const float inv_cap = SOFTCAP ? 1.0f / a.soft_cap : 0.f;

  // lane l owns token start + 64t + l of tile t (clamped to the last valid token of the split)
  auto tile_slot = [&](int t, int& slot) -> int { return fd_tile_slot<kTile>(a, w, bt_row, t, lane, slot); };
  // ... or, with chunked work items, token n0 + l of the tile that starts at n0 in a split that ends at n_end
  auto token_slot = [&](int n0, int n_end, int& slot) -> int {
    const int n = min(n0 + lane, n_end - 1);
    const int pidx = page_index(a, n);
    slot = n - pidx * a.P;
    return bt_row[pidx];
  };
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

  float m[NB], l[NB];
  f32x4 acc[NB][8];  // acc[nb][j][i] = O[head 16*nb + c][dim 16*(r & 7) + 8*(r >> 3) + j], r = 4g + i
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    m[nb] = -INFINITY;
    l[nb] = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[nb][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  int pg_next = 0, slot_next = 0;
  int rv_cur = 0;  // flat rows of the tile whose V is still to be requested

  // n0 / n_end: first token of the tile and end of its split (for the mask); lookup2(slot): table entry and slot of
  // this lane's token two tiles ahead.
  auto tile = [&](const int n0, const int n_end, auto&& lookup2, auto has_next_tag) {
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
      pg_next = lookup2(slot_next);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- S^T = K . Q^T, four 16-token sub-tiles
    f32x4 s[NB][4];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) s[nb][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
        const u32x2 kk = *(const u32x2*)(kb + (16 * tt + c) * kKRow + (4 * ks + g) * 8);
        const uint32_t k0 = kk[0], k1 = kk[1];
        u32x4 ak = {Mma<T>::from_fp8(k0, false), Mma<T>::from_fp8(k0, true), Mma<T>::from_fp8(k1, false),
                    Mma<T>::from_fp8(k1, true)};
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) s[nb][tt] = Mma<T>::run(ak, qop[nb][ks], s[nb][tt]);
      }
    }
    // ---- online softmax: x[4*tt + i] <-> token 16*tt + 4g + i, head 16*nb + c
    const bool full = n0 + kTile <= n_end;
    u32x4 pop[NB][2];  // P^T B operands: block kb, element e <-> token 16*(2kb + e/4) + 4g + e%4
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float x[16];
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v = s[nb][tt][i];
          if (SOFTCAP) {
            v = fd_softcap(v * kq_scale, a.soft_cap, inv_cap) * FD_LOG2E;
          } else {
            v *= scale2;
          }
          x[4 * tt + i] = v;
        }
      }
      if (!full) {   // only the last tile of a range has tokens to mask (wave-uniform branch)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          if (n0 + 16 * (e >> 2) + 4 * g + (e & 3) >= n_end) x[e] = -INFINITY;
      }
      bool moved;
      const float alpha = fd_softmax_step(x, m[nb], l[nb], moved);
      if (moved) {
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[nb][j] *= alpha;
      }
#pragma unroll
      for (int kblk = 0; kblk < 2; ++kblk)
#pragma unroll
        for (int q2 = 0; q2 < 4; ++q2)
          pop[nb][kblk][q2] = Mma<T>::pack(x[8 * kblk + 2 * q2], x[8 * kblk + 2 * q2 + 1]);
    }

    // ---- V: dequantise, transpose 8 tokens x 8 dims per block, O^T += V^T . P^T
#pragma unroll
    for (int kblk = 0; kblk < 2; ++kblk) {
      uint32_t cv[8][4];  // cv[e][jp] = dims (2jp, 2jp+1) of token e as packed 16-bit
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t v0 = vraw[8 * kblk + e][0], v1 = vraw[8 * kblk + e][1];
        cv[e][0] = Mma<T>::from_fp8(v0, false);
        cv[e][1] = Mma<T>::from_fp8(v0, true);
        cv[e][2] = Mma<T>::from_fp8(v1, false);
        cv[e][3] = Mma<T>::from_fp8(v1, true);
      }
      if constexpr (HAS_NEXT) {
        // this block's V registers have just been consumed: refill them in place with the next tile's rows
        __builtin_amdgcn_sched_barrier(0);
        issue_v(rv_cur, kblk);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
        u32x4 vop;
#pragma unroll
        for (int q2 = 0; q2 < 4; ++q2) vop[q2] = __builtin_amdgcn_perm(cv[2 * q2 + 1][j >> 1], cv[2 * q2][j >> 1], sel);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb][j] = Mma<T>::run(vop, pop[nb][kblk], acc[nb][j]);
      }
    }
  };

  // A wave's finished state -> its own LDS buffer (the K staging buffer), in cta_merge_store's layout, already
  // multiplied by the V scale.
  float* part = (float*)kb;
  auto stage_partial = [&](float* part) {
    wave_lds_fence();
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float lsum = l[nb];
      lsum += __shfl_xor(lsum, 16);
      lsum += __shfl_xor(lsum, 32);
      const int h = 16 * nb + c;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 4 * g + i;
        const int dim0 = 16 * (r & 7) + 8 * (r >> 3);
        f32x4 lo = {acc[nb][0][i], acc[nb][1][i], acc[nb][2][i], acc[nb][3][i]};
        f32x4 hi = {acc[nb][4][i], acc[nb][5][i], acc[nb][6][i], acc[nb][7][i]};
        *(f32x4*)(part + h * kD + dim0) = lo * v_scale;
        *(f32x4*)(part + h * kD + dim0 + 4) = hi * v_scale;
      }
      if (g == 0) {
        part[kHB * kD + h] = m[nb];
        part[kHB * kD + kHB + h] = lsum;
      }
    }
  };
  const int nheads = min(kHB, a.G - w.hb * kHB);
  // Chunked work items: a finished split -> a parked slot as the finished partial: fp32 LSEs of the head slots,
  // then normalised rows in mid_dtype, times the V scale.  A lane holds eight consecutive dims of head 16*nb + c per i.
  auto park_final = [&](char* slot) {
    wave_lds_fence();
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float lsum = l[nb];
      lsum += __shfl_xor(lsum, 16);
      lsum += __shfl_xor(lsum, 32);
      const int h = 16 * nb + c;
      if (h < nheads) {
        const float inv = lsum > 0.f ? v_scale / lsum : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 4 * g + i;
          float v[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) v[j] = acc[nb][j][i] * inv;
          park_store8(slot + kHB * 4, h * kD + 16 * (r & 7) + 8 * (r >> 3), a.mid_dtype, v);
        }
        if (g == 0) ((float*)slot)[h] = lsum > 0.f ? (m[nb] + fd_log2(lsum)) * FD_LN2 : -INFINITY;
      }
    }
  };

  if constexpr (CHUNK) {
    // Wave-uniform cursors over the tiles of the wave's splits (as in the 16-bit kernel): a tile starts at `base`
    // inside a split that ends at `end`; the cursor stops on the wave's last tile.
    const int per = __builtin_amdgcn_readfirstlane(w.per);
    const int run_end = __builtin_amdgcn_readfirstlane(w.end);
    const int head0 = w.kvh * a.G + w.hb * kHB;
    const int s_cur = __builtin_amdgcn_readfirstlane(w.s);
    const int s_lim = s_cur + __builtin_amdgcn_readfirstlane(w.ns);
    struct Cur { int base, end; };
    auto advance = [&](const Cur cur) -> Cur {
      Cur n = cur;
      n.base += kTile;
      if (n.base >= cur.end) {
        n.base = cur.end;
        n.end = min(cur.end + per, run_end);
      }
      return n.base >= run_end ? cur : n;
    };
    // Finished partials other than the wave's last one wait in LDS behind the staging buffers (a.park slots per
    // wave); all of them are stored when the wave has issued its last load.
    char* park = smem + a.hpw * a.nsub * kWaveLds + (size_t)(wave * a.park) * a.park_bytes;
    int parked = 0;
    bool last_staged = false;
    Cur cur{__builtin_amdgcn_readfirstlane(w.start), 0};
    cur.end = min(cur.base + per, run_end);
    if (cur.base < run_end) {
      Cur look = advance(cur);
      int slot0;
      const int pg0 = token_slot(cur.base, cur.end, slot0);
      pg_next = token_slot(look.base, look.end, slot_next);
      look = advance(look);
      __builtin_amdgcn_sched_barrier(0);
      rv_cur = flat_row(pg0, slot0);
      issue_k(rv_cur);
      issue_v(rv_cur, 0);
      issue_v(rv_cur, 1);
      __builtin_amdgcn_sched_barrier(0);
      auto lookup2 = [&](int& slot) -> int { return token_slot(look.base, look.end, slot); };
      while (!(cur.end >= run_end && cur.base + kTile >= cur.end)) {   // all tiles but the wave's last one
        tile(cur.base, cur.end, lookup2, std::true_type{});
        if (cur.base + kTile >= cur.end) {   // that was the last tile of a split
          park_final(park + parked * a.park_bytes);
          ++parked;
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            m[nb] = -INFINITY;
            l[nb] = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[nb][j] = f32x4{0.f, 0.f, 0.f, 0.f};
          }
        }
        cur = advance(cur);
        look = advance(look);
      }
      tile(cur.base, cur.end, lookup2, std::false_type{});
      park_final(kb);   // the wave's last split: its staging buffer is free now
      last_staged = true;
    }
    wave_lds_fence();
    for (int i = 0; s_cur + i < s_lim; ++i) {   // splits beyond the sequence's end are stored as empty
      const bool empty = i > parked || (i == parked && !last_staged);
      wave_copy_parked<kHB, kD>(a, i < parked ? park + i * a.park_bytes : kb, w.b, head0, nheads, s_cur + i, empty);
    }
  } else {
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
      for (int t = t0; t < t1 - 1; ++t)
        tile(w.start + t * kTile, w.end, [&](int& slot) -> int { return tile_slot(min(t + 2, t1 - 1), slot); },
             std::true_type{});
      tile(w.start + (t1 - 1) * kTile, w.end, [&](int& slot) -> int { return tile_slot(t1 - 1, slot); },
           std::false_type{});
    }

    // ---- wave result -> LDS, then workgroup merge
    stage_partial(part);
    __syncthreads();
    cta_merge_store<kHB, kD>(a, (float*)smem, kWaveLds / 4, w, nheads);
    if (a.tickets) fused_combine<kD>(a, w, w.kvh * a.G + w.hb * kHB, nheads, (float*)smem);  // hpw == 1 when fused
  }
}

}  // namespace

template <typename T, bool CHUNK>
static auto pick_kernel2(bool soft_cap, int nb) -> void (*)(const SplitArgs) {
  if (nb == 2) return soft_cap ? fd_split_mfma_fp8_kernel<T, true, 2, CHUNK> : fd_split_mfma_fp8_kernel<T, false, 2, CHUNK>;
  return soft_cap ? fd_split_mfma_fp8_kernel<T, true, 1, CHUNK> : fd_split_mfma_fp8_kernel<T, false, 1, CHUNK>;
}
template <typename T>
static auto pick_kernel(bool soft_cap, int nb, bool chunk) -> void (*)(const SplitArgs) {
  return chunk ? pick_kernel2<T, true>(soft_cap, nb) : pick_kernel2<T, false>(soft_cap, nb);
}

int fd_launch_split_mfma_fp8(hipStream_t stream, const SplitArgs& a, int q_dtype, int waves, bool soft_cap) {
  const dim3 grid = fd_split_grid(a);
  const unsigned block = 64u * waves;
  const int nb = a.hbsz > 16 ? 2 : 1;   // a.hbsz = query heads per head block: up to 16, or up to 32 (two per wave)
  size_t lds = (size_t)waves * wave_lds(nb);
  if (a.chunk > 1) lds += (size_t)waves * a.park * a.park_bytes;   // parked partials
  if (a.tickets) {  // the fused combine stages (S + num_extra) LSEs per head in LDS
    const size_t need = (size_t)(a.S + a.num_extra) * 16 * nb * 4;
    if (need > lds) lds = need;
  }
  void (*kern)(const SplitArgs) = nullptr;
  if (q_dtype == FD_BF16) {
    kern = pick_kernel<__bf16>(soft_cap, nb, a.chunk > 1);
  } else if (q_dtype == FD_F16) {
    kern = pick_kernel<_Float16>(soft_cap, nb, a.chunk > 1);
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
