// Split-KV GQA paged decode on MFMA (gfx950), head_dim 128, 16-bit KV cache.
//
// Replaces kernel_gqa_fwd_batch_decode_split_kv
// (python/triton_dist/kernels/nvidia/flash_decode.py:130-239) for every GQA group
// (the query heads of a KV head are padded to blocks of 16, the MFMA N).
//
// Decomposition: one workgroup per (sequence, split, KV head, block of <=16*NB
// query heads); its W waves take contiguous runs of 32-token tiles of the split
// and are merged through LDS at the end.  NB = 2 (groups above 16 query heads):
// a wave serves two 16-head blocks from the same K and V registers -- the loads,
// the LDS staging and the V transpose are shared, only the MFMAs and the softmax
// are done per block.
//
// Per 32-token tile and wave (lane = 16*g + c):
//   * 8 + 8 global_load_dwordx4: load i fetches, for every g, the full 256-byte
//     K (and V) row of token tau(g,i) = 4g + (i&3) + 16(i>>2); the 16 lanes of a
//     wave row read consecutive 16-byte chunks, so every load instruction covers
//     four whole rows.  Row addresses come from one block-table lookup per
//     token (lanes 0..31), broadcast with ds_bpermute.
//   * K is staged row-major in LDS (row pitch 272 B: conflict-free 128-bit
//     reads) and read back in the MFMA A layout: lane (g, m) <- K[token m][8
//     dims of chunk 4*ks+g].   S^T[token][head] = K . Q^T on
//     v_mfma_f32_16x16x32_bf16/f16 with Q as the B operand (heads padded to 16).
//     The result leaves lane (g, c) with the scores of head c for tokens
//     4g..4g+3 (+16): exactly the tokens whose V rows the lane holds.
//   * Online softmax in registers (base-2 domain); the row maximum is reduced
//     over the 4 wave rows with two bpermutes, the row sum stays per lane until
//     the end.
//   * V never touches LDS: the 8x8 16-bit blocks a lane holds are transposed
//     with v_perm_b32 into the A operand of O^T[dim][head] += V^T . P^T, so the
//     accumulator also lives in the "lane c = head c" layout and is rescaled
//     without any cross-lane traffic.
#include <type_traits>

#include "fd_common.h"
#include "fd_mma.h"

namespace {

constexpr int kD = 128;
constexpr int kTile = 32;         // tokens per tile
constexpr int kKRow = 272;        // LDS pitch of a staged K row in bytes (256 + 16 pad)
constexpr int kKTile = kTile * kKRow;   // 8704 B of staged K per wave
// LDS per wave: the K staging buffer, reused for the wave's partial result (16*NB heads x (128 + 2) floats)
constexpr int wave_lds(int nb) { return nb == 1 ? kKTile : (16 * nb * kD + 2 * 16 * nb) * 4; }
static_assert(wave_lds(1) >= (16 * kD + 2 * 16) * 4 && wave_lds(2) >= kKTile, "partial result and K tile share the buffer");
static_assert(wave_lds(1) >= 16 * 4 + 16 * kD * 4 && wave_lds(2) >= 32 * 4 + 32 * kD * 4, "a finished fp32 partial fits the staging buffer");

#ifndef FD_MFMA_OCC
#define FD_MFMA_OCC
#endif

// CHUNK: a workgroup walks SplitArgs::chunk consecutive splits.  Every wave owns whole splits: it streams their tiles
// as one run -- Q operands, table row and the K/V pipeline stay alive across a split boundary -- puts each finished
// split's state aside in LDS, and at the end normalises and stores one partial per split itself (no workgroup merge),
// so the caller gets exactly S partials in the reference layout [B, Hq, S, D(+1)] (flash_decode.py:193-195, 235-239)
// from S / chunk long work items.
template <typename T, bool SOFTCAP, int NB, bool CHUNK>
__global__ void __launch_bounds__(NB == 2 ? 256 : 512) FD_MFMA_OCC fd_split_mfma16_kernel(const SplitArgs a) {
  constexpr int kHB = 16 * NB;             // head slots per wave
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

  // Q as the MFMA B operand: lane (g, c) holds Q[head 16*nb + c][32*ks + 8g .. +7].
  u32x4 qop[NB][4];
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
  const char* kbase = (const char*)a.k + ((int64_t)w.kvh * a.sk_h) * 2 + c * 16;
  // (V head dim 64: the 16 lanes of a wave row fetch the 8 chunks of a 128-byte row twice; 256: this wave's half)
  const char* vbase = (const char*)a.v + ((int64_t)w.kvh * a.sv_h) * 2 + (c & a.v_chunk_mask) * 16 + w.vh * 256;
  const int k_pitch = (int)(a.sk_t * 2);
  const int v_pitch = (int)(a.sv_t * 2);
  char* kb = smem + wave * kWaveLds;

  float scale2 = a.sm_scale * FD_LOG2E;  // scores are kept in the base-2 domain
  const float inv_cap = SOFTCAP ? 1.0f / a.soft_cap : 0.f;

  // lane (l & 31) looks up token start + 32t + (l & 31)
  auto tile_slot = [&](int t, int& slot) -> int { return fd_tile_slot<kTile>(a, w, bt_row, t, lane & 31, slot); };
  // ... or, with chunked work items, token n0 + (l & 31) of the tile that starts at n0 in a split that ends at n_end
  auto token_slot = [&](int n0, int n_end, int& slot) -> int {
    const int n = min(n0 + (lane & 31), n_end - 1);
    const int pidx = page_index(a, n);
    slot = n - pidx * a.P;
    return bt_row[pidx];
  };

  // VEARLY (two head blocks per wave, one workgroup per split): a tile's compute is long enough there that a V tile
  // requested only when its predecessor has been consumed leaves the wave with half its bytes in flight for most of
  // the tile.  V gets a second register set instead, and V(t+1) is requested together with K(t+1) at the start of
  // tile t; the tiles of a run alternate between the sets (compile-time parity, the loop is unrolled by two).  With one
  // head block per wave the same change loses: that kernel streams at what the memory gives, and more requests in
  // flight only lengthen the queues (config 2 44.4 -> 45.1 us, a 131072-token sequence 84.8 -> 86.1 us).
  constexpr bool VEARLY = NB == 2 && !CHUNK;
  constexpr int VB = VEARLY ? 2 : 1;
  u32x4 kraw[8], vraw[VB][8];
  int rows[8];
  auto fetch_rows = [&](int page, int slot) {
    // flat cache row = page * P + slot, page clamped into the pool so a corrupt table cannot fault
    const int rv = fd_flat_row(a, page, slot);
#pragma unroll
    for (int i = 0; i < 8; ++i) rows[i] = __shfl(rv, 4 * g + (i & 3) + 16 * (i >> 2));
  };
  auto issue_k = [&]() {
#pragma unroll
    for (int i = 0; i < 8; ++i) kraw[i] = load_stream_b128(kbase + (int64_t)rows[i] * k_pitch);
  };
  auto issue_v = [&](auto set_tag) {
    constexpr int SET = decltype(set_tag)::value;
#pragma unroll
    for (int i = 0; i < 8; ++i) vraw[SET][i] = load_stream_b128(vbase + (int64_t)rows[i] * v_pitch);
  };

  float m[NB];          // running max of head 16*nb + c (identical in the 4 wave rows)
  float l[NB];          // this lane's share of the running sum
  f32x4 acc[NB][8];     // acc[nb][j][i] = O[head 16*nb + c][dim 32g + 8i + j]
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    m[nb] = -INFINITY;
    l[nb] = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[nb][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  int pg_next = 0, slot_next = 0;

  // One tile.  HAS_NEXT is a compile-time flag (the last tile of the wave is peeled off the loop),
  // so the steady-state loop has no branch around a load and the wait counts stay exact:
  // K(t+1) and V(t+1) are in flight while tile t is being computed.
  // n0 / n_end: first token of the tile and end of its split (for the mask); lookup2(slot): table entry and slot of
  // this lane's token two tiles ahead.
  // set_tag: the V register set that holds this tile (always 0 without VEARLY).
  auto tile = [&](const int n0, const int n_end, auto&& lookup2, auto has_next_tag, auto set_tag) {
    constexpr bool HAS_NEXT = decltype(has_next_tag)::value;
    constexpr int SET = decltype(set_tag)::value;
    static_assert(SET < VB, "V register set");
    // ---- K tile -> LDS, then start fetching the next tile's K into the freed registers
    wave_lds_fence();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int tau = 4 * g + (i & 3) + 16 * (i >> 2);
      *(u32x4*)(kb + tau * kKRow + c * 16) = kraw[i];
    }
    wave_lds_fence();
    if constexpr (HAS_NEXT) {
      // the machine scheduler must not sink these loads (or hoist later ones) across this point:
      // the whole pipeline depends on K(t+1) being requested before tile t is computed
      __builtin_amdgcn_sched_barrier(0);
      fetch_rows(pg_next, slot_next);
      issue_k();
      if constexpr (VEARLY) issue_v(std::integral_constant<int, (SET ^ 1) & (VB - 1)>{});
      pg_next = lookup2(slot_next);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- S^T = K . Q^T
    f32x4 s0[NB], s1[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) s0[nb] = s1[nb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      u32x4 a0 = *(const u32x4*)(kb + c * kKRow + (4 * ks + g) * 16);
      u32x4 a1 = *(const u32x4*)(kb + (16 + c) * kKRow + (4 * ks + g) * 16);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        s0[nb] = Mma<T>::run(a0, qop[nb][ks], s0[nb]);
        s1[nb] = Mma<T>::run(a1, qop[nb][ks], s1[nb]);
      }
    }
    // ---- online softmax (head 16*nb + c, tokens tau(g, 0..7))
    const bool full = n0 + kTile <= n_end;
    u32x4 pop[NB];  // P^T as the B operand: element e <-> token tau(g, e)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float x[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        x[i] = s0[nb][i];
        x[4 + i] = s1[nb][i];
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float v = x[i];
        if (SOFTCAP) {
          v = fd_softcap(v * a.sm_scale, a.soft_cap, inv_cap) * FD_LOG2E;
        } else {
          v *= scale2;
        }
        x[i] = v;
      }
      if (!full) {   // only the last tile of a range has tokens to mask (wave-uniform branch)
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (n0 + 4 * g + (i & 3) + 16 * (i >> 2) >= n_end) x[i] = -INFINITY;
      }
      bool moved;
      const float alpha = fd_softmax_step(x, m[nb], l[nb], moved);
      if (moved) {
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[nb][j] *= alpha;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) pop[nb][e] = Mma<T>::pack(x[2 * e], x[2 * e + 1]);
    }

    // ---- V: transpose the lane's 8 tokens x 8 dims block into 8 A operands, O^T += V^T . P^T.
    // The next tile's V is requested as soon as the last raw V register has been consumed.  With two head
    // blocks the operands are built in two halves to stay within the register file.
    constexpr int kHalf = NB == 1 ? 8 : 4;
#pragma unroll
    for (int j0 = 0; j0 < 8; j0 += kHalf) {
      u32x4 vop[kHalf];
#pragma unroll
      for (int jj = 0; jj < kHalf; ++jj) {
        const int j = j0 + jj;
        const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          vop[jj][e] = __builtin_amdgcn_perm(vraw[SET][2 * e + 1][j >> 1], vraw[SET][2 * e][j >> 1], sel);
      }
      if constexpr (HAS_NEXT && !VEARLY) {
        if (j0 + kHalf == 8) {
          __builtin_amdgcn_sched_barrier(0);
          issue_v(set_tag);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
#pragma unroll
      for (int jj = 0; jj < kHalf; ++jj) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb][j0 + jj] = Mma<T>::run(vop[jj], pop[nb], acc[nb][j0 + jj]);
      }
    }
  };

  // A wave's finished state -> its own LDS buffer (the K staging buffer), in cta_merge_store's layout.
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
        f32x4 lo = {acc[nb][0][i], acc[nb][1][i], acc[nb][2][i], acc[nb][3][i]};
        f32x4 hi = {acc[nb][4][i], acc[nb][5][i], acc[nb][6][i], acc[nb][7][i]};
        *(f32x4*)(part + h * kD + 32 * g + 8 * i) = lo;
        *(f32x4*)(part + h * kD + 32 * g + 8 * i + 4) = hi;
      }
      if (g == 0) {
        part[kHB * kD + h] = m[nb];
        part[kHB * kD + kHB + h] = lsum;
      }
    }
  };
  const int nheads = min(kHB, a.G - w.hb * kHB);
  // Chunked work items: a finished split -> a parked slot as the finished partial: fp32 LSEs of the head slots,
  // then normalised rows in mid_dtype.  A lane holds eight consecutive dims of head 16*nb + c per i.
  auto park_final = [&](char* slot) {
    wave_lds_fence();
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float lsum = l[nb];
      lsum += __shfl_xor(lsum, 16);
      lsum += __shfl_xor(lsum, 32);
      const int h = 16 * nb + c;
      if (h < nheads) {
        const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) v[j] = acc[nb][j][i] * inv;
          park_store8(slot + kHB * 4, h * kD + 32 * g + 8 * i, a.mid_dtype, v);
        }
        if (g == 0) ((float*)slot)[h] = lsum > 0.f ? (m[nb] + fd_log2(lsum)) * FD_LN2 : -INFINITY;
      }
    }
  };

  if constexpr (CHUNK) {
    // Wave-uniform cursors over the tiles of the wave's splits: a tile starts at `base` inside a split that ends at
    // `end`; the tile after the last one of a split is the first one of the next split (splits are `per` tokens apart,
    // only the last non-empty one may be shorter).  The cursor stops on the wave's last tile.
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
      fetch_rows(pg0, slot0);
      issue_k();
      issue_v(std::integral_constant<int, 0>{});
      __builtin_amdgcn_sched_barrier(0);
      auto lookup2 = [&](int& slot) -> int { return token_slot(look.base, look.end, slot); };
      while (!(cur.end >= run_end && cur.base + kTile >= cur.end)) {   // all tiles but the wave's last one
        tile(cur.base, cur.end, lookup2, std::true_type{}, std::integral_constant<int, 0>{});
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
      tile(cur.base, cur.end, lookup2, std::false_type{}, std::integral_constant<int, 0>{});
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
      // same request order as in the loop (table entry of the next tile before the K/V rows), so the
      // wait counts at the loop head are exact on the first iteration as well
      __builtin_amdgcn_sched_barrier(0);
      fetch_rows(pg0, slot0);
      issue_k();
      issue_v(std::integral_constant<int, 0>{});
      __builtin_amdgcn_sched_barrier(0);
      using Set0 = std::integral_constant<int, 0>;
      using Set1 = std::integral_constant<int, VB - 1>;   // the other V register set, if there is one
      auto inner = [&](int t, auto set_tag) {   // a tile that has a successor
        tile(w.start + t * kTile, w.end, [&](int& slot) -> int { return tile_slot(min(t + 2, t1 - 1), slot); },
             std::true_type{}, set_tag);
      };
      auto last = [&](auto set_tag) {
        tile(w.start + (t1 - 1) * kTile, w.end, [&](int& slot) -> int { return tile_slot(t1 - 1, slot); },
             std::false_type{}, set_tag);
      };
      if constexpr (VEARLY) {
        int t = t0;
        for (; t + 2 < t1; t += 2) {
          inner(t, Set0{});
          inner(t + 1, Set1{});
        }
        if (t + 1 < t1) {   // two tiles left
          inner(t, Set0{});
          last(Set1{});
        } else {
          last(Set0{});
        }
      } else {
        for (int t = t0; t < t1 - 1; ++t) inner(t, Set0{});
        last(Set0{});
      }
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
  if (nb == 2) return soft_cap ? fd_split_mfma16_kernel<T, true, 2, CHUNK> : fd_split_mfma16_kernel<T, false, 2, CHUNK>;
  return soft_cap ? fd_split_mfma16_kernel<T, true, 1, CHUNK> : fd_split_mfma16_kernel<T, false, 1, CHUNK>;
}
template <typename T>
static auto pick_kernel(bool soft_cap, int nb, bool chunk) -> void (*)(const SplitArgs) {
  return chunk ? pick_kernel2<T, true>(soft_cap, nb) : pick_kernel2<T, false>(soft_cap, nb);
}

// a.hbsz = query heads per head block: up to 16 (one MFMA column block per wave) or 32 (two)
int fd_launch_split_mfma(hipStream_t stream, const SplitArgs& a, int kv_dtype, int waves, bool soft_cap) {
  const dim3 grid = fd_split_grid(a);
  const unsigned block = 64u * waves;
  const int nb = a.hbsz > 16 ? 2 : 1;
  size_t lds = (size_t)waves * wave_lds(nb);
  if (a.chunk > 1) lds += (size_t)waves * a.park * a.park_bytes;   // parked partials
  if (a.tickets) {  // the fused combine stages (S + num_extra) LSEs per head in LDS
    const size_t need = (size_t)(a.S + a.num_extra) * 16 * nb * 4;
    if (need > lds) lds = need;
  }
  void (*kern)(const SplitArgs) = nullptr;
  if (kv_dtype == FD_BF16) {
    kern = pick_kernel<__bf16>(soft_cap, nb, a.chunk > 1);
  } else if (kv_dtype == FD_F16) {
    kern = pick_kernel<_Float16>(soft_cap, nb, a.chunk > 1);
  } else {
    return FD_ERR_UNSUPPORTED;
  }
  if (lds > 64 * 1024) {
    // more than the default 64 KB of dynamic LDS per workgroup (gfx950 has 160 KB per CU)
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return FD_ERR_LAUNCH;
  }
  hipLaunchKernelGGL(kern, grid, dim3(block), lds, stream, a);
  return hipGetLastError() == hipSuccess ? FD_OK : FD_ERR_LAUNCH;
}
