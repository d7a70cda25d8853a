// LSE-weighted combine of split / rank partials, and the sequence scheduler (gfx950).
//
// fd_combine_kernel replaces the reference's three combine kernels
// (python/triton_dist/kernels/nvidia/flash_decode.py:308-360 plain, :393-449
// intra-rank with merged LSE, :482-532 inter-rank).  The reference walks the
// partials sequentially with a running max.  Here a 256-thread workgroup per
// (sequence, head, column chunk) first brings all partial LSEs into LDS (one
// load per thread), every thread derives M = max and the weights
// w_s = e^{LSE_s - M} from there, and then the threads -- laid out as ROWS row
// groups x CG column groups of 4 columns -- accumulate sum_s w_s * O_s with
// 128-bit loads that do not depend on each other.  The row groups are summed
// through LDS.  The value is the reference's: out = sum_s softmax(LSE)_s * O_s,
// LSE = logsumexp_s(LSE_s); the cost is two dependent memory round trips
// instead of S.  CG is chosen per launch: D/4 (one workgroup per row of the
// output) down to 4 (D/16 workgroups per row, 64 row groups), so that a step
// with few output rows and many partials (one long sequence, few heads)
// still spreads over the chip and needs few loads per thread.
#include "fd_common.h"

namespace {

constexpr int kCombineThreads = 256;
constexpr int kMaxPartials = 1024;  // LSEs staged in LDS per pass
constexpr int kPrefetch = 8;        // partial rows a thread requests before the weights are known

// max of v[0..n) (LDS), the same value in every lane: a strided scan per lane, then a butterfly over the wave
__device__ __forceinline__ float wave_max_of(const float* v, int n) {
  float m = -INFINITY;
  for (int i = threadIdx.x & 63; i < n; i += 64) m = fmaxf(m, v[i]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  return m;
}

template <int D>
__global__ void __launch_bounds__(kCombineThreads) fd_combine_kernel(const CombineArgs a) {
  const int CG = 1 << a.cg_shift;              // column groups of this workgroup (one 128-bit chunk of fp32 each)
  const int ROWS = kCombineThreads >> a.cg_shift;   // partial rows in flight per pass
  const int chunks = (D / 4) >> a.cg_shift;    // workgroups per output row (a power of two)
  __shared__ float s_lse[kMaxPartials];
  __shared__ __align__(16) float s_acc[kCombineThreads * 4];   // [ROWS][4 * CG]
  __shared__ float s_l[kCombineThreads / 4];                   // [ROWS], ROWS <= 64

  const int tid = threadIdx.x;
  const int row = blockIdx.x / chunks;
  const int col0 = (blockIdx.x - row * chunks) * 4 * CG;   // first column of this workgroup
  const int b = row / a.Hq;
  const int h = row - b * a.Hq;
  const int S = a.num_partials;
  const int NP = S + a.num_extra;
  const int64_t mid_base = (int64_t)b * a.s_mb + (int64_t)h * a.s_mh;

  // Partials written by this library's split kernel in the same call: every slot holds defined values (an
  // empty split is out = 0, lse = -inf), so validity needs no kv_lens and rows may be read before their weights
  // are known.
  const bool own = a.all_slots_written && a.mode != FD_COMBINE_RANK;
  int kv_len = 0, per = 0;
  if (a.mode != FD_COMBINE_RANK && !own) {
    kv_len = (int)min((int64_t)max(a.seqlens[b], 0), a.capacity);   // the length the split kernels worked with
    per = tokens_per_range(kv_len, S, a.s_magic, a.s_shift, a.per_mask, a.adapt);
  }
  // LSE of partial s, -inf when the partial is not valid
  auto partial_lse = [&](int s) -> float {
    if (s >= S) {   // extras: always valid, unless they stand for other ranks whose lengths say otherwise
      if (a.rank_lens) {
        const int e = s - S;
        if (a.rank_lens[(int64_t)(e < a.this_rank ? e : e + 1) * a.batch + b] <= 0) return -INFINITY;
      }
      return a.extra_lse[((int64_t)(s - S) * a.batch + b) * a.Hq + h];
    }
    if (a.mode == FD_COMBINE_RANK) {
      if (a.seqlens[(int64_t)s * a.batch + b] <= 0) return -INFINITY;
    } else if (!own && (int64_t)per * s >= kv_len) {  // empty split range
      return -INFINITY;
    }
    if (a.mid_lse) return a.mid_lse[((int64_t)b * a.Hq + h) * S + s];
    return load_as_f32(a.mid_o, mid_base + (int64_t)s * a.s_ms + D, a.mid_dtype);
  };

  const int r = tid >> a.cg_shift;
  const int c = col0 / 4 + (tid - (r << a.cg_shift));   // 128-bit column group within the row
  const bool vec_mid = a.vec_mid != 0;
  auto load_row = [&](int s) -> f32x4 {   // this thread's 4 columns of partial s
    f32x4 o;
    if (s < S) {
      const int64_t off = mid_base + (int64_t)s * a.s_ms + 4 * c;
      if (vec_mid && a.mid_dtype == FD_F32) {
        o = *(const f32x4*)((const float*)a.mid_o + off);
      } else if (vec_mid) {   // four packed 16-bit values in one 64-bit load
        const u32x2 w = *(const u32x2*)((const uint16_t*)a.mid_o + off);
        if (a.mid_dtype == FD_F16) {
          // halves taken apart as integers: with 2-element half vectors the compiler used the first dword twice
          o = f32x4{f16_bits_to_f32(w[0] & 0xffffu), f16_bits_to_f32(w[0] >> 16), f16_bits_to_f32(w[1] & 0xffffu),
                    f16_bits_to_f32(w[1] >> 16)};
        } else {
          o = f32x4{bf16_bits_to_f32(w[0] & 0xffffu), bf16_bits_to_f32(w[0] >> 16), bf16_bits_to_f32(w[1] & 0xffffu),
                    bf16_bits_to_f32(w[1] >> 16)};
        }
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) o[k] = load_as_f32(a.mid_o, off + k, a.mid_dtype);
      }
    } else {
      const int64_t off = (((int64_t)(s - S) * a.batch + b) * a.Hq + h) * D + 4 * c;
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = load_as_f32(a.extra_out, off + k, a.out_dtype);
    }
    return o;
  };
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float M = -INFINITY;  // running max over the passes (one pass unless NP > kMaxPartials)
  float L = 0.f;        // sum of the weights of this thread's rows
  // local_out: the merge of the S split partials alone goes there as well (this rank's slot of a staged buffer), with
  // weights relative to the maximum over those S, so that a far larger LSE among the extras cannot flush them to zero
  const bool two = a.local_out != nullptr;   // (the host admits it only with NP <= kMaxPartials: one pass)
  f32x4 acc_loc = {0.f, 0.f, 0.f, 0.f};
  float M_loc = -INFINITY, L_loc = 0.f;

  if (own && NP <= ROWS * kPrefetch) {
    // one dependent round trip: the rows are requested together with the LSEs
    f32x4 pre[kPrefetch];
#pragma unroll
    for (int p = 0; p < kPrefetch; ++p) {
      const int s = r + p * ROWS;
      pre[p] = s < NP ? load_row(s) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
    for (int i = tid; i < NP; i += kCombineThreads) s_lse[i] = partial_lse(i);
    __syncthreads();
    M = wave_max_of(s_lse, NP);
    if (two) M_loc = wave_max_of(s_lse, S);
    if (M > -INFINITY) {
#pragma unroll
      for (int p = 0; p < kPrefetch; ++p) {
        const int s = r + p * ROWS;
        const float wgt = s < NP ? __expf(s_lse[s] - M) : 0.f;
        if (wgt != 0.f) acc += pre[p] * wgt;   // (the row of an extra that does not count may hold anything)
        L += wgt;
        if (two && s < S && M_loc > -INFINITY) {
          const float wl = __expf(s_lse[s] - M_loc);
          acc_loc += pre[p] * wl;
          L_loc += wl;
        }
      }
    }
  } else {
    for (int p0 = 0; p0 < NP; p0 += kMaxPartials) {
      const int cnt = min(kMaxPartials, NP - p0);
      __syncthreads();
      for (int i = tid; i < cnt; i += kCombineThreads) s_lse[i] = partial_lse(p0 + i);
      __syncthreads();
      const float m_pass = wave_max_of(s_lse, cnt);
      const float m_new = fmaxf(M, m_pass);
      if (m_new == -INFINITY) continue;  // nothing valid so far (uniform)
      const float resc = __expf(M - m_new);  // 0 on the first valid pass
      acc *= resc;
      L *= resc;
      M = m_new;
      if (two) M_loc = wave_max_of(s_lse, min(cnt, S));
      for (int i = r; i < cnt; i += ROWS) {
        const float wgt = __expf(s_lse[i] - M);
        const float wl = two && i < S && M_loc > -INFINITY ? __expf(s_lse[i] - M_loc) : 0.f;
        if (wgt == 0.f && wl == 0.f) continue;
        const f32x4 row = load_row(p0 + i);
        if (wgt != 0.f) acc += row * wgt;
        L += wgt;
        if (wl != 0.f) acc_loc += row * wl;
        L_loc += wl;
      }
    }
  }
  // Sum over the ROWS row groups in two short steps instead of one thread per column walking all of them (64 dependent
  // LDS reads for a 16-column chunk): thread (g, col) adds the four rows g, g + NG, g + 2 NG, g + 3 NG of its column
  // (ROWS = 4 NG), the NG sums of a column go back through LDS, and the sum of the weights is a butterfly over one wave.
  const int ncol = 4 * CG;
  const int NG = kCombineThreads / ncol;        // = ROWS / 4
  const int col = tid & (ncol - 1);
  const int g = tid >> (a.cg_shift + 2);
  // dst / dst_base / dst_dtype: the output row; lse_col: the LSE goes to column D of it; lse_sep: and / or there
  auto reduce_store = [&](const f32x4 acc_t, const float L_t, const float M_t, void* dst, int64_t dst_base, int dst_dtype,
                          bool lse_col, float* lse_sep) {
    *(f32x4*)&s_acc[tid * 4] = acc_t;   // row r, columns 4 * (tid % CG) .. + 3 of the chunk
    if ((tid & (CG - 1)) == 0) s_l[r] = L_t;
    __syncthreads();
    float part4 = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) part4 += s_acc[(g + k * NG) * ncol + col];
    float lw = (tid & 63) < ROWS ? s_l[tid & 63] : 0.f;   // ROWS <= 64
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) lw += __shfl_xor(lw, off);
    __syncthreads();
    s_acc[g * ncol + col] = part4;
    __syncthreads();
    if (tid < ncol) {
      float o = 0.f;
      for (int i = 0; i < NG; ++i) o += s_acc[i * ncol + tid];
      const float Lsum = lw;
      const float inv = Lsum > 0.f ? 1.0f / Lsum : 0.f;
      store_from_f32(dst, dst_base + col0 + tid, dst_dtype, o * inv);
      if (tid == 0 && col0 == 0) {
        const float lse = Lsum > 0.f ? M_t + __logf(Lsum) : -INFINITY;
        if (lse_col) store_from_f32(dst, dst_base + D, dst_dtype, lse);
        if (lse_sep) *lse_sep = lse;
      }
    }
  };
  if (two) {
    reduce_store(acc_loc, L_loc, M_loc, a.local_out, (int64_t)b * a.s_lb + (int64_t)h * a.s_lh, a.local_dtype, true, nullptr);
    __syncthreads();
  }
  reduce_store(acc, L, M, a.out, (int64_t)b * a.s_ob + (int64_t)h * a.s_oh, a.out_dtype, a.mode == FD_COMBINE_SPLIT_LSE,
               a.lse_out ? a.lse_out + (int64_t)b * a.Hq + h : nullptr);
}

// Up to MAXP (16, 32 or 64) partials produced by this library's split kernel in the same call, rows readable four
// values at a time, LSEs in their own fp32 buffer: every slot is written (an empty split holds out = 0, lse = -inf),
// so validity needs no kv_lens, and the row loads do not wait for the LSEs -- both are requested at once, which
// leaves one dependent memory round trip.  The kernel is short on purpose: one workgroup per output row on a chip
// that the step's split kernel has just vacated runs at one wave per SIMD, where every instruction of the wave is
// latency.  Thread (r, c): partials r, r + ROWS, ... and 128-bit column chunk c.  Lane i of every wave loads LSE i
// (MAXP <= 64 = one per lane); the maximum is a butterfly over the wave and a thread takes the LSEs of its own
// partials from the lanes that hold them, so nothing goes through LDS before the final sum.
template <int D, int MAXP, int MID, bool VEC, int CG>
__global__ void __launch_bounds__(kCombineThreads) fd_combine_own_kernel(const CombineArgs a) {
  // CG column groups of four columns per workgroup: D / 4 = the whole output row (one workgroup per row), or fewer --
  // D / 4 / CG workgroups per row -- where a step has few output rows and many partials (one long sequence), so that
  // the chip sees at least a workgroup per CU and a thread walks few partials.
  constexpr int ROWS = kCombineThreads / CG;
  constexpr int PASSES = (MAXP + ROWS - 1) / ROWS;
  constexpr int CHUNKS = D / 4 / CG;
  constexpr int NCOL = 4 * CG;
  static_assert(MAXP <= 64, "one LSE per lane");
  static_assert(VEC || CG == D / 4, "column-strided rows come as whole rows");
  __shared__ __align__(16) float s_acc[ROWS][NCOL];
  __shared__ float s_l[ROWS];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int row = CHUNKS == 1 ? (int)blockIdx.x : (int)blockIdx.x / CHUNKS;
  const int col0 = CHUNKS == 1 ? 0 : ((int)blockIdx.x - row * CHUNKS) * NCOL;
  const int b = row / a.Hq;
  const int h = row - b * a.Hq;
  const int S = a.num_partials;
  const int64_t mid_base = (int64_t)b * a.s_mb + (int64_t)h * a.s_mh + col0;
  const int r = tid / CG;
  const int c = tid - r * CG;
  // VEC: rows start on multiples of four elements and a thread owns columns 4c .. 4c + 3 (one 128- or 64-bit load);
  // else (the reference's [.., D + 1] rows) it owns columns c, c + CG, c + 2 CG, c + 3 CG, so that consecutive
  // threads still read consecutive elements.
  f32x4 o[PASSES];
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int s = r + p * ROWS;
    o[p] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (s < S) {
      const int64_t off = mid_base + (int64_t)s * a.s_ms + (VEC ? 4 * c : c);
      if constexpr (!VEC) {
#pragma unroll
        for (int k = 0; k < 4; ++k) o[p][k] = load_as_f32(a.mid_o, off + k * CG, MID);
      } else if constexpr (MID == FD_F32) {
        o[p] = *(const f32x4*)((const float*)a.mid_o + off);
      } else {
        const u32x2 w = *(const u32x2*)((const uint16_t*)a.mid_o + off);
        if constexpr (MID == FD_F16) {
          o[p] = f32x4{f16_bits_to_f32(w[0] & 0xffffu), f16_bits_to_f32(w[0] >> 16), f16_bits_to_f32(w[1] & 0xffffu),
                       f16_bits_to_f32(w[1] >> 16)};
        } else {
          o[p] = f32x4{bf16_bits_to_f32(w[0] & 0xffffu), bf16_bits_to_f32(w[0] >> 16), bf16_bits_to_f32(w[1] & 0xffffu),
                       bf16_bits_to_f32(w[1] >> 16)};
        }
      }
    }
  }
  float mine = -INFINITY;   // LSE of partial `lane`: from its own buffer, or from column D of the partial's row
  if (lane < S) {
    mine = a.mid_lse ? a.mid_lse[((int64_t)b * a.Hq + h) * S + lane]
                     : load_as_f32(a.mid_o, mid_base - col0 + (int64_t)lane * a.s_ms + D, MID);
    // partials of other ranks: rank `lane` counts iff it holds tokens of this sequence (flash_decode.py:513-515);
    // what its slot holds otherwise is not looked at (the rows are requested, their values dropped below)
    if (a.mode == FD_COMBINE_RANK && a.seqlens[(int64_t)lane * a.batch + b] <= 0) mine = -INFINITY;
  }
  float M = mine;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off));
  float L = 0.f;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int s = r + p * ROWS;
    const float own = __shfl(mine, s & 63);          // -inf for empty and absent splits: weight 0
    const float wgt = M > -INFINITY && s < S ? __expf(own - M) : 0.f;
    if (wgt != 0.f) acc += o[p] * wgt;   // (a slot that does not count may hold anything, NaN included)
    L += wgt;
  }
  if constexpr (VEC) {
    *(f32x4*)&s_acc[r][4 * c] = acc;
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) s_acc[r][c + k * CG] = acc[k];
  }
  if (c == 0) s_l[r] = L;
  __syncthreads();
  if (tid < NCOL) {
    float v = 0.f, Lsum = 0.f;
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      v += s_acc[i][tid];
      Lsum += s_l[i];
    }
    const float inv = Lsum > 0.f ? 1.0f / Lsum : 0.f;
    const int64_t out_base = (int64_t)b * a.s_ob + (int64_t)h * a.s_oh;
    store_from_f32(a.out, out_base + col0 + tid, a.out_dtype, v * inv);
    if (tid == 0 && col0 == 0) {
      const float res = Lsum > 0.f ? M + __logf(Lsum) : -INFINITY;
      if (a.mode == FD_COMBINE_SPLIT_LSE) store_from_f32(a.out, out_base + D, a.out_dtype, res);
      if (a.lse_out) a.lse_out[(int64_t)b * a.Hq + h] = res;
    }
  }
}

// order[rank] = sequence index, sequences ranked by kv_len descending, ties by index (fd_rank_sequence).
__global__ void __launch_bounds__(256) fd_schedule_kernel(const int32_t* __restrict__ kv_lens, int batch, int t_shift,
                                                          int32_t* __restrict__ order) {
  __shared__ __align__(16) int32_t s_len[kRankChunk];
  const int gid = blockIdx.x * blockDim.x + threadIdx.x;
  int mine;
  const int rank = fd_rank_sequence(gid, batch, t_shift, [&](int j) { return kv_lens[j]; }, s_len, &mine);
  const int i = gid >> t_shift;
  if ((gid & ((1 << t_shift) - 1)) == 0 && i < batch) order[rank] = i;
}

// One workgroup: the (sequence, range) issue order of a decode step (fd_schedule_items_block).
__global__ void __launch_bounds__(kMaxItemBatch) fd_schedule_items_kernel(const int32_t* __restrict__ kv_lens, int batch,
                                                                        int64_t capacity, RangePlan ranges,
                                                                        int32_t* __restrict__ items) {
  __shared__ uint64_t s_key[kMaxItemBatch];
  __shared__ int32_t s_n[kMaxItemBatch];
  auto len_of = [&](int j) {
    const int64_t len = kv_lens[j];
    return (int)(len < 0 ? 0 : (len > capacity ? capacity : len));   // as the split kernels clamp it
  };
  fd_schedule_items_block(threadIdx.x, batch, len_of, ranges, items, s_key, s_n);
}

}  // namespace

int fd_launch_combine(hipStream_t stream, const CombineArgs& args) {
  CombineArgs a = args;
  const int64_t rows = (int64_t)a.batch * a.Hq;
  void (*kern)(const CombineArgs) = nullptr;
  // The short kernel: this library's own partials in the same call (all slots written) or the per-rank partials of the
  // inter-rank merge (validity by the ranks' lengths), at most 64 of them and no extras.  Rows that are readable four
  // values at a time are spread over several workgroups where the step has few output rows (one long sequence: 96
  // rows x 42 partials as 384 workgroups of 32 columns: 4.5 -> 3.1 us behind the split kernel against the general
  // kernel's run-time loops); the caller's [.., D + 1] rows come as whole rows.
  const int np_own = a.num_partials <= 16 ? 16 : (a.num_partials <= 32 ? 32 : 64);
  const bool small = (a.all_slots_written || a.mode == FD_COMBINE_RANK) && a.num_extra == 0 && !a.local_out &&
                     a.num_partials <= 64 && (a.vec_mid || a.num_partials <= 32 || rows >= 256);
  // Column groups per workgroup.  Start with the whole row (D/4) and halve while the grid is under one workgroup per
  // CU and a thread would still have more than two partials to walk (short kernel: down to 8 groups of four columns).
  int cg = a.D / 4;
  const int64_t np = (int64_t)a.num_partials + a.num_extra;
  const int cg_min = small ? 8 : 4;
  while ((!small || a.vec_mid) && cg > cg_min && rows * (a.D / 4 / cg) < 256 && np > 2 * (kCombineThreads / cg)) cg >>= 1;
  a.cg_shift = 0;
  while ((1 << a.cg_shift) < cg) ++a.cg_shift;
  const int64_t wgs = rows * (a.D / 4 / cg);
  if (wgs >= ((int64_t)1 << 31)) return FD_ERR_TOO_LARGE;
  const unsigned grid = (unsigned)wgs;
#define FD_OWN_N(D_, M_, V_, C_) (np_own == 16 ? fd_combine_own_kernel<D_, 16, M_, V_, C_> : np_own == 32 ? fd_combine_own_kernel<D_, 32, M_, V_, C_> : fd_combine_own_kernel<D_, 64, M_, V_, C_>)
#define FD_OWN_V(D_, M_) (!a.vec_mid ? FD_OWN_N(D_, M_, false, D_ / 4) : cg == D_ / 4 ? FD_OWN_N(D_, M_, true, D_ / 4) : \
                          cg == D_ / 8 ? FD_OWN_N(D_, M_, true, (D_ / 8 >= 8 ? D_ / 8 : 8)) : cg == 16 ? FD_OWN_N(D_, M_, true, 16) : FD_OWN_N(D_, M_, true, 8))
#define FD_OWN(D_) (a.mid_dtype == FD_F32 ? FD_OWN_V(D_, FD_F32) : a.mid_dtype == FD_F16 ? FD_OWN_V(D_, FD_F16) : FD_OWN_V(D_, FD_BF16))
  switch (a.D) {
    case 64: kern = small ? FD_OWN(64) : fd_combine_kernel<64>; break;
    case 128: kern = small ? FD_OWN(128) : fd_combine_kernel<128>; break;
    case 256: kern = small ? FD_OWN(256) : fd_combine_kernel<256>; break;
    default: return FD_ERR_UNSUPPORTED;
  }
#undef FD_OWN_N
#undef FD_OWN_V
#undef FD_OWN
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kCombineThreads), 0, stream, a);
  return hipGetLastError() == hipSuccess ? FD_OK : FD_ERR_LAUNCH;
}

int fd_launch_schedule(hipStream_t stream, const int32_t* kv_lens, int batch, int32_t* order) {
  const int t_shift = fd_rank_shift(batch);
  const unsigned grid = (unsigned)((((int64_t)batch << t_shift) + 255) / 256);
  hipLaunchKernelGGL(fd_schedule_kernel, dim3(grid), dim3(256), 0, stream, kv_lens, batch, t_shift, order);
  return hipGetLastError() == hipSuccess ? FD_OK : FD_ERR_LAUNCH;
}

int fd_launch_schedule_items(hipStream_t stream, const int32_t* kv_lens, int batch, int64_t capacity,
                             const RangePlan& ranges, int32_t* items) {
  if (batch > kMaxItemBatch) return FD_ERR_TOO_LARGE;
  unsigned threads = 256;   // the batch rounded up to a power of two; at least 256 to write the list
  while ((int)threads < batch) threads <<= 1;
  hipLaunchKernelGGL(fd_schedule_items_kernel, dim3(1), dim3(threads), 0, stream, kv_lens, batch, capacity, ranges, items);
  return hipGetLastError() == hipSuccess ? FD_OK : FD_ERR_LAUNCH;
}
