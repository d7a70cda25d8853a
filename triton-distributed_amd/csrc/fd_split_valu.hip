// Split-KV GQA paged decode with VALU dot products (gfx950).
//
// Replaces kernel_gqa_fwd_batch_decode_split_kv
// (python/triton_dist/kernels/nvidia/flash_decode.py:130-239) where the MFMA
// kernels do not apply: fp32 caches or queries, fp8 caches with head_dim 64,
// a cache dtype that differs from the query's -- and whenever the caller forces
// this path.
// Any KV dtype (fp32, fp16, bf16, fp8-e4m3 with per-head scales) is dequantised
// to fp32 in registers; all arithmetic is fp32.
//
// A cache row of one KV head (D elements) is read by LPR = D*sizeof/16 lanes
// with one 128-bit load each, so a wave covers TPI = 64/LPR whole rows per load
// instruction.  Each of the TPI lane groups runs its own online softmax over
// the tokens it sees (tokens rg, rg+TPI, ... of every tile) for up to GH query
// heads; lane groups are merged with bpermutes at the end of the split, waves
// of a workgroup through LDS.
//
// K and V head dims may differ (flash_decode.py:765-774 takes v_head_dim from the V cache, K_DIM / V_DIM :162-163):
// a V row then has its own geometry -- LPRV lanes per row, TPIV rows per load instruction -- so the token a lane
// group multiplies with V is not the token it scored; the probabilities move between the two geometries with
// bpermutes, and the running maximum is kept wave-wide so that one rescale factor serves both.
#include "fd_common.h"

namespace {

template <int KV>
struct KvTraits;
template <>
struct KvTraits<FD_F32> {
  static constexpr int E = 4;
  static __device__ __forceinline__ void cvt(const u32x4& r, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(r[i]);
  }
};
template <>
struct KvTraits<FD_BF16> {
  static constexpr int E = 8;
  static __device__ __forceinline__ void cvt(const u32x4& r, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(r[i] << 16);
      f[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
    }
  }
};
template <>
struct KvTraits<FD_F16> {
  static constexpr int E = 8;
  static __device__ __forceinline__ void cvt(const u32x4& r, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t w = r[i];  // bit_cast of a vector-element lvalue would read element 0
      f16x2 h = __builtin_bit_cast(f16x2, w);
      f[2 * i] = (float)h[0];
      f[2 * i + 1] = (float)h[1];
    }
  }
};
template <>
struct KvTraits<FD_FP8_E4M3> {
  static constexpr int E = 16;
  static __device__ __forceinline__ void cvt(const u32x4& r, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(r[i], false);
      f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(r[i], true);
      f[4 * i] = lo[0];
      f[4 * i + 1] = lo[1];
      f[4 * i + 2] = hi[0];
      f[4 * i + 3] = hi[1];
    }
  }
};

template <int KV, int D, int DV, int GH>
__global__ void __launch_bounds__(512) fd_split_valu_kernel(const SplitArgs a) {
  using Tr = KvTraits<KV>;
  constexpr int E = Tr::E;            // elements per 16-byte chunk
  constexpr int LPR = D / E;          // lanes per K row
  constexpr int TPI = 64 / LPR;       // K rows per load instruction
  constexpr int U = 4;                // K load instructions per tile
  constexpr int TILE = U * TPI;       // tokens per tile
  constexpr int LPRV = DV / E;        // the same for V rows of DV elements
  constexpr int TPIV = 64 / LPRV;
  constexpr int UV = TILE / TPIV;
  constexpr int ESZ = 16 / E;         // bytes per element
  constexpr int PART = (GH * DV + 2 * GH + 3) & ~3;  // floats per wave partial (16-byte multiple)
  constexpr bool SAME = D == DV;
  static_assert(LPR >= 1 && LPR <= 64 && TILE <= 64, "unsupported geometry");
  static_assert(LPRV >= 1 && LPRV <= 64 && UV >= 1 && UV * TPIV == TILE, "unsupported V geometry");

  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int rg = lane / LPR;          // lane group = row within a load instruction
  const int c = lane % LPR;           // chunk of the row
  const int rgv = lane / LPRV;        // the same in the geometry of the V rows
  const int cv = lane % LPRV;

  const WorkItem w = decode_work_item(a);   // this wave: KV head w.kvh, token sub-range w.sub of w.nsub
  if (w.skip) return;   // empty range, and the combine does not expect a partial from it
  const int ntok = w.end - w.start;
  const int ntiles = ntok > 0 ? (ntok + TILE - 1) / TILE : 0;
  const int tpw = div_uniform(ntiles + w.nsub - 1, w.nsub);
  const int t0 = w.sub * tpw;
  const int t1 = min(t0 + tpw, ntiles);

  const int head0 = w.kvh * a.G + w.hb * GH;
  const int nheads = min(GH, a.G - w.hb * GH);

  // q[h][c*E .. c*E+E) in fp32, pre-multiplied by the softmax scale (and the K dequant scale).
  float kq_scale = a.sm_scale;
  if (KV == FD_FP8_E4M3) kq_scale *= a.k_scale[w.kvh];   // the V scale multiplies the finished accumulators
  const bool softcap = a.soft_cap > 0.f;
  const float inv_cap = softcap ? 1.0f / a.soft_cap : 0.f;
  const float post = softcap ? 1.0f : FD_LOG2E;  // without soft-cap scores go straight to base 2
  float qf[GH][E];
#pragma unroll
  for (int h = 0; h < GH; ++h) {
    const int hh = min(h, nheads - 1);
    const int64_t off = (int64_t)w.b * a.sq_b + (int64_t)(head0 + hh) * a.sq_h + c * E;
#pragma unroll
    for (int e = 0; e < E; ++e) qf[h][e] = load_as_f32(a.q, off + e, a.q_dtype) * kq_scale * post;
  }

  const int32_t* bt_row = a.bt + (int64_t)w.b * a.sbt;
  const char* kbase = (const char*)a.k + ((int64_t)w.kvh * a.sk_h) * ESZ + c * 16;
  const char* vbase = (const char*)a.v + ((int64_t)w.kvh * a.sv_h) * ESZ + cv * 16;
  const int k_pitch = (int)(a.sk_t * ESZ);
  const int v_pitch = (int)(a.sv_t * ESZ);

  auto tile_rows = [&](int t) -> int {
    int n = w.start + t * TILE + (lane % TILE);
    n = min(n, w.end - 1);
    return token_row(a, bt_row, n);
  };

  float m[GH], l[GH], acc[GH][E];
#pragma unroll
  for (int h = 0; h < GH; ++h) {
    m[h] = -INFINITY;
    l[h] = 0.f;
#pragma unroll
    for (int e = 0; e < E; ++e) acc[h][e] = 0.f;
  }

  u32x4 kraw[U], vraw[UV];
  int rv_next = 0;
  auto issue = [&](int rv) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int row = __shfl(rv, u * TPI + rg);
      kraw[u] = load_stream_b128(kbase + (int64_t)row * k_pitch);
      if constexpr (SAME) vraw[u] = load_stream_b128(vbase + (int64_t)row * v_pitch);
    }
    if constexpr (!SAME) {
#pragma unroll
      for (int u = 0; u < UV; ++u) {
        const int row = __shfl(rv, u * TPIV + rgv);
        vraw[u] = load_stream_b128(vbase + (int64_t)row * v_pitch);
      }
    }
  };
  if (t0 < t1) {
    issue(tile_rows(t0));
    if (t0 + 1 < t1) rv_next = tile_rows(t0 + 1);
  }

  for (int t = t0; t < t1; ++t) {
    u32x4 kc[U], vc[UV];
#pragma unroll
    for (int u = 0; u < U; ++u) kc[u] = kraw[u];
#pragma unroll
    for (int u = 0; u < UV; ++u) vc[u] = vraw[u];
    if (t + 1 < t1) {
      issue(rv_next);
      if (t + 2 < t1) rv_next = tile_rows(t + 2);
    }
    const int n0 = w.start + t * TILE;
    float sc[GH][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float kf[E];
      Tr::cvt(kc[u], kf);
#pragma unroll
      for (int h = 0; h < GH; ++h) {
        float d = 0.f;
#pragma unroll
        for (int e = 0; e < E; ++e) d = fmaf(qf[h][e], kf[e], d);
#pragma unroll
        for (int o = 1; o < LPR; o <<= 1) d += __shfl_xor(d, o);
        if (softcap) d = fd_softcap(d, a.soft_cap, inv_cap) * FD_LOG2E;
        sc[h][u] = (n0 + u * TPI + rg < w.end) ? d : -INFINITY;
      }
    }
    float p[GH][U];
#pragma unroll
    for (int h = 0; h < GH; ++h) {
      float mx = sc[h][0];
#pragma unroll
      for (int u = 1; u < U; ++u) mx = fmaxf(mx, sc[h][u]);
      if (!SAME) {   // one maximum for the whole wave: the accumulators live in another lane geometry
#pragma unroll
        for (int o = LPR; o < 64; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
      }
      const float m_new = fmaxf(m[h], mx);
      // A lane group can see only masked tokens in the last tile: keep its state empty.
      const float m_use = m_new > -INFINITY ? m_new : 0.f;
      const float alpha = fd_exp2(m[h] - m_use);
      float ps = 0.f;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        p[h][u] = fd_exp2(sc[h][u] - m_use);
        ps += p[h][u];
      }
      l[h] = l[h] * alpha + ps;
#pragma unroll
      for (int e = 0; e < E; ++e) acc[h][e] *= alpha;
      m[h] = m_new;
    }
    if constexpr (SAME) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float vf[E];
        Tr::cvt(vc[u], vf);
#pragma unroll
        for (int h = 0; h < GH; ++h)
#pragma unroll
          for (int e = 0; e < E; ++e) acc[h][e] = fmaf(p[h][u], vf[e], acc[h][e]);
      }
    } else {
      // V load uv holds, for this lane, token uv * TPIV + rgv of the tile; its probability sits in the K geometry
      // at load u = token / TPI, lane group token % TPI (any lane of that group).
#pragma unroll
      for (int uv = 0; uv < UV; ++uv) {
        float vf[E];
        Tr::cvt(vc[uv], vf);
#pragma unroll
        for (int h = 0; h < GH; ++h) {
          float pv;
          if constexpr (TPIV >= TPI) {
            constexpr int R = TPIV / TPI;        // K loads that one V load spans
            const int src = (rgv % TPI) * LPR;
            pv = 0.f;
#pragma unroll
            for (int j = 0; j < R; ++j) {
              const float cand = __shfl(p[h][uv * R + j], src);
              pv = (rgv / TPI == j) ? cand : pv;
            }
          } else {
            constexpr int R = TPI / TPIV;        // V loads that one K load spans
            pv = __shfl(p[h][uv / R], ((uv % R) * TPIV + rgv) * LPR);
          }
#pragma unroll
          for (int e = 0; e < E; ++e) acc[h][e] = fmaf(pv, vf[e], acc[h][e]);
        }
      }
    }
  }

  // ---- merge the lane groups of the wave (all-reduce over lanes with equal chunk index)
#pragma unroll
  for (int h = 0; h < GH; ++h) {
    float M = m[h];
    float sf = 1.0f;
    if (SAME) {   // every lane group kept its own running maximum
#pragma unroll
      for (int o = LPR; o < 64; o <<= 1) M = fmaxf(M, __shfl_xor(M, o));
      sf = M > -INFINITY ? fd_exp2(m[h] - M) : 0.f;
    }
    float L = l[h] * sf;
#pragma unroll
    for (int o = LPR; o < 64; o <<= 1) L += __shfl_xor(L, o);
#pragma unroll
    for (int e = 0; e < E; ++e) {
      float x = acc[h][e] * sf;
#pragma unroll
      for (int o = LPRV; o < 64; o <<= 1) x += __shfl_xor(x, o);
      acc[h][e] = x;
    }
    m[h] = M;
    l[h] = L;
  }
  float* part = (float*)smem + wave * PART;
  if (rgv == 0) {
    const float v_scale = KV == FD_FP8_E4M3 ? a.v_scale[w.kvh] : 1.0f;   // V dequantisation, once
#pragma unroll
    for (int h = 0; h < GH; ++h) {
#pragma unroll
      for (int e = 0; e < E; ++e) part[h * DV + cv * E + e] = acc[h][e] * v_scale;
      if (cv == 0) {
        part[GH * DV + h] = m[h];
        part[GH * DV + GH + h] = l[h];
      }
    }
  }
  __syncthreads();
  cta_merge_store<GH, DV>(a, (float*)smem, PART, w, nheads);
  if (a.tickets) fused_combine<DV>(a, w, head0, nheads, (float*)smem);  // hpw == 1 when fused
}

template <int KV, int D, int DV>
int launch_kdv(hipStream_t stream, const SplitArgs& a, int waves) {
  const dim3 grid = fd_split_grid(a);
  const unsigned block = 64u * waves;
  void (*kern)(const SplitArgs) = nullptr;
  int gh = a.hbsz;
  if (gh == 1) kern = fd_split_valu_kernel<KV, D, DV, 1>;
  else if (gh == 2) kern = fd_split_valu_kernel<KV, D, DV, 2>;
  else if (gh == 4) kern = fd_split_valu_kernel<KV, D, DV, 4>;
  else return FD_ERR_UNSUPPORTED;
  size_t lds = (size_t)waves * ((gh * DV + 2 * gh + 3) & ~3) * 4;
  if (a.tickets) {  // the fused combine stages (S + num_extra) LSEs per head in LDS
    const size_t need = (size_t)(a.S + a.num_extra) * gh * 4;
    if (need > lds) lds = need;
  }
  if (lds > 64 * 1024) {
    // more than the default 64 KB of dynamic LDS per workgroup (gfx950 has 160 KB per CU)
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return FD_ERR_LAUNCH;
  }
  hipLaunchKernelGGL(kern, grid, dim3(block), lds, stream, a);
  return hipGetLastError() == hipSuccess ? FD_OK : FD_ERR_LAUNCH;
}

template <int KV, int D>
int launch_kd(hipStream_t stream, const SplitArgs& a, int v_head_dim, int waves) {
  if (v_head_dim == D) return launch_kdv<KV, D, D>(stream, a, waves);
  if constexpr (KV != FD_FP8_E4M3) {   // K and V head dims that differ: not for fp8 caches
    switch (v_head_dim) {
      case 64: return launch_kdv<KV, D, 64>(stream, a, waves);
      case 128: return launch_kdv<KV, D, 128>(stream, a, waves);
      case 256: return launch_kdv<KV, D, 256>(stream, a, waves);
    }
  }
  return FD_ERR_UNSUPPORTED;
}

template <int KV>
int launch_k(hipStream_t stream, const SplitArgs& a, int head_dim, int v_head_dim, int waves) {
  switch (head_dim) {
    case 64: return launch_kd<KV, 64>(stream, a, v_head_dim, waves);
    case 128: return launch_kd<KV, 128>(stream, a, v_head_dim, waves);
    case 256: return launch_kd<KV, 256>(stream, a, v_head_dim, waves);
    default: return FD_ERR_UNSUPPORTED;
  }
}

}  // namespace

int fd_launch_split_valu(hipStream_t stream, const SplitArgs& a, int kv_dtype, int head_dim, int v_head_dim, int waves) {
  switch (kv_dtype) {
    case FD_F32: return launch_k<FD_F32>(stream, a, head_dim, v_head_dim, waves);
    case FD_F16: return launch_k<FD_F16>(stream, a, head_dim, v_head_dim, waves);
    case FD_BF16: return launch_k<FD_BF16>(stream, a, head_dim, v_head_dim, waves);
    case FD_FP8_E4M3: return launch_k<FD_FP8_E4M3>(stream, a, head_dim, v_head_dim, waves);
    default: return FD_ERR_UNSUPPORTED;
  }
}
