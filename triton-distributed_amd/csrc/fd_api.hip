// extern "C" entry points of libflash_decode_gfx950.so: argument validation,
// kernel selection and launch.  Declarations and the reference interfaces they
// replace are in include/flash_decode.h.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "fd_common.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int dtype_size(int dt) {
  switch (dt) {
    case FD_F32: return 4;
    case FD_F16:
    case FD_BF16: return 2;
    case FD_FP8_E4M3: return 1;
    default: return 0;
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int ilog2_exact(int x) {
  if (x <= 0 || (x & (x - 1))) return -1;
  int r = 0;
  while ((1 << r) < x) ++r;
  return r;
}

// Waves per workgroup when the caller does not choose: enough waves to put
// about 8 on every CU (256 CUs), but never more waves than 32-token tiles a
// split can have.
int choose_waves(int64_t workgroups, int64_t max_tokens_per_split, int tile) {
  int64_t tiles = (max_tokens_per_split + tile - 1) / tile;
  int w = 1;
  while (w < 8 && workgroups * w < 2048 && w * 2 <= tiles) w *= 2;
  const char* env = getenv("FD_WAVES_PER_BLOCK");
  if (env) {
    int e = atoi(env);
    if (e == 1 || e == 2 || e == 4 || e == 8) w = e;
  }
  return w;
}

}  // namespace

extern "C" {

const char* fd_last_error(void) { return g_err; }

int fd_abi_version(void) { return FD_ABI_VERSION; }

int fd_split_kv(void* stream, const void* q, const void* k_cache, const void* v_cache, void* out_split,
                float* lse_split, float sm_scale, const int32_t* block_table, const int32_t* kv_lens, int32_t batch,
                int64_t stride_q_bs, int64_t stride_q_h, int64_t stride_k_tok, int64_t stride_k_h,
                int64_t stride_v_tok, int64_t stride_v_h, int64_t stride_o_bs, int64_t stride_o_h,
                int64_t stride_o_split, int64_t stride_table_bs, const int32_t* seq_order, const fd_params* p) {
  if (!p) return fail(FD_ERR_INVALID_ARG, "fd_split_kv: params is NULL");
  if (!q || !k_cache || !v_cache || !out_split || !block_table || !kv_lens)
    return fail(FD_ERR_INVALID_ARG, "fd_split_kv: NULL tensor pointer");
  if (batch < 0) return fail(FD_ERR_INVALID_ARG, "fd_split_kv: batch = %d", batch);
  if (batch == 0) return FD_OK;
  if (p->q_heads <= 0 || p->kv_heads <= 0 || p->q_heads % p->kv_heads != 0)
    return fail(FD_ERR_INVALID_ARG, "fd_split_kv: q_heads %d must be a positive multiple of kv_heads %d", p->q_heads,
                p->kv_heads);
  if (p->page_size <= 0 || p->num_splits <= 0 || p->num_pages <= 0 || p->max_pages_per_seq <= 0)
    return fail(FD_ERR_INVALID_ARG, "fd_split_kv: page_size/num_splits/num_pages/max_pages_per_seq must be > 0");
  if ((int64_t)p->num_pages * p->page_size >= (int64_t)1 << 31)
    return fail(FD_ERR_TOO_LARGE, "fd_split_kv: pool of %lld token rows exceeds 2^31",
                (long long)p->num_pages * p->page_size);
  if ((int64_t)p->max_pages_per_seq * p->page_size >= (int64_t)1 << 31)
    return fail(FD_ERR_TOO_LARGE, "fd_split_kv: block table capacity exceeds 2^31 tokens");
  const int D = p->head_dim;
  if (D != 64 && D != 128 && D != 256) return fail(FD_ERR_UNSUPPORTED, "fd_split_kv: head_dim %d (64/128/256)", D);
  const int qsz = dtype_size(p->q_dtype), kvsz = dtype_size(p->kv_dtype), msz = dtype_size(p->mid_dtype);
  if (!qsz || p->q_dtype == FD_FP8_E4M3) return fail(FD_ERR_UNSUPPORTED, "fd_split_kv: q_dtype %d", p->q_dtype);
  if (!kvsz) return fail(FD_ERR_UNSUPPORTED, "fd_split_kv: kv_dtype %d", p->kv_dtype);
  if (!msz || p->mid_dtype == FD_FP8_E4M3) return fail(FD_ERR_UNSUPPORTED, "fd_split_kv: mid_dtype %d", p->mid_dtype);
  if (p->kv_dtype == FD_FP8_E4M3 && (!p->k_scale || !p->v_scale))
    return fail(FD_ERR_INVALID_ARG, "fd_split_kv: fp8 KV cache needs k_scale and v_scale");
  const int kv_elems16 = 16 / kvsz;
  if (!aligned16(k_cache) || !aligned16(v_cache) || stride_k_tok % kv_elems16 || stride_k_h % kv_elems16 ||
      stride_v_tok % kv_elems16 || stride_v_h % kv_elems16)
    return fail(FD_ERR_ALIGNMENT, "fd_split_kv: K/V rows must be 16-byte aligned (pointer and token/head strides)");
  if (stride_k_tok <= 0 || stride_v_tok <= 0 || stride_k_tok * kvsz >= ((int64_t)1 << 31) ||
      stride_v_tok * kvsz >= ((int64_t)1 << 31))
    return fail(FD_ERR_INVALID_ARG, "fd_split_kv: token stride out of range");
  const int G = p->q_heads / p->kv_heads;
  const int64_t max_tok_split = ((int64_t)p->max_pages_per_seq * p->page_size + p->num_splits - 1) / p->num_splits;

  SplitArgs a;
  memset(&a, 0, sizeof(a));
  a.q = q; a.k = k_cache; a.v = v_cache; a.out = out_split; a.lse = lse_split;
  a.bt = block_table; a.kv_lens = kv_lens; a.order = seq_order;
  a.k_scale = p->k_scale; a.v_scale = p->v_scale;
  a.sq_b = stride_q_bs; a.sq_h = stride_q_h; a.sk_t = stride_k_tok; a.sk_h = stride_k_h;
  a.sv_t = stride_v_tok; a.sv_h = stride_v_h; a.so_b = stride_o_bs; a.so_h = stride_o_h; a.so_s = stride_o_split;
  a.sbt = stride_table_bs;
  a.sm_scale = sm_scale; a.soft_cap = p->soft_cap > 0.f ? p->soft_cap : 0.f;
  a.batch = batch; a.Hq = p->q_heads; a.Hkv = p->kv_heads; a.G = G; a.S = p->num_splits; a.P = p->page_size;
  a.log2P = ilog2_exact(p->page_size);
  a.max_pages = p->max_pages_per_seq; a.num_pages = p->num_pages;
  a.q_dtype = p->q_dtype; a.mid_dtype = p->mid_dtype;
  a.vec_out = (p->mid_dtype == FD_F32 && aligned16(out_split) && stride_o_bs % 4 == 0 && stride_o_h % 4 == 0 &&
               stride_o_split % 4 == 0) ? 1 : 0;

  const bool mfma_ok = D == 128 && G >= 4 && (G <= 16 || G % 16 == 0) &&
                       (p->kv_dtype == FD_BF16 || p->kv_dtype == FD_F16) && p->q_dtype == p->kv_dtype &&
                       aligned16(q) && stride_q_bs % 8 == 0 && stride_q_h % 8 == 0;
  bool use_mfma = mfma_ok;
  if (p->path == FD_PATH_VALU) use_mfma = false;
  if (p->path == FD_PATH_MFMA && !mfma_ok)
    return fail(FD_ERR_UNSUPPORTED,
                "fd_split_kv: MFMA path needs head_dim 128, group >= 4 (<= 16 or a multiple of 16), 16-bit KV of the "
                "query's dtype and 16-byte aligned q rows");
  if (p->waves_per_block != 0 && p->waves_per_block != 1 && p->waves_per_block != 2 && p->waves_per_block != 4 &&
      p->waves_per_block != 8)
    return fail(FD_ERR_INVALID_ARG, "fd_split_kv: waves_per_block %d (0, 1, 2, 4 or 8)", p->waves_per_block);

  int rc;
  if (use_mfma) {
    a.hbsz = G < 16 ? G : 16;
    a.nhb = (G + 15) / 16;
    const int64_t wgs = (int64_t)batch * a.S * a.Hkv * a.nhb;
    if (wgs >= ((int64_t)1 << 31)) return fail(FD_ERR_TOO_LARGE, "fd_split_kv: %lld workgroups", (long long)wgs);
    const int waves = p->waves_per_block ? p->waves_per_block : choose_waves(wgs, max_tok_split, 32);
    rc = fd_launch_split_mfma((hipStream_t)stream, a, p->kv_dtype, waves, a.soft_cap > 0.f);
  } else {
    a.hbsz = G >= 4 ? 4 : (G >= 2 ? 2 : 1);
    if (G == 3) a.hbsz = 4;
    a.nhb = (G + a.hbsz - 1) / a.hbsz;
    const int64_t wgs = (int64_t)batch * a.S * a.Hkv * a.nhb;
    if (wgs >= ((int64_t)1 << 31)) return fail(FD_ERR_TOO_LARGE, "fd_split_kv: %lld workgroups", (long long)wgs);
    const int tile = 4 * (64 / (D * kvsz / 16));
    const int waves = p->waves_per_block ? p->waves_per_block : choose_waves(wgs, max_tok_split, tile);
    rc = fd_launch_split_valu((hipStream_t)stream, a, p->kv_dtype, D, waves);
  }
  if (rc == FD_ERR_LAUNCH) return fail(rc, "fd_split_kv: launch failed: %s", hipGetErrorString(hipGetLastError()));
  if (rc != FD_OK) return fail(rc, "fd_split_kv: no kernel for kv_dtype %d, head_dim %d, group %d", p->kv_dtype, D, G);
  return FD_OK;
}

int fd_combine(void* stream, const void* mid_o, const float* mid_lse, void* out, float* lse_out,
               const int32_t* seqlens, int32_t batch, int32_t q_heads, int32_t num_partials, int64_t stride_mid_ob,
               int64_t stride_mid_oh, int64_t stride_mid_os, int64_t stride_obs, int64_t stride_oh, int32_t mode,
               const void* extra_out, const float* extra_lse, int32_t num_extra, const fd_params* p) {
  if (!p) return fail(FD_ERR_INVALID_ARG, "fd_combine: params is NULL");
  if (!mid_o || !out || !seqlens) return fail(FD_ERR_INVALID_ARG, "fd_combine: NULL tensor pointer");
  if (batch < 0 || q_heads <= 0 || num_partials <= 0 || num_extra < 0)
    return fail(FD_ERR_INVALID_ARG, "fd_combine: batch %d, q_heads %d, num_partials %d, num_extra %d", batch, q_heads,
                num_partials, num_extra);
  if (batch == 0) return FD_OK;
  if (mode != FD_COMBINE_SPLIT && mode != FD_COMBINE_SPLIT_LSE && mode != FD_COMBINE_RANK)
    return fail(FD_ERR_INVALID_ARG, "fd_combine: mode %d", mode);
  if (num_extra > 0 && (!extra_out || !extra_lse))
    return fail(FD_ERR_INVALID_ARG, "fd_combine: num_extra > 0 needs extra_out and extra_lse");
  if (p->head_dim <= 0 || p->head_dim > 256) return fail(FD_ERR_UNSUPPORTED, "fd_combine: head_dim %d", p->head_dim);
  if (!dtype_size(p->mid_dtype) || p->mid_dtype == FD_FP8_E4M3 || !dtype_size(p->out_dtype) ||
      p->out_dtype == FD_FP8_E4M3)
    return fail(FD_ERR_UNSUPPORTED, "fd_combine: mid_dtype %d / out_dtype %d", p->mid_dtype, p->out_dtype);
  if ((int64_t)batch * q_heads >= ((int64_t)1 << 31)) return fail(FD_ERR_TOO_LARGE, "fd_combine: batch * q_heads");
  CombineArgs a;
  memset(&a, 0, sizeof(a));
  a.mid_o = mid_o; a.mid_lse = mid_lse; a.out = out; a.lse_out = lse_out; a.seqlens = seqlens;
  a.extra_out = extra_out; a.extra_lse = extra_lse;
  a.s_mb = stride_mid_ob; a.s_mh = stride_mid_oh; a.s_ms = stride_mid_os; a.s_ob = stride_obs; a.s_oh = stride_oh;
  a.batch = batch; a.Hq = q_heads; a.D = p->head_dim; a.num_partials = num_partials; a.num_extra = num_extra;
  a.mode = mode; a.mid_dtype = p->mid_dtype; a.out_dtype = p->out_dtype;
  int rc = fd_launch_combine((hipStream_t)stream, a);
  if (rc != FD_OK) return fail(rc, "fd_combine: launch failed: %s", hipGetErrorString(hipGetLastError()));
  return FD_OK;
}

int fd_schedule(void* stream, const int32_t* kv_lens, int32_t batch, int32_t* seq_order) {
  if (!kv_lens || !seq_order) return fail(FD_ERR_INVALID_ARG, "fd_schedule: NULL pointer");
  if (batch < 0) return fail(FD_ERR_INVALID_ARG, "fd_schedule: batch = %d", batch);
  if (batch == 0) return FD_OK;
  int rc = fd_launch_schedule((hipStream_t)stream, kv_lens, batch, seq_order);
  if (rc != FD_OK) return fail(rc, "fd_schedule: launch failed: %s", hipGetErrorString(hipGetLastError()));
  return FD_OK;
}

}  // extern "C"
