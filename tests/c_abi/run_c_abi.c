/*
 * A consumer of the C ABI with no Python in the loop: fills a small paged decode problem, runs fd_decode (and
 * fd_decode_planned, fd_decode_noalloc, fd_schedule, fd_plan_splits, fd_kv_append) from libflash_decode_gfx950.so on the GPU and checks the result
 * against the plain-C oracle (oracle/c/ref_decode.c).  Exit code 0 = all checks passed.
 *
 *   gcc -O2 -std=c11 -D__HIP_PLATFORM_AMD__ tests/c_abi/run_c_abi.c oracle/c/ref_decode.c -Iinclude -I/opt/rocm/include \
 *       -Ltriton-distributed_amd -lflash_decode_gfx950 -L/opt/rocm/lib -lamdhip64 -lm -o tests/c_abi/run_c_abi
 */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "flash_decode.h"

int ref_paged_decode_f32(const float* q, const float* k_cache, const float* v_cache, const int32_t* block_table,
                         const int32_t* kv_lens, int32_t batch, int32_t q_heads, int32_t kv_heads, int32_t head_dim,
                         int32_t page_size, int32_t num_pages, int32_t max_pages, float scale, float soft_cap,
                         float* out, float* lse);

#define HIP_OK(x)                                                                  \
  do {                                                                             \
    hipError_t e_ = (x);                                                           \
    if (e_ != hipSuccess) {                                                        \
      fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_));   \
      return 2;                                                                    \
    }                                                                              \
  } while (0)
#define FD_OK_OR_DIE(x)                                                            \
  do {                                                                             \
    int s_ = (x);                                                                  \
    if (s_ != FD_OK) {                                                             \
      fprintf(stderr, "%s:%d: status %d: %s\n", __FILE__, __LINE__, s_, fd_last_error()); \
      return 3;                                                                    \
    }                                                                              \
  } while (0)

static uint32_t rng_state = 12345u;
static float frand(void) {  /* uniform in [-1, 1), a fixed sequence */
  rng_state = rng_state * 1664525u + 1013904223u;
  return (float)((rng_state >> 8) & 0xFFFF) / 32768.0f - 1.0f;
}

static void* to_device(const void* host, size_t bytes) {
  void* d = NULL;
  if (hipMalloc(&d, bytes) != hipSuccess) return NULL;
  if (hipMemcpy(d, host, bytes, hipMemcpyHostToDevice) != hipSuccess) return NULL;
  return d;
}

int main(void) {
  enum { B = 3, HQ = 8, HKV = 2, D = 128, P = 16, MAXP = 8, PAGES = 3 * MAXP + 1, S = 4 };
  const int32_t kv_lens[B] = {101, 0, 37};
  const float scale = 0.08838834764f, soft_cap = 30.0f;
  if (fd_abi_version() != FD_ABI_VERSION) {
    fprintf(stderr, "ABI version %d != header %d\n", fd_abi_version(), FD_ABI_VERSION);
    return 1;
  }

  const size_t nq = (size_t)B * HQ * D, nkv = (size_t)PAGES * P * HKV * D;
  float* q = (float*)malloc(nq * 4);
  float* k = (float*)malloc(nkv * 4);
  float* v = (float*)malloc(nkv * 4);
  int32_t bt[B * MAXP];
  for (size_t i = 0; i < nq; ++i) q[i] = 2.0f * frand();
  for (size_t i = 0; i < nkv; ++i) k[i] = 2.0f * frand();
  for (size_t i = 0; i < nkv; ++i) v[i] = 2.0f * frand();
  for (int i = 0; i < B * MAXP; ++i) bt[i] = (i * 7 + 3) % PAGES;   /* a fixed scatter, pages shared on purpose */

  float* ref_out = (float*)malloc(nq * 4);
  float ref_lse[B * HQ];
  if (ref_paged_decode_f32(q, k, v, bt, kv_lens, B, HQ, HKV, D, P, PAGES, MAXP, scale, soft_cap, ref_out, ref_lse)) return 1;

  void *dq = to_device(q, nq * 4), *dk = to_device(k, nkv * 4), *dv = to_device(v, nkv * 4);
  void *dbt = to_device(bt, sizeof(bt)), *dlens = to_device(kv_lens, sizeof(kv_lens));
  void *dmid = NULL, *dout = NULL, *dlse = NULL, *dorder = NULL;
  if (!dq || !dk || !dv || !dbt || !dlens) return 2;
  HIP_OK(hipMalloc(&dmid, (size_t)B * HQ * S * (D + 1) * 4));
  HIP_OK(hipMalloc(&dout, nq * 4));
  HIP_OK(hipMalloc(&dlse, sizeof(ref_lse)));
  HIP_OK(hipMalloc(&dorder, B * 4));

  fd_params p;
  memset(&p, 0, sizeof(p));
  p.q_heads = HQ; p.kv_heads = HKV; p.head_dim = D; p.page_size = P; p.num_splits = S; p.num_pages = PAGES;
  p.max_pages_per_seq = MAXP; p.q_dtype = FD_F32; p.kv_dtype = FD_F32; p.mid_dtype = FD_F32; p.out_dtype = FD_F32;
  p.soft_cap = soft_cap;
  const int planned = fd_plan_splits(&p, B);
  if (planned < 1 || planned > S) { fprintf(stderr, "fd_plan_splits -> %d\n", planned); return 1; }

  FD_OK_OR_DIE(fd_schedule(NULL, (const int32_t*)dlens, B, (int32_t*)dorder));
  FD_OK_OR_DIE(fd_decode(NULL, dq, dk, dv, dmid, NULL, dout, (float*)dlse, scale, (const int32_t*)dbt,
                         (const int32_t*)dlens, B, (int64_t)HQ * D, D, (int64_t)HKV * D, D, (int64_t)HKV * D, D,
                         (int64_t)HQ * S * (D + 1), (int64_t)S * (D + 1), D + 1, MAXP, (int64_t)HQ * D, D,
                         (const int32_t*)dorder, FD_COMBINE_SPLIT, NULL, NULL, 0, NULL, &p));
  HIP_OK(hipDeviceSynchronize());
  float* out = (float*)malloc(nq * 4);
  float lse[B * HQ];
  int32_t order[B];
  HIP_OK(hipMemcpy(out, dout, nq * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(lse, dlse, sizeof(lse), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(order, dorder, sizeof(order), hipMemcpyDeviceToHost));

  int bad = 0;
  if (order[0] != 0 || order[1] != 2 || order[2] != 1) { fprintf(stderr, "order %d %d %d\n", order[0], order[1], order[2]); ++bad; }
  double worst = 0.0;
  for (size_t i = 0; i < nq; ++i) {
    const double e = fabs((double)out[i] - (double)ref_out[i]);
    if (e > worst) worst = e;
    if (!(e <= 2e-4)) ++bad;
  }
  for (int i = 0; i < B * HQ; ++i) {
    if (isinf(ref_lse[i])) { if (!(isinf(lse[i]) && lse[i] < 0)) ++bad; continue; }
    if (!(fabs((double)lse[i] - (double)ref_lse[i]) <= 1e-5 * fmax(1.0, fabs((double)ref_lse[i])))) ++bad;
  }
  printf("fd_decode (fp32, soft cap, scheduled, %d planned of %d splits): max |out - ref| = %.3e\n", planned, S, worst);

  /* the planned step: the library picks splits, ranges, partial type and issue order; the caller only brings a
     workspace of the size the library names -- the path a binding should take when nobody looks at the partials */
  {
    fd_decode_args a;
    memset(&a, 0, sizeof(a));
    a.params = p;
    a.params.num_splits = -1;   /* no hint */
    fd_launch_plan lp;
    FD_OK_OR_DIE(fd_plan_decode(&a.params, B, 0, FD_STEP_SCHEDULE, &lp));
    const int64_t need = fd_workspace_bytes(&a.params, B, 0, FD_STEP_SCHEDULE);
    if (need <= 0 || need != lp.workspace_bytes || lp.num_splits < 1 || lp.order_kind == FD_ORDER_NONE) {
      fprintf(stderr, "fd_workspace_bytes -> %lld (plan %lld, %d splits, order %d)\n", (long long)need,
              (long long)lp.workspace_bytes, lp.num_splits, lp.order_kind);
      return 1;
    }
    void *dws = NULL, *dout3 = NULL, *dlse3 = NULL;
    HIP_OK(hipMalloc(&dws, (size_t)need));
    HIP_OK(hipMalloc(&dout3, nq * 4));
    HIP_OK(hipMalloc(&dlse3, sizeof(ref_lse)));
    HIP_OK(hipMemset(dws, 0xff, (size_t)need));   /* the workspace's contents mean nothing: NaNs */
    a.q = dq; a.k_cache = dk; a.v_cache = dv; a.workspace = dws; a.workspace_bytes = need; a.out = dout3;
    a.lse_out = (float*)dlse3; a.block_table = (const int32_t*)dbt; a.kv_lens = (const int32_t*)dlens;
    a.stride_q_bs = (int64_t)HQ * D; a.stride_q_h = D; a.stride_k_tok = (int64_t)HKV * D; a.stride_k_h = D;
    a.stride_v_tok = (int64_t)HKV * D; a.stride_v_h = D; a.stride_table_bs = MAXP; a.stride_obs = (int64_t)HQ * D;
    a.stride_oh = D; a.sm_scale = scale; a.batch = B; a.combine_mode = FD_COMBINE_SPLIT; a.flags = FD_STEP_SCHEDULE;
    FD_OK_OR_DIE(fd_decode_planned(NULL, &a));
    HIP_OK(hipDeviceSynchronize());
    float* out3 = (float*)malloc(nq * 4);
    float lse3[B * HQ];
    HIP_OK(hipMemcpy(out3, dout3, nq * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(lse3, dlse3, sizeof(lse3), hipMemcpyDeviceToHost));
    double worst3 = 0.0;
    for (size_t i = 0; i < nq; ++i) {
      const double e = fabs((double)out3[i] - (double)ref_out[i]);
      if (e > worst3) worst3 = e;
      if (!(e <= 2e-4)) ++bad;
    }
    for (int i = 0; i < B * HQ; ++i) {
      if (isinf(ref_lse[i])) { if (!(isinf(lse3[i]) && lse3[i] < 0)) ++bad; continue; }
      if (!(fabs((double)lse3[i] - (double)ref_lse[i]) <= 1e-5 * fmax(1.0, fabs((double)ref_lse[i])))) ++bad;
    }
    printf("fd_decode_planned (%d splits, workspace %lld bytes, order kind %d): max |out - ref| = %.3e\n", lp.num_splits,
           (long long)need, lp.order_kind, worst3);
    /* a workspace that is too small is refused with the size in the message, nothing is launched */
    a.workspace_bytes = need - 1;
    if (fd_decode_planned(NULL, &a) != FD_ERR_INVALID_ARG || strstr(fd_last_error(), "workspace") == NULL) ++bad;
  }

  /* the entry point that allocates nothing (partials in the library's static device array): the same bits */
  void *dout2 = NULL, *dlse2 = NULL;
  HIP_OK(hipMalloc(&dout2, nq * 4));
  HIP_OK(hipMalloc(&dlse2, sizeof(ref_lse)));
  FD_OK_OR_DIE(fd_decode_noalloc(NULL, dq, dk, dv, dout2, (float*)dlse2, scale, (const int32_t*)dbt, (const int32_t*)dlens, B,
                                 (int64_t)HQ * D, D, (int64_t)HKV * D, D, (int64_t)HKV * D, D, MAXP, (int64_t)HQ * D, D,
                                 (const int32_t*)dorder, FD_COMBINE_SPLIT, NULL, NULL, 0, &p));
  HIP_OK(hipDeviceSynchronize());
  float* out2 = (float*)malloc(nq * 4);
  float lse2[B * HQ];
  HIP_OK(hipMemcpy(out2, dout2, nq * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(lse2, dlse2, sizeof(lse2), hipMemcpyDeviceToHost));
  if (memcmp(out, out2, nq * 4) != 0 || memcmp(lse, lse2, sizeof(lse)) != 0) { fprintf(stderr, "fd_decode_noalloc differs from fd_decode\n"); ++bad; }
  if (fd_build_id() == NULL || strlen(fd_build_id()) == 0) { fprintf(stderr, "fd_build_id is empty\n"); ++bad; }
  printf("fd_decode_noalloc: bit-identical to fd_decode = %s; library build id %s\n", bad ? "no" : "yes", fd_build_id());

  /* the write side: append one token per sequence (fp32 -> fp32 is a copy) and read it back */
  float knew[B * HKV * D], vnew[B * HKV * D];
  for (int i = 0; i < B * HKV * D; ++i) { knew[i] = frand(); vnew[i] = frand(); }
  void *dkn = to_device(knew, sizeof(knew)), *dvn = to_device(vnew, sizeof(vnew)), *dlens2 = NULL;
  if (!dkn || !dvn) return 2;
  HIP_OK(hipMalloc(&dlens2, sizeof(kv_lens)));
  FD_OK_OR_DIE(fd_kv_append(NULL, dkn, dvn, dk, dv, (const int32_t*)dbt, (const int32_t*)dlens, (int32_t*)dlens2, NULL, B, 1,
                            (int64_t)HKV * D, (int64_t)HKV * D, D, (int64_t)HKV * D, (int64_t)HKV * D, D,
                            (int64_t)HKV * D, D, (int64_t)HKV * D, D, MAXP, NULL, &p));
  HIP_OK(hipDeviceSynchronize());
  int32_t lens2[B];
  HIP_OK(hipMemcpy(lens2, dlens2, sizeof(lens2), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(k, dk, nkv * 4, hipMemcpyDeviceToHost));
  for (int b = 0; b < B; ++b) {
    if (lens2[b] != kv_lens[b] + 1) ++bad;
    const int n = kv_lens[b], page = bt[b * MAXP + n / P];
    const float* row = k + (((size_t)page * P + n % P) * HKV) * D;
    if (memcmp(row, knew + (size_t)b * HKV * D, sizeof(float) * HKV * D) != 0) ++bad;
  }
  /* an invalid call reports, it does not abort */
  p.head_dim = 100;
  if (fd_decode(NULL, dq, dk, dv, dmid, NULL, dout, NULL, scale, (const int32_t*)dbt, (const int32_t*)dlens, B, HQ * D, D,
                HKV * D, D, HKV * D, D, HQ * S * (D + 1), S * (D + 1), D + 1, MAXP, HQ * D, D, NULL, FD_COMBINE_SPLIT,
                NULL, NULL, 0, NULL, &p) != FD_ERR_UNSUPPORTED || strstr(fd_last_error(), "head_dim") == NULL)
    ++bad;
  printf("%s\n", bad ? "FAILED" : "PASSED");
  return bad ? 1 : 0;
}
