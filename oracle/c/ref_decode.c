/*
 * Plain-C restatement of the decode oracle.  TEST INFRASTRUCTURE ONLY: nothing in the shipped
 * library links or calls this file; the tests use it as a second, independent checker next to
 * oracle/ref_decode.py (which it must agree with) and the C consumer of the ABI under
 * tests/c_abi/ uses it where Python is not in the loop.
 *
 * Follows ref_paged_attn in python/triton_dist/test/nvidia/test_decode_attn.py:70-120: per
 * sequence, token n of the cache lives at page block_table[b][n / P], slot n % P
 * (lines 93-99); consecutive query heads share a KV head (repeat_interleave, 101-103);
 * scores = scale * q . k (105), optional soft cap cap * tanh(s / cap) (111-112), softmax over
 * the kv_len tokens (113), out = P . V (115).  Differences from that text, as in the Python
 * restatement: the query is not scaled in place, P is not rounded to V's dtype, and the
 * natural-log log-sum-exp of the scores is returned as well (what the kernels emit,
 * python/triton_dist/kernels/nvidia/flash_decode.py:239).  All arithmetic in double.
 *
 * Layouts (contiguous, fp32): q [B, Hq, D]; k_cache, v_cache [num_pages, P, Hkv, D];
 * block_table [B, max_pages] int32; kv_lens [B] int32; out [B, Hq, D]; lse [B, Hq].
 * A sequence with kv_len <= 0 yields out = 0, lse = -inf.  Page ids are clamped into the pool.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

#if defined(__GNUC__)
#define REF_API __attribute__((visibility("default")))
#else
#define REF_API
#endif

REF_API int ref_paged_decode_f32(const float* q, const float* k_cache, const float* v_cache,
                                 const int32_t* block_table, const int32_t* kv_lens, int32_t batch,
                                 int32_t q_heads, int32_t kv_heads, int32_t head_dim, int32_t page_size,
                                 int32_t num_pages, int32_t max_pages, float scale, float soft_cap, float* out,
                                 float* lse) {
  if (batch < 0 || q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads || head_dim <= 0 || page_size <= 0 ||
      num_pages <= 0 || max_pages <= 0)
    return -1;
  const int group = q_heads / kv_heads;
  const int64_t cap_tokens = (int64_t)max_pages * page_size;
  double* scores = NULL;
  int64_t scores_cap = 0;
  for (int b = 0; b < batch; ++b) {
    int64_t n_tok = kv_lens[b];
    if (n_tok < 0) n_tok = 0;
    if (n_tok > cap_tokens) n_tok = cap_tokens;
    if (n_tok > scores_cap) {
      free(scores);
      scores = (double*)malloc((size_t)n_tok * sizeof(double));
      if (!scores) return -2;
      scores_cap = n_tok;
    }
    for (int h = 0; h < q_heads; ++h) {
      const int kvh = h / group;
      const float* qv = q + ((int64_t)b * q_heads + h) * head_dim;
      float* o = out + ((int64_t)b * q_heads + h) * head_dim;
      for (int d = 0; d < head_dim; ++d) o[d] = 0.f;
      if (n_tok == 0) {
        lse[(int64_t)b * q_heads + h] = -INFINITY;
        continue;
      }
      double mx = -INFINITY;
      for (int64_t n = 0; n < n_tok; ++n) {
        int32_t page = block_table[(int64_t)b * max_pages + n / page_size];
        if (page < 0) page = 0;
        if (page >= num_pages) page = num_pages - 1;
        const float* kr = k_cache + (((int64_t)page * page_size + n % page_size) * kv_heads + kvh) * head_dim;
        double s = 0.0;
        for (int d = 0; d < head_dim; ++d) s += (double)qv[d] * (double)kr[d];
        s *= (double)scale;
        if (soft_cap > 0.f) s = (double)soft_cap * tanh(s / (double)soft_cap);
        scores[n] = s;
        if (s > mx) mx = s;
      }
      double total = 0.0;
      for (int64_t n = 0; n < n_tok; ++n) {
        scores[n] = exp(scores[n] - mx);
        total += scores[n];
      }
      double* acc = (double*)calloc((size_t)head_dim, sizeof(double));
      if (!acc) { free(scores); return -2; }
      for (int64_t n = 0; n < n_tok; ++n) {
        int32_t page = block_table[(int64_t)b * max_pages + n / page_size];
        if (page < 0) page = 0;
        if (page >= num_pages) page = num_pages - 1;
        const float* vr = v_cache + (((int64_t)page * page_size + n % page_size) * kv_heads + kvh) * head_dim;
        const double w = scores[n] / total;
        for (int d = 0; d < head_dim; ++d) acc[d] += w * (double)vr[d];
      }
      for (int d = 0; d < head_dim; ++d) o[d] = (float)acc[d];
      free(acc);
      lse[(int64_t)b * q_heads + h] = (float)(mx + log(total));
    }
  }
  free(scores);
  return 0;
}
