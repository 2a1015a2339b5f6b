/*
 * Plain-C restatement of the attention forward the reference asks its vendor kernel for.
 * TEST INFRASTRUCTURE ONLY: never linked into, loaded by or shipped with the product library.
 *
 * Follows, one row of the score matrix at a time:
 *   the oracle of the reference's own test, test/torch_ops/test_scaled_dot_product_attention.py:78-161
 *     (scores = scale q.k, bottom-right causal mask col > row + Lk - Lq from :46-75, softmax, rows with no visible
 *      key -> 0, P V, query head h reads kv head h / (Hq/Hk) as in the "(h g)" repeat at :119-120), and
 *   the launcher's data contract, torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:113-129,147-161
 *     (packed rows addressed through int32 cu_seqlens, fp32 compute, LSE buffer [Hq, total_q]).
 * LSE = ln sum_j exp(score_j) over visible j; +inf for a row with no visible key.
 * Accumulation is in double so that this file is an independent check of the numpy restatement
 * (oracle/attention_oracle.py), not a copy of its rounding.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

static void one_row(const float* q, const float* k, const float* v, int64_t k_row_stride, int64_t v_row_stride, int Lk,
                    int visible, int D, double scale, float* out, float* lse, double* scratch) {
  /* visible = number of leading keys this row may see (0..Lk) */
  double m = -INFINITY;
  for (int j = 0; j < visible; ++j) {
    const float* kj = k + (int64_t)j * k_row_stride;
    double s = 0.0;
    for (int d = 0; d < D; ++d) s += (double)q[d] * (double)kj[d];
    s *= scale;
    scratch[j] = s;
    if (s > m) m = s;
  }
  (void)Lk;
  if (visible <= 0) {
    for (int d = 0; d < D; ++d) out[d] = 0.0f;
    *lse = INFINITY;
    return;
  }
  double l = 0.0;
  for (int j = 0; j < visible; ++j) {
    scratch[j] = exp(scratch[j] - m);
    l += scratch[j];
  }
  for (int d = 0; d < D; ++d) {
    double acc = 0.0;
    for (int j = 0; j < visible; ++j) acc += scratch[j] * (double)v[(int64_t)j * v_row_stride + d];
    out[d] = (float)(acc / l);
  }
  *lse = (float)(m + log(l));
}

/* Dense: q,out [B,Hq,Sq,D], k,v [B,Hk,Sk,D], lse [B,Hq,Sq]; all contiguous fp32.  Returns 0, or -1 on bad sizes. */
int fa_oracle_forward_dense(const float* q, const float* k, const float* v, float* out, float* lse, int B, int Hq, int Hk,
                            int Sq, int Sk, int D, float scale, int causal) {
  if (B <= 0 || Hq <= 0 || Hk <= 0 || Hq % Hk || D <= 0 || Sq < 0 || Sk < 0) return -1;
  const int g = Hq / Hk;
  double* scratch = (double*)malloc(sizeof(double) * (size_t)(Sk > 0 ? Sk : 1));
  if (!scratch) return -1;
  for (int b = 0; b < B; ++b)
    for (int h = 0; h < Hq; ++h) {
      const float* kb = k + ((int64_t)b * Hk + h / g) * Sk * D;
      const float* vb = v + ((int64_t)b * Hk + h / g) * Sk * D;
      for (int i = 0; i < Sq; ++i) {
        int visible = Sk;
        if (causal) {
          visible = i + Sk - Sq + 1; /* col <= row + Lk - Lq */
          if (visible < 0) visible = 0;
          if (visible > Sk) visible = Sk;
        }
        const int64_t r = ((int64_t)b * Hq + h) * Sq + i;
        one_row(q + r * D, kb, vb, D, D, Sk, visible, D, (double)scale, out + r * D, lse + r, scratch);
      }
    }
  free(scratch);
  return 0;
}

/* Packed: q,out [Tq,Hq,D], k,v [Tk,Hk,D], cu_seqlens int32 [B+1], lse [Hq,Tq]; contiguous fp32. */
int fa_oracle_forward_packed(const float* q, const float* k, const float* v, float* out, float* lse, const int32_t* cu_q,
                             const int32_t* cu_k, int B, int Hq, int Hk, int D, int64_t Tq, float scale, int causal) {
  if (B <= 0 || Hq <= 0 || Hk <= 0 || Hq % Hk || D <= 0) return -1;
  const int g = Hq / Hk;
  int maxk = 1;
  for (int b = 0; b < B; ++b)
    if (cu_k[b + 1] - cu_k[b] > maxk) maxk = cu_k[b + 1] - cu_k[b];
  double* scratch = (double*)malloc(sizeof(double) * (size_t)maxk);
  if (!scratch) return -1;
  for (int b = 0; b < B; ++b) {
    const int Lq = cu_q[b + 1] - cu_q[b], Lk = cu_k[b + 1] - cu_k[b];
    for (int h = 0; h < Hq; ++h) {
      const float* kb = k + ((int64_t)cu_k[b] * Hk + h / g) * D;
      const float* vb = v + ((int64_t)cu_k[b] * Hk + h / g) * D;
      for (int i = 0; i < Lq; ++i) {
        int visible = Lk;
        if (causal) {
          visible = i + Lk - Lq + 1;
          if (visible < 0) visible = 0;
          if (visible > Lk) visible = Lk;
        }
        const int64_t t = (int64_t)cu_q[b] + i;
        one_row(q + (t * Hq + h) * D, kb, vb, (int64_t)Hk * D, (int64_t)Hk * D, Lk, visible, D, (double)scale,
                out + (t * Hq + h) * D, lse + (int64_t)h * Tq + t, scratch);
      }
    }
  }
  free(scratch);
  return 0;
}
