/*
 * C twin of the CPU oracle (attn_oracle.py).  TEST INFRASTRUCTURE ONLY: it is linked by tests and
 * by nothing that ships.  Dependency-free C99 so that it also builds with host sanitizers.
 *
 * attn_ref_fwd  : out_i = sum_j softmax_j(scale q_i.k_j) v_j, lse_i = log sum_j exp(scale q_i.k_j)
 *                 for one (batch, head): q [Sq][D], k [Sk][D], v [Sk][D] row-major float,
 *                 accumulation in double.  Contract of the (out, lse) registry adapters,
 *                 xfuser/core/distributed/attention_backend.py:504-516.
 * attn_ref_merge: one fold of the ring merge in double,
 *                 torch/distributed/tensor/experimental/_context_parallel/_attention.py:181-182
 *                 (reached by xfuser/core/long_ctx_attention/ring/ring_flash_attn.py:138).
 */
#include <math.h>
#include <stddef.h>
#include <stdlib.h>

int attn_ref_fwd(const float* q, const float* k, const float* v, long Sq, long Sk, int D,
                 double scale, double* out, double* lse) {
  double* s = (double*)malloc(sizeof(double) * (size_t)Sk);
  if (!s) return -1;
  for (long i = 0; i < Sq; i++) {
    double m = -INFINITY;
    for (long j = 0; j < Sk; j++) {
      double acc = 0.0;
      for (int d = 0; d < D; d++) acc += (double)q[i * D + d] * (double)k[j * D + d];
      s[j] = acc * scale;
      if (s[j] > m) m = s[j];
    }
    double l = 0.0;
    for (long j = 0; j < Sk; j++) {
      s[j] = exp(s[j] - m);
      l += s[j];
    }
    for (int d = 0; d < D; d++) {
      double acc = 0.0;
      for (long j = 0; j < Sk; j++) acc += s[j] * (double)v[j * D + d];
      out[i * D + d] = acc / l;
    }
    lse[i] = m + log(l);
  }
  free(s);
  return 0;
}

static double sigmoid(double x) { return 1.0 / (1.0 + exp(-x)); }
static double logsigmoid(double x) { return (x < 0 ? x : 0.0) - log1p(exp(-fabs(x))); }

/* rows x D accumulators; lse per row. In place on out/lse. */
void attn_ref_merge(double* out, double* lse, const double* block_out, const double* block_lse,
                    long rows, int D) {
  for (long r = 0; r < rows; r++) {
    double w = sigmoid(block_lse[r] - lse[r]);
    for (int d = 0; d < D; d++) {
      double o = out[r * D + d];
      out[r * D + d] = o - w * (o - block_out[r * D + d]);
    }
    lse[r] = lse[r] - logsigmoid(lse[r] - block_lse[r]);
  }
}
