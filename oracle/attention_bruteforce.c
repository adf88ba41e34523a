/*
 * fp64 brute-force attention forward and backward.  TEST INFRASTRUCTURE ONLY:
 * the product never links this file.
 *
 * Explicit loops, no library calls beyond exp/log, restating the formula of
 * reference test.py:13-26 and the backward identities of reference
 * kernel/fused_mha_kernel.cu:598-603, 653-656 for one (batch, head) slice at a
 * time.  Used to pin oracle/attention_oracle.py on small cases and to produce
 * the fixtures under tests/golden/.
 *
 * Layout: q, k, v, dout, out, dq, dk, dv are (B, N, H, D) doubles,
 * lse is (B, H, N) doubles (reference kernel/fused_mha_kernel.cu:57-67).
 */
#include <math.h>
#include <stdlib.h>

static size_t idx(int b, int i, int h, int j, int N, int H, int D) {
  return (((size_t)b * N + i) * H + h) * D + j;
}

/* Returns 0 on success, 1 on allocation failure. */
int attention_bruteforce(const double *q, const double *k, const double *v, const double *dout,
                         double *out, double *lse, double *dq, double *dk, double *dv,
                         int B, int N, int H, int D, double scale, int causal) {
  double *p = (double *)malloc(sizeof(double) * N);
  double *dp = (double *)malloc(sizeof(double) * N);
  if (!p || !dp) { free(p); free(dp); return 1; }
  for (size_t t = 0; t < (size_t)B * N * H * D; ++t) { dq[t] = 0; dk[t] = 0; dv[t] = 0; }
  for (int b = 0; b < B; ++b)
    for (int h = 0; h < H; ++h)
      for (int i = 0; i < N; ++i) {
        int last = causal ? i : N - 1; /* key j visible iff j <= i */
        double mx = -INFINITY;
        for (int j = 0; j <= last; ++j) {
          double s = 0;
          for (int e = 0; e < D; ++e) s += q[idx(b, i, h, e, N, H, D)] * k[idx(b, j, h, e, N, H, D)];
          p[j] = s * scale;
          if (p[j] > mx) mx = p[j];
        }
        double sum = 0;
        for (int j = 0; j <= last; ++j) { p[j] = exp(p[j] - mx); sum += p[j]; }
        for (int j = 0; j <= last; ++j) p[j] /= sum;
        lse[((size_t)b * H + h) * N + i] = mx + log(sum);
        for (int e = 0; e < D; ++e) {
          double o = 0;
          for (int j = 0; j <= last; ++j) o += p[j] * v[idx(b, j, h, e, N, H, D)];
          out[idx(b, i, h, e, N, H, D)] = o;
        }
        /* backward of this row */
        double delta = 0;
        for (int j = 0; j <= last; ++j) {
          double t = 0;
          for (int e = 0; e < D; ++e) t += dout[idx(b, i, h, e, N, H, D)] * v[idx(b, j, h, e, N, H, D)];
          dp[j] = t;
          delta += p[j] * t;
        }
        for (int j = 0; j <= last; ++j) {
          double ds = p[j] * (dp[j] - delta) * scale;
          for (int e = 0; e < D; ++e) {
            dv[idx(b, j, h, e, N, H, D)] += p[j] * dout[idx(b, i, h, e, N, H, D)];
            dq[idx(b, i, h, e, N, H, D)] += ds * k[idx(b, j, h, e, N, H, D)];
            dk[idx(b, j, h, e, N, H, D)] += ds * q[idx(b, i, h, e, N, H, D)];
          }
        }
      }
  free(p);
  free(dp);
  return 0;
}
