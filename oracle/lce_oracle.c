/* Plain-C restatement of the lm-head log-prob + entropy path.  TEST INFRASTRUCTURE ONLY:
 * nothing shipped links or loads this file; it is the second, independent statement of the math
 * that the torch restatement (lce_oracle.py) and the HIP kernels are checked against.
 *
 * Inputs are fp32 arrays (callers pass bf16-rounded values widened to fp32 when they emulate
 * the bf16 path); every reduction is carried in double.
 *
 * Follows (reference tree):
 *   forward : verl/utils/kernel/kernels.py:306-329 (z = (h.W^T) * (1/tau), online max / sum-exp /
 *             sum z*exp), :419-433 (entropy = log(accu) + max - b, logprob = z_label - lse)
 *   backward: verl/utils/kernel/kernels.py:1443-1507 (dz), :1714-1724 (d_hidden, d_weight)
 * Build: see Makefile (gcc -O2 -fopenmp -shared).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static void row_logits(const float* h, const float* W, int64_t H, int64_t V, double rcp_tau, double* z) {
  for (int64_t v = 0; v < V; ++v) {
    const float* w = W + v * H;
    double s = 0.0;
    for (int64_t k = 0; k < H; ++k) s += (double)h[k] * (double)w[k];
    z[v] = s * rcp_tau;
  }
}

/* out: logprob[T], entropy[T], maxv[T], accu[T], eb[T] (all double) */
int lce_oracle_forward(const float* hidden, const float* weight, const int64_t* labels, int64_t T, int64_t H,
                       int64_t V, double temperature, double* logprob, double* entropy, double* maxv,
                       double* accu, double* eb) {
  const double rcp_tau = 1.0 / temperature;
  int bad = 0;
#pragma omp parallel
  {
    double* z = (double*)malloc(sizeof(double) * (size_t)V);
#pragma omp for schedule(static)
    for (int64_t t = 0; t < T; ++t) {
      if (labels[t] < 0 || labels[t] >= V) { bad = 1; continue; }
      row_logits(hidden + t * H, weight, H, V, rcp_tau, z);
      double m = -INFINITY;
      for (int64_t v = 0; v < V; ++v) m = z[v] > m ? z[v] : m;
      double a = 0.0, b = 0.0;
      for (int64_t v = 0; v < V; ++v) {
        double e = exp(z[v] - m);
        a += e;
        b += z[v] * e;
      }
      b /= a;
      double lse = m + log(a);
      logprob[t] = z[labels[t]] - lse;
      entropy[t] = lse - b;
      maxv[t] = m; accu[t] = a; eb[t] = b;
    }
    free(z);
  }
  return bad ? -1 : 0;
}

/* g_lp[T], g_ent[T] (g_ent may be NULL); out: d_hidden[T*H], d_weight[V*H] (double, overwritten) */
int lce_oracle_backward(const float* hidden, const float* weight, const int64_t* labels, int64_t T, int64_t H,
                        int64_t V, double temperature, const double* g_lp, const double* g_ent,
                        double* d_hidden, double* d_weight) {
  const double rcp_tau = 1.0 / temperature;
  memset(d_weight, 0, sizeof(double) * (size_t)(V * H));
  double* z = (double*)malloc(sizeof(double) * (size_t)V);
  for (int64_t t = 0; t < T; ++t) {
    const float* h = hidden + t * H;
    row_logits(h, weight, H, V, rcp_tau, z);
    double m = -INFINITY;
    for (int64_t v = 0; v < V; ++v) m = z[v] > m ? z[v] : m;
    double a = 0.0, b = 0.0;
    for (int64_t v = 0; v < V; ++v) { double e = exp(z[v] - m); a += e; b += z[v] * e; }
    b /= a;
    double* dh = d_hidden + t * H;
    for (int64_t k = 0; k < H; ++k) dh[k] = 0.0;
    for (int64_t v = 0; v < V; ++v) {
      double p = exp(z[v] - m) / a;
      double dz = g_lp[t] * ((v == labels[t] ? 1.0 : 0.0) - p);
      if (g_ent) dz -= g_ent[t] * p * (z[v] - b);
      dz *= rcp_tau;
      const float* w = weight + v * H;
      double* dw = d_weight + v * H;
      for (int64_t k = 0; k < H; ++k) { dh[k] += dz * (double)w[k]; dw[k] += dz * (double)h[k]; }
    }
  }
  free(z);
  return 0;
}
