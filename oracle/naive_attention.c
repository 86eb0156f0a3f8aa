/*
 * Plain-C restatement of naive causal attention, forward and backward, in fp64.
 * TEST INFRASTRUCTURE ONLY: a second, torch-free statement of the same mathematics as
 * oracle/naive_attention.py, used to cross-check that oracle and as a checker in tests.
 * Never linked into or called from the shipped library.
 *
 * Follows the reference's ground truth (tests/test_flash_attention_2.py:288-294):
 *   S = scale * Q K^T, drop col > row (top-left anchored, also for Nq != Nk),
 *   P = softmax(S), O = P V
 * and the tile maths of the reference backward, untiled
 * (src/flash_attention_triton/_triton_kernels_v2.py:299-348):
 *   dV = P^T dO, dP = dO V^T, delta = rowsum(dO * O), dS = P * (dP - delta),
 *   dQ = scale * dS K, dK = scale * dS^T Q.
 *
 * All arrays are contiguous fp64 for ONE (batch, head) slice:
 *   q, d_o, o, dq: [nq][d];  k, v, dk, dv: [nk][d];  lse, delta: [nq].
 * Pinned by: tests/test_oracle.py (brute force, special cases, finite differences,
 * agreement with the torch oracle and with torch's scaled_dot_product_attention).
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

static int last_col(int row, int nk) { return row < nk - 1 ? row : nk - 1; }

/* Row-wise probabilities of one query row into p[0..last]; returns the row's log-sum-exp. */
static double softmax_row(const double *q, const double *k, int d, int row, int nk, double scale,
                          double *p) {
  int last = last_col(row, nk);
  double m = -INFINITY;
  for (int j = 0; j <= last; j++) {
    double s = 0.0;
    for (int c = 0; c < d; c++) s += q[(size_t)row * d + c] * k[(size_t)j * d + c];
    p[j] = s * scale;
    if (p[j] > m) m = p[j];
  }
  double z = 0.0;
  for (int j = 0; j <= last; j++) {
    p[j] = exp(p[j] - m);
    z += p[j];
  }
  for (int j = 0; j <= last; j++) p[j] /= z;
  return m + log(z);
}

int oracle_attention_forward(const double *q, const double *k, const double *v, int nq, int nk,
                             int d, double scale, double *o, double *lse) {
  double *p = (double *)malloc(sizeof(double) * (size_t)nk);
  if (!p) return 1;
  for (int i = 0; i < nq; i++) {
    int last = last_col(i, nk);
    lse[i] = softmax_row(q, k, d, i, nk, scale, p);
    for (int c = 0; c < d; c++) {
      double acc = 0.0;
      for (int j = 0; j <= last; j++) acc += p[j] * v[(size_t)j * d + c];
      o[(size_t)i * d + c] = acc;
    }
  }
  free(p);
  return 0;
}

int oracle_attention_backward(const double *q, const double *k, const double *v,
                              const double *d_o, int nq, int nk, int d, double scale, double *dq,
                              double *dk, double *dv, double *delta) {
  double *p = (double *)malloc(sizeof(double) * (size_t)nk);
  double *orow = (double *)malloc(sizeof(double) * (size_t)d);
  if (!p || !orow) {
    free(p);
    free(orow);
    return 1;
  }
  memset(dq, 0, sizeof(double) * (size_t)nq * d);
  memset(dk, 0, sizeof(double) * (size_t)nk * d);
  memset(dv, 0, sizeof(double) * (size_t)nk * d);
  for (int i = 0; i < nq; i++) {
    int last = last_col(i, nk);
    softmax_row(q, k, d, i, nk, scale, p);
    double dl = 0.0;
    for (int c = 0; c < d; c++) {
      double acc = 0.0;
      for (int j = 0; j <= last; j++) acc += p[j] * v[(size_t)j * d + c];
      orow[c] = acc;
      dl += acc * d_o[(size_t)i * d + c];
    }
    delta[i] = dl;
    for (int j = 0; j <= last; j++) {
      double dp = 0.0;
      for (int c = 0; c < d; c++) dp += d_o[(size_t)i * d + c] * v[(size_t)j * d + c];
      double ds = p[j] * (dp - dl) * scale;
      for (int c = 0; c < d; c++) {
        dv[(size_t)j * d + c] += p[j] * d_o[(size_t)i * d + c];
        dq[(size_t)i * d + c] += ds * k[(size_t)j * d + c];
        dk[(size_t)j * d + c] += ds * q[(size_t)i * d + c];
      }
    }
  }
  free(p);
  free(orow);
  return 0;
}
