/*
 * Plain-C restatement of the mask-routed linear / SwiGLU FFN maths, in double precision on raw
 * bf16 bit patterns.  Test infrastructure: an oracle that does not go through torch's matmul.
 *
 *   linear forward   y[m,n]  = sum_k x[m,k] * W_sel(m)[n,k]                 (linear.py:76-159 computes this per tile)
 *   ffn forward      out[m,:] = W2_sel (silu(W1_sel x[m]) * (W3_sel x[m]))  (ffn.py:15-113 then linear.py:76-159)
 *   linear backward  dx[m,k] = sum_n g[m,n] W_sel(m)[n,k];  dW_g[n,k] = sum_{m in g} g[m,n] x[m,k]
 *                                                                           (linear.py:242-326, 329-415)
 * Weights are nn.Linear-style row-major [N, K].  mask: one byte per row, non-zero = visual.
 * All results are doubles; rounding to bf16 is left to the caller.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static double bf(uint16_t v) {
  uint32_t u = (uint32_t)v << 16;
  float f;
  memcpy(&f, &u, 4);
  return (double)f;
}

/* round a double to the nearest bf16 (ties to even), returned as double */
static double round_bf16(double d) {
  float f = (float)d;
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return d; /* NaN */
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  memcpy(&f, &u, 4);
  return (double)f;
}

void ref_masked_linear_fwd(const uint16_t* x, const uint16_t* Wv, const uint16_t* Wt, const uint8_t* mask,
                           double* y, int64_t M, int64_t K, int64_t N) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    const uint16_t* W = mask[m] ? Wv : Wt;
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k) acc += bf(x[m * K + k]) * bf(W[n * K + k]);
      y[m * N + n] = acc;
    }
  }
}

/* round_mid != 0: the [M,h] intermediate is rounded to bf16 once before the down projection. */
void ref_masked_ffn_fwd(const uint16_t* x, const uint16_t* W1, const uint16_t* W2, const uint16_t* W3,
                        const uint16_t* U1, const uint16_t* U2, const uint16_t* U3, const uint8_t* mask,
                        double* out, int64_t M, int64_t d, int64_t h, int round_mid) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    const uint16_t* P1 = mask[m] ? W1 : U1;
    const uint16_t* P2 = mask[m] ? W2 : U2;
    const uint16_t* P3 = mask[m] ? W3 : U3;
    double* mid = (double*)malloc(sizeof(double) * (size_t)(h > 0 ? h : 1));
    for (int64_t j = 0; j < h; ++j) {
      double t1 = 0.0, t3 = 0.0;
      for (int64_t k = 0; k < d; ++k) {
        const double xv = bf(x[m * d + k]);
        t1 += xv * bf(P1[j * d + k]);
        t3 += xv * bf(P3[j * d + k]);
      }
      double v = t1 / (1.0 + exp(-t1)) * t3;
      mid[j] = round_mid ? round_bf16(v) : v;
    }
    for (int64_t n = 0; n < d; ++n) {
      double acc = 0.0;
      for (int64_t j = 0; j < h; ++j) acc += mid[j] * bf(P2[n * h + j]);
      out[m * d + n] = acc;
    }
    free(mid);
  }
}

void ref_masked_linear_bwd(const uint16_t* g, const uint16_t* x, const uint16_t* Wv, const uint16_t* Wt,
                           const uint8_t* mask, double* dx, double* dWv, double* dWt, int64_t M, int64_t K,
                           int64_t N) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    const uint16_t* W = mask[m] ? Wv : Wt;
    for (int64_t k = 0; k < K; ++k) {
      double acc = 0.0;
      for (int64_t n = 0; n < N; ++n) acc += bf(g[m * N + n]) * bf(W[n * K + k]);
      dx[m * K + k] = acc;
    }
  }
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t k = 0; k < K; ++k) {
      double av = 0.0, at = 0.0;
      for (int64_t m = 0; m < M; ++m) {
        const double p = bf(g[m * N + n]) * bf(x[m * K + k]);
        if (mask[m]) av += p; else at += p;
      }
      dWv[n * K + k] = av;
      dWt[n * K + k] = at;
    }
  }
}

/* perm = stable partition of 0..M-1 by mask (visual rows first); counts[0..1]. */
/* MaskedFFN backward by the chain rule, row by row (the op the reference declares but leaves at
 * NotImplementedError, ffn_kernel/ops.py:34-38; decomposition sketched in README.md:159-172, with
 * the textbook silu'(t) = s + t s (1 - s)).  Weight gradients are accumulated serially so that the
 * result does not depend on threading.  round_mid: round t1, t3, dh, dt1, dt3 and the intermediate
 * to bf16 where a kernel that stores them in bf16 does.
 * dx [M, d]; dW1, dW3, dU1, dU3 [h, d]; dW2, dU2 [d, h] (all zero-filled by the caller). */
void ref_masked_ffn_bwd(const uint16_t* g, const uint16_t* x, const uint16_t* W1, const uint16_t* W2,
                        const uint16_t* W3, const uint16_t* U1, const uint16_t* U2, const uint16_t* U3,
                        const uint8_t* mask, double* dx, double* dW1, double* dW2, double* dW3, double* dU1,
                        double* dU2, double* dU3, int64_t M, int64_t d, int64_t h, int round_mid) {
  double* dt1 = (double*)malloc(sizeof(double) * (size_t)(h > 0 ? h : 1));
  double* dt3 = (double*)malloc(sizeof(double) * (size_t)(h > 0 ? h : 1));
  double* mid = (double*)malloc(sizeof(double) * (size_t)(h > 0 ? h : 1));
  for (int64_t m = 0; m < M; ++m) {
    const uint16_t* P1 = mask[m] ? W1 : U1;
    const uint16_t* P2 = mask[m] ? W2 : U2;
    const uint16_t* P3 = mask[m] ? W3 : U3;
    double* D1 = mask[m] ? dW1 : dU1;
    double* D2 = mask[m] ? dW2 : dU2;
    double* D3 = mask[m] ? dW3 : dU3;
    for (int64_t j = 0; j < h; ++j) {
      double t1 = 0.0, t3 = 0.0, dh = 0.0;
      for (int64_t k = 0; k < d; ++k) {
        const double xv = bf(x[m * d + k]);
        t1 += xv * bf(P1[j * d + k]);
        t3 += xv * bf(P3[j * d + k]);
        dh += bf(g[m * d + k]) * bf(P2[k * h + j]);
      }
      if (round_mid) { t1 = round_bf16(t1); t3 = round_bf16(t3); dh = round_bf16(dh); }
      const double s = 1.0 / (1.0 + exp(-t1));
      const double silu = t1 * s;
      dt1[j] = dh * t3 * (s + silu * (1.0 - s));
      dt3[j] = dh * silu;
      mid[j] = silu * t3;
      if (round_mid) { dt1[j] = round_bf16(dt1[j]); dt3[j] = round_bf16(dt3[j]); mid[j] = round_bf16(mid[j]); }
    }
    for (int64_t k = 0; k < d; ++k) {
      double acc = 0.0;
      for (int64_t j = 0; j < h; ++j) acc += dt1[j] * bf(P1[j * d + k]) + dt3[j] * bf(P3[j * d + k]);
      dx[m * d + k] = acc;
    }
    for (int64_t j = 0; j < h; ++j)
      for (int64_t k = 0; k < d; ++k) {
        const double xv = bf(x[m * d + k]);
        D1[j * d + k] += dt1[j] * xv;
        D3[j * d + k] += dt3[j] * xv;
        D2[k * h + j] += bf(g[m * d + k]) * mid[j];
      }
  }
  free(dt1); free(dt3); free(mid);
}

void ref_route(const uint8_t* mask, int64_t M, int32_t* perm, int32_t* counts) {
  int64_t nv = 0;
  for (int64_t m = 0; m < M; ++m) nv += mask[m] != 0;
  int64_t iv = 0, it = nv;
  for (int64_t m = 0; m < M; ++m) {
    if (mask[m]) perm[iv++] = (int32_t)m; else perm[it++] = (int32_t)m;
  }
  counts[0] = (int32_t)nv;
  counts[1] = (int32_t)(M - nv);
}
