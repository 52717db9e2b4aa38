/*
 * ref_ops.c -- TEST INFRASTRUCTURE, not product code.
 *
 * Plain-C, double-accumulating, loop-by-loop restatement of the arithmetic of
 * fattorib/tritonformer's operators.  It exists to pin oracle/ref_torch.py (the
 * PyTorch fp32 oracle) with an independent brute-force implementation,
 * including explicit closed-form backward passes that do not go through
 * autograd.  Only tests/ may load it.  All matrices are dense row-major float.
 *
 * Reference semantics followed (paths relative to the reference repo):
 *   linear        tritonformer/linear.py:10-102, kernels/gemm.py:355-356,562-569
 *                 (y = [relu](x W + b), W is (in,out); relu grad mask is y > 0,
 *                 kernels/activation.py:22)
 *   layer norm    kernels/layernorm.py:46-54 (biased variance,
 *                 rstd = 1/sqrt(var+eps)), :124-133 (dx), :200-218 (dgamma, dbeta)
 *   softmax       kernels/softmax.py:21-34, :80-92
 *   cross entropy kernels/crossentropy.py:30-44 (per-row -log softmax[label]),
 *                 :93-107 (softmax - onehot), crossentropy.py:24 (times grad_out)
 *   attention     kernels/attention.py:128-132 (mask q >= k), :193 (scale
 *                 1/sqrt(hd)), kernels/biased_attention.py:101-106 (bias added
 *                 after scaling), tritonformer/attention.py:60 (no bias grad)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

void ref_linear_fwd(int M, int N, int K, const float* x, const float* w, const float* bias, int relu, float* y) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int k = 0; k < K; ++k) acc += (double)x[(size_t)m * K + k] * (double)w[(size_t)k * N + n];
      if (bias) acc += bias[n];
      if (relu && acc < 0.0) acc = 0.0;
      y[(size_t)m * N + n] = (float)acc;
    }
}

/* act may be NULL (no relu); otherwise dy is masked by act > 0 first. */
void ref_linear_bwd(int M, int N, int K, const float* x, const float* w, const float* dy, const float* act,
                    float* dx, float* dw, float* db) {
  for (int m = 0; m < M; ++m)
    for (int k = 0; k < K; ++k) {
      double acc = 0.0;
      for (int n = 0; n < N; ++n) {
        double g = dy[(size_t)m * N + n];
        if (act && !(act[(size_t)m * N + n] > 0.f)) g = 0.0;
        acc += g * (double)w[(size_t)k * N + n];
      }
      dx[(size_t)m * K + k] = (float)acc;
    }
  for (int k = 0; k < K; ++k)
    for (int n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int m = 0; m < M; ++m) {
        double g = dy[(size_t)m * N + n];
        if (act && !(act[(size_t)m * N + n] > 0.f)) g = 0.0;
        acc += (double)x[(size_t)m * K + k] * g;
      }
      dw[(size_t)k * N + n] = (float)acc;
    }
  if (db)
    for (int n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int m = 0; m < M; ++m) {
        double g = dy[(size_t)m * N + n];
        if (act && !(act[(size_t)m * N + n] > 0.f)) g = 0.0;
        acc += g;
      }
      db[n] = (float)acc;
    }
}

void ref_layernorm_fwd(int rows, int d, const float* x, const float* gamma, const float* beta, double eps, float* y) {
  for (int r = 0; r < rows; ++r) {
    const float* xr = x + (size_t)r * d;
    double mean = 0.0, var = 0.0;
    for (int c = 0; c < d; ++c) mean += xr[c];
    mean /= d;
    for (int c = 0; c < d; ++c) var += (xr[c] - mean) * (xr[c] - mean);
    var /= d;
    const double rstd = 1.0 / sqrt(var + eps);
    for (int c = 0; c < d; ++c) y[(size_t)r * d + c] = (float)((xr[c] - mean) * rstd * gamma[c] + beta[c]);
  }
}

void ref_layernorm_bwd(int rows, int d, const float* x, const float* gamma, const float* dy, double eps, float* dx,
                       float* dgamma, float* dbeta) {
  double* dg = (double*)calloc(d, sizeof(double));
  double* db = (double*)calloc(d, sizeof(double));
  for (int r = 0; r < rows; ++r) {
    const float* xr = x + (size_t)r * d;
    const float* gr = dy + (size_t)r * d;
    double mean = 0.0, var = 0.0;
    for (int c = 0; c < d; ++c) mean += xr[c];
    mean /= d;
    for (int c = 0; c < d; ++c) var += (xr[c] - mean) * (xr[c] - mean);
    var /= d;
    const double rstd = 1.0 / sqrt(var + eps);
    double c1 = 0.0, c2 = 0.0;
    for (int c = 0; c < d; ++c) {
      const double xh = (xr[c] - mean) * rstd, g = (double)gr[c] * gamma[c];
      c1 += g * xh;
      c2 += g;
      dg[c] += (double)gr[c] * xh;
      db[c] += gr[c];
    }
    c1 /= d;
    c2 /= d;
    for (int c = 0; c < d; ++c) {
      const double xh = (xr[c] - mean) * rstd, g = (double)gr[c] * gamma[c];
      dx[(size_t)r * d + c] = (float)((g - xh * c1 - c2) * rstd);
    }
  }
  for (int c = 0; c < d; ++c) { dgamma[c] = (float)dg[c]; dbeta[c] = (float)db[c]; }
  free(dg);
  free(db);
}

void ref_softmax_fwd(int rows, int cols, const float* x, float* y) {
  for (int r = 0; r < rows; ++r) {
    const float* xr = x + (size_t)r * cols;
    double m = xr[0], s = 0.0;
    for (int c = 1; c < cols; ++c) if (xr[c] > m) m = xr[c];
    for (int c = 0; c < cols; ++c) s += exp(xr[c] - m);
    for (int c = 0; c < cols; ++c) y[(size_t)r * cols + c] = (float)(exp(xr[c] - m) / s);
  }
}

void ref_softmax_bwd(int rows, int cols, const float* y, const float* dy, float* dx) {
  for (int r = 0; r < rows; ++r) {
    double s = 0.0;
    for (int c = 0; c < cols; ++c) s += (double)y[(size_t)r * cols + c] * dy[(size_t)r * cols + c];
    for (int c = 0; c < cols; ++c)
      dx[(size_t)r * cols + c] = (float)(y[(size_t)r * cols + c] * (dy[(size_t)r * cols + c] - s));
  }
}

void ref_cross_entropy_fwd(int rows, int V, const float* logits, const int64_t* labels, float* loss) {
  for (int r = 0; r < rows; ++r) {
    const float* xr = logits + (size_t)r * V;
    double m = xr[0], s = 0.0;
    for (int c = 1; c < V; ++c) if (xr[c] > m) m = xr[c];
    for (int c = 0; c < V; ++c) s += exp(xr[c] - m);
    loss[r] = (float)(log(s) + m - xr[labels[r]]);
  }
}

void ref_cross_entropy_bwd(int rows, int V, const float* logits, const int64_t* labels, const float* gout,
                           float* dlogits) {
  for (int r = 0; r < rows; ++r) {
    const float* xr = logits + (size_t)r * V;
    double m = xr[0], s = 0.0;
    for (int c = 1; c < V; ++c) if (xr[c] > m) m = xr[c];
    for (int c = 0; c < V; ++c) s += exp(xr[c] - m);
    for (int c = 0; c < V; ++c) {
      double p = exp(xr[c] - m) / s;
      if (c == labels[r]) p -= 1.0;
      dlogits[(size_t)r * V + c] = (float)(p * gout[r]);
    }
  }
}

/* q,k,v,o,dO,dq,dk,dv: contiguous (BH, S, hd); bias: NULL or (nh, Sb, Sb) with head = bh % nh.
 * Pass dO == NULL for forward only. */
void ref_attention(int BH, int nh, int S, int hd, const float* q, const float* k, const float* v, const float* bias,
                   int Sb, float* o, const float* dO, float* dq, float* dk, float* dv) {
  const double scale = 1.0 / sqrt((double)hd);
  double* p = (double*)malloc(sizeof(double) * S);
  double* dp = (double*)malloc(sizeof(double) * S);
  if (dO)
    for (size_t i = 0; i < (size_t)BH * S * hd; ++i) { dq[i] = 0.f; dk[i] = 0.f; dv[i] = 0.f; }
  for (int bh = 0; bh < BH; ++bh) {
    const size_t base = (size_t)bh * S * hd;
    const int h = bh % nh;
    for (int i = 0; i < S; ++i) {
      double m = -INFINITY, sum = 0.0;
      for (int j = 0; j <= i; ++j) {
        double s = 0.0;
        for (int d = 0; d < hd; ++d) s += (double)q[base + (size_t)i * hd + d] * k[base + (size_t)j * hd + d];
        s *= scale;
        if (bias) s += bias[((size_t)h * Sb + i) * Sb + j];
        p[j] = s;
        if (s > m) m = s;
      }
      for (int j = 0; j <= i; ++j) { p[j] = exp(p[j] - m); sum += p[j]; }
      for (int j = 0; j <= i; ++j) p[j] /= sum;
      for (int d = 0; d < hd; ++d) {
        double acc = 0.0;
        for (int j = 0; j <= i; ++j) acc += p[j] * v[base + (size_t)j * hd + d];
        o[base + (size_t)i * hd + d] = (float)acc;
      }
      if (!dO) continue;
      double delta = 0.0;
      for (int j = 0; j <= i; ++j) {
        double acc = 0.0;
        for (int d = 0; d < hd; ++d) acc += (double)dO[base + (size_t)i * hd + d] * v[base + (size_t)j * hd + d];
        dp[j] = acc;
        delta += p[j] * acc;
      }
      for (int j = 0; j <= i; ++j) {
        const double ds = p[j] * (dp[j] - delta) * scale;
        for (int d = 0; d < hd; ++d) {
          dq[base + (size_t)i * hd + d] += (float)(ds * k[base + (size_t)j * hd + d]);
          dk[base + (size_t)j * hd + d] += (float)(ds * q[base + (size_t)i * hd + d]);
          dv[base + (size_t)j * hd + d] += (float)(p[j] * dO[base + (size_t)i * hd + d]);
        }
      }
    }
  }
  free(p);
  free(dp);
}
