/*
 * Plain-C, double-precision, brute-force restatement of the hot path.
 * TEST INFRASTRUCTURE ONLY: nothing in the shipped package links this file.
 *
 * It shares no code with the PyTorch oracle (no matmul, no autograd): every
 * output element is an explicit sum, so a transposed operand, a dropped term
 * or a wrong sign in either oracle shows up as a disagreement between them.
 *
 *   la_naive_fwd   O = (Q K^T * M) V,  M[i][j] = exp(-s_h (i-j)) [i>=j]
 *                  (lightning_attn/ops/torch/linear_attention.py:4-34)
 *   la_naive_bwd   closed-form gradients of the same expression
 *                  (what lightning_attn/ops/triton/lightning_attn2.py:88-395
 *                  evaluates block by block)
 *   la_slopes      lightning_attn/utils/utils.py:6-31
 *   srms_fwd/bwd   lightning_attn/ops/torch/srmsnorm.py:14-18 and
 *                  lightning_attn/ops/triton/srmsnorm.py:12-74
 *
 * Layout: q,k (b,h,n,d), v,o,do (b,h,n,e), row-major doubles.  s has h entries
 * or is NULL (no decay).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static double dotd(const double *a, const double *b, int64_t m) {
    double acc = 0.0;
    for (int64_t t = 0; t < m; ++t) acc += a[t] * b[t];
    return acc;
}

void la_naive_fwd(const double *q, const double *k, const double *v, const double *s, double *o,
                  int64_t b, int64_t h, int64_t n, int64_t d, int64_t e) {
    for (int64_t bh = 0; bh < b * h; ++bh) {
        const double rate = s ? s[bh % h] : 0.0;
        const double *Q = q + bh * n * d, *K = k + bh * n * d, *V = v + bh * n * e;
        double *O = o + bh * n * e;
        for (int64_t i = 0; i < n; ++i) {
            for (int64_t c = 0; c < e; ++c) O[i * e + c] = 0.0;
            for (int64_t j = 0; j <= i; ++j) {
                const double w = exp(-rate * (double)(i - j)) * dotd(Q + i * d, K + j * d, d);
                for (int64_t c = 0; c < e; ++c) O[i * e + c] += w * V[j * e + c];
            }
        }
    }
}

void la_naive_bwd(const double *q, const double *k, const double *v, const double *s, const double *go,
                  double *dq, double *dk, double *dv, int64_t b, int64_t h, int64_t n, int64_t d, int64_t e) {
    memset(dq, 0, sizeof(double) * (size_t)(b * h * n * d));
    memset(dk, 0, sizeof(double) * (size_t)(b * h * n * d));
    memset(dv, 0, sizeof(double) * (size_t)(b * h * n * e));
    for (int64_t bh = 0; bh < b * h; ++bh) {
        const double rate = s ? s[bh % h] : 0.0;
        const double *Q = q + bh * n * d, *K = k + bh * n * d, *V = v + bh * n * e, *G = go + bh * n * e;
        double *DQ = dq + bh * n * d, *DK = dk + bh * n * d, *DV = dv + bh * n * e;
        for (int64_t i = 0; i < n; ++i) {
            for (int64_t j = 0; j <= i; ++j) {
                const double w = exp(-rate * (double)(i - j));
                const double gv = w * dotd(G + i * e, V + j * e, e); /* d loss / d score(i,j) */
                const double qk = w * dotd(Q + i * d, K + j * d, d); /* masked score(i,j)     */
                for (int64_t t = 0; t < d; ++t) {
                    DQ[i * d + t] += gv * K[j * d + t];
                    DK[j * d + t] += gv * Q[i * d + t];
                }
                for (int64_t c = 0; c < e; ++c) DV[j * e + c] += qk * G[i * e + c];
            }
        }
    }
}

/* out[i] = slope of head i, before the float32 rounding the reference applies. */
static void slopes_pow2(double *out, int64_t m) {
    const double start = pow(2.0, -pow(2.0, -(log2((double)m) - 3.0)));
    for (int64_t i = 0; i < m; ++i) out[i] = start * pow(start, (double)i);
}

void la_slopes(double *out, int64_t h) {
    int64_t p = 1;
    while (2 * p <= h) p *= 2;
    slopes_pow2(out, p);
    if (p == h) return;
    double *tmp = (double *)malloc(sizeof(double) * (size_t)(2 * p));
    slopes_pow2(tmp, 2 * p);
    for (int64_t i = 0; i < h - p; ++i) out[p + i] = tmp[2 * i];
    free(tmp);
}

void srms_fwd(const double *x, double *y, double *rstd, int64_t rows, int64_t cols, double eps) {
    for (int64_t r = 0; r < rows; ++r) {
        const double *X = x + r * cols;
        const double rs = 1.0 / sqrt(dotd(X, X, cols) / (double)cols + eps);
        rstd[r] = rs;
        for (int64_t c = 0; c < cols; ++c) y[r * cols + c] = X[c] * rs;
    }
}

void srms_bwd(const double *x, const double *dy, double *dx, int64_t rows, int64_t cols, double eps) {
    for (int64_t r = 0; r < rows; ++r) {
        const double *X = x + r * cols, *G = dy + r * cols;
        const double rs = 1.0 / sqrt(dotd(X, X, cols) / (double)cols + eps);
        const double m = dotd(X, G, cols) * rs / (double)cols; /* mean(xhat * dy) */
        for (int64_t c = 0; c < cols; ++c) dx[r * cols + c] = (G[c] - X[c] * rs * m) * rs;
    }
}
