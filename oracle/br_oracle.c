/*
 * br_oracle.c -- see br_oracle.h.  TEST INFRASTRUCTURE ONLY: parity checker
 * and timed CPU baseline; never linked into the shipped path.
 *
 * Plain C + OpenMP.  fp32 storage, fp64 accumulation, one rounding at the
 * end of every reduction.
 */
#include "br_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int orc_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ---------------------------------------------------------------- GEMMs -- */
/* C[m,n] (+)= alpha * sum_k A[m,k] B[n,k]   (both K-contiguous) */
static void gemm_nt(const float* A, const float* B, float* C, int64_t m,
                    int64_t n, int64_t k, double alpha, const float* bias,
                    int accumulate) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t i = 0; i < m; i++) {
        for (int64_t j = 0; j < n; j++) {
            const float* a = A + i * k;
            const float* b = B + j * k;
            double acc = 0.0;
#pragma omp simd reduction(+ : acc)
            for (int64_t p = 0; p < k; p++) acc += (double)a[p] * (double)b[p];
            acc *= alpha;
            if (bias) acc += (double)bias[j];
            if (accumulate) acc += (double)C[i * n + j];
            C[i * n + j] = (float)acc;
        }
    }
}

/* C[m,n] (+)= alpha * sum_k A[m,k] B[k,n] */
static void gemm_nn(const float* A, const float* B, float* C, int64_t m,
                    int64_t n, int64_t k, double alpha, int accumulate) {
#pragma omp parallel
    {
        double* acc = (double*)malloc(sizeof(double) * (size_t)n);
#pragma omp for schedule(static)
        for (int64_t i = 0; i < m; i++) {
            for (int64_t j = 0; j < n; j++) acc[j] = 0.0;
            for (int64_t p = 0; p < k; p++) {
                const double a = (double)A[i * k + p];
                const float* b = B + p * n;
#pragma omp simd
                for (int64_t j = 0; j < n; j++) acc[j] += a * (double)b[j];
            }
            for (int64_t j = 0; j < n; j++) {
                double v = acc[j] * alpha;
                if (accumulate) v += (double)C[i * n + j];
                C[i * n + j] = (float)v;
            }
        }
        free(acc);
    }
}

/* C[m,n] (+)= alpha * sum_k A[k,m] B[k,n] */
static void gemm_tn(const float* A, const float* B, float* C, int64_t m,
                    int64_t n, int64_t k, double alpha, int accumulate) {
#pragma omp parallel
    {
        double* acc = (double*)malloc(sizeof(double) * (size_t)n);
#pragma omp for schedule(static)
        for (int64_t i = 0; i < m; i++) {
            for (int64_t j = 0; j < n; j++) acc[j] = 0.0;
            for (int64_t p = 0; p < k; p++) {
                const double a = (double)A[p * m + i];
                if (a == 0.0) continue;
                const float* b = B + p * n;
#pragma omp simd
                for (int64_t j = 0; j < n; j++) acc[j] += a * (double)b[j];
            }
            for (int64_t j = 0; j < n; j++) {
                double v = acc[j] * alpha;
                if (accumulate) v += (double)C[i * n + j];
                C[i * n + j] = (float)v;
            }
        }
        free(acc);
    }
}

/* ------------------------------------------------------------ LayerNorm -- */
void orc_layernorm_fwd(const float* x, const float* gamma, const float* beta,
                       float* y, float* mean_out, float* var_out,
                       int64_t rows, int64_t cols, float eps) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        const float* xr = x + r * cols;
        double s = 0.0, ss = 0.0;
        for (int64_t c = 0; c < cols; c++) {
            s += (double)xr[c];
            ss += (double)xr[c] * (double)xr[c];
        }
        const double mean = s / (double)cols;
        /* normalize_kernels.cu:64: eps is folded into the stored variance */
        const double var = ss / (double)cols - mean * mean + (double)eps;
        const double rstd = 1.0 / sqrt(var);
        if (mean_out) mean_out[r] = (float)mean;
        if (var_out) var_out[r] = (float)var;
        float* yr = y + r * cols;
        for (int64_t c = 0; c < cols; c++) {
            yr[c] = (float)(((double)xr[c] - mean) * rstd * (double)gamma[c] +
                            (double)beta[c]);
        }
    }
}

/* normalize_kernels.cu:14-17 */
static inline double add_eps(double g, double eps) {
    return fabs(g) > eps ? g : (g < 0.0 ? -eps : eps);
}

void orc_layernorm_bwd(const float* dy, const float* y, const float* gamma,
                       const float* beta, const float* var_in,
                       float* dgamma, float* dbeta, float* dx,
                       int64_t rows, int64_t cols, float eps) {
    const double e = (double)eps;
    /* column sums (normalize_kernels.cu:276-291): dbeta, dgamma overwritten */
#pragma omp parallel for schedule(static)
    for (int64_t c = 0; c < cols; c++) {
        const double g = add_eps((double)gamma[c], e);
        const double b = (double)beta[c];
        double sb = 0.0, sg = 0.0;
        for (int64_t r = 0; r < rows; r++) {
            const double d = (double)dy[r * cols + c];
            const double xhat = ((double)y[r * cols + c] - b) / g;
            sb += d;
            sg += xhat * d;
        }
        dbeta[c] = (float)sb;
        dgamma[c] = (float)sg;
    }
    /* row pass (normalize_kernels.cu:154-220) */
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        /* :166 -- eps is added a second time on top of the stored var+eps */
        const double rstd = 1.0 / sqrt((double)var_in[r] + e);
        double s1 = 0.0, s2 = 0.0;
        for (int64_t c = 0; c < cols; c++) {
            const double dxhat = (double)dy[r * cols + c] * (double)gamma[c];
            const double xhat = ((double)y[r * cols + c] - (double)beta[c]) /
                                add_eps((double)gamma[c], e);
            s1 += dxhat;
            s2 += dxhat * xhat;
        }
        s1 /= (double)cols;
        s2 /= (double)cols;
        for (int64_t c = 0; c < cols; c++) {
            const double dxhat = (double)dy[r * cols + c] * (double)gamma[c];
            const double xhat = ((double)y[r * cols + c] - (double)beta[c]) /
                                add_eps((double)gamma[c], e);
            dx[r * cols + c] = (float)((dxhat - s1 - xhat * s2) * rstd);
        }
    }
}

/* ----------------------------------------------------------------- GELU -- */
static inline float gelu_fwd_one(double v) {
    /* gelu.cu:42 -- fp32 literals 0.79788456F and 0.03567741F */
    const double c0 = (double)0.79788456f, c1 = (double)0.03567741f;
    return (float)(v * (0.5 + 0.5 * tanh(v * (c0 + c1 * v * v))));
}

static inline float gelu_bwd_one(float dy, double x) {
    /* gelu.cu:65-68 -- double literals; tanh_out and ff are stored in float */
    const float t = (float)tanh(0.79788456 * x * (1 + 0.044715 * x * x));
    const double td = (double)t;
    const float ff = (float)(0.5 * x * ((1 - td * td) *
                                        (0.79788456 + 0.1070322243 * x * x)) +
                             0.5 * (1 + td));
    return ff * dy;
}

void orc_gelu_fwd(const float* x, float* y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) y[i] = gelu_fwd_one((double)x[i]);
}

void orc_gelu_bwd(const float* dy, const float* x, float* dx, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) dx[i] = gelu_bwd_one(dy[i], (double)x[i]);
}

void orc_bias_gelu_fwd(const float* x, const float* bias, float* y,
                       int64_t rows, int64_t cols) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < cols; c++)
            y[r * cols + c] =
                gelu_fwd_one((double)x[r * cols + c] + (double)bias[c]);
}

void orc_bias_gelu_bwd(const float* dy, const float* x, const float* bias,
                       float* dx, float* dbias, int64_t rows, int64_t cols) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < cols; c++)
            dx[r * cols + c] = gelu_bwd_one(
                dy[r * cols + c], (double)x[r * cols + c] + (double)bias[c]);
    if (dbias) {
#pragma omp parallel for schedule(static)
        for (int64_t c = 0; c < cols; c++) {
            double s = 0.0;
            for (int64_t r = 0; r < rows; r++) s += (double)dx[r * cols + c];
            dbias[c] = (float)s;
        }
    }
}

/* --------------------------------------------------------------- Linear -- */
void orc_linear_fwd(const float* x, const float* w, const float* b, float* y,
                    int64_t n, int64_t in, int64_t out) {
    gemm_nt(x, w, y, n, out, in, 1.0, b, 0);
}

void orc_linear_bwd(const float* dy, const float* x, const float* w,
                    float* dx, float* dw, float* db, int64_t n, int64_t in,
                    int64_t out) {
    /* cuda_tensor.cpp:738-760: bias grad = column sum of dy */
#pragma omp parallel for schedule(static)
    for (int64_t o = 0; o < out; o++) {
        double s = 0.0;
        for (int64_t r = 0; r < n; r++) s += (double)dy[r * out + o];
        db[o] = (float)s;
    }
    /* :763-783 weight grad first (x is still intact when dx aliases it) */
    gemm_tn(dy, x, dw, out, in, n, 1.0, 0);
    /* :785-806 input grad */
    gemm_nn(dy, w, dx, n, in, out, 1.0, 0);
}

/* ------------------------------------------------------- transpose 0213 -- */
void orc_transpose_0213(const float* x, float* y, int64_t s0, int64_t s1,
                        int64_t s2, int64_t s3) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t a = 0; a < s0; a++)
        for (int64_t b = 0; b < s1; b++)
            for (int64_t c = 0; c < s2; c++)
                memcpy(y + ((a * s2 + c) * s1 + b) * s3,
                       x + ((a * s1 + b) * s2 + c) * s3,
                       sizeof(float) * (size_t)s3);
}

/* -------------------------------------------------------- broadcast add -- */
void orc_add_bcast(const float* a, const int64_t* as, const float* b,
                   const int64_t* bs, float* c) {
    const int64_t st3 = bs[3] == 1 ? 0 : 1;
    const int64_t st2 = bs[2] == 1 ? 0 : bs[3];
    const int64_t st1 = bs[1] == 1 ? 0 : bs[2] * bs[3];
    const int64_t st0 = bs[0] == 1 ? 0 : bs[1] * bs[2] * bs[3];
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t i0 = 0; i0 < as[0]; i0++)
        for (int64_t i1 = 0; i1 < as[1]; i1++)
            for (int64_t i2 = 0; i2 < as[2]; i2++) {
                const int64_t base = ((i0 * as[1] + i1) * as[2] + i2) * as[3];
                const float* bp = b + i0 * st0 + i1 * st1 + i2 * st2;
                for (int64_t i3 = 0; i3 < as[3]; i3++)
                    c[base + i3] = a[base + i3] + bp[i3 * st3];
            }
}

/* ------------------------------------------------------------ attention -- */
void orc_qk(const float* q, const float* k, float* s, int64_t bh, int64_t t,
            int64_t hd) {
    /* cuda_tensor.cpp:292: alpha is rounded to float before use */
    const double alpha = (double)(float)(1.0 / sqrt((double)hd));
    for (int64_t i = 0; i < bh; i++)
        gemm_nt(q + i * t * hd, k + i * t * hd, s + i * t * t, t, t, hd, alpha,
                NULL, 0);
}

void orc_softmax_fwd(const float* x, float* y, int64_t rows, int64_t cols) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        const float* xr = x + r * cols;
        float* yr = y + r * cols;
        double mx = (double)xr[0];
        for (int64_t c = 1; c < cols; c++)
            if ((double)xr[c] > mx) mx = (double)xr[c];
        double s = 0.0;
        for (int64_t c = 0; c < cols; c++) s += exp((double)xr[c] - mx);
        for (int64_t c = 0; c < cols; c++)
            yr[c] = (float)(exp((double)xr[c] - mx) / s);
    }
}

void orc_softmax_bwd(const float* dy, const float* y, float* dx, int64_t rows,
                     int64_t cols) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        double dot = 0.0;
        for (int64_t c = 0; c < cols; c++)
            dot += (double)dy[r * cols + c] * (double)y[r * cols + c];
        for (int64_t c = 0; c < cols; c++)
            dx[r * cols + c] = (float)((double)y[r * cols + c] *
                                       ((double)dy[r * cols + c] - dot));
    }
}

void orc_attn(const float* p, const float* v, float* o, int64_t bh, int64_t t,
              int64_t hd) {
    for (int64_t i = 0; i < bh; i++)
        gemm_nn(p + i * t * t, v + i * t * hd, o + i * t * hd, t, hd, t, 1.0,
                0);
}

void orc_attn_bwd(const float* d_o, const float* p, const float* v, float* dp,
                  float* dv, int64_t bh, int64_t t, int64_t hd) {
    for (int64_t i = 0; i < bh; i++) {
        /* dV = P^T dO (cuda_tensor.cpp:846-864) */
        gemm_tn(p + i * t * t, d_o + i * t * hd, dv + i * t * hd, t, hd, t,
                1.0, 0);
        /* dP = dO V^T (:866-884) */
        gemm_nt(d_o + i * t * hd, v + i * t * hd, dp + i * t * t, t, t, hd,
                1.0, NULL, 0);
    }
}

void orc_softmax_attn_bwd(const float* d_o, const float* p, const float* v,
                          float* ds, float* dv, int64_t bh, int64_t t,
                          int64_t hd) {
    float* stage = (float*)malloc(sizeof(float) * (size_t)(t * t));
    float* dp = (float*)malloc(sizeof(float) * (size_t)(t * t));
    for (int64_t i = 0; i < bh; i++) {
        const float* pi = p + i * t * t;
        gemm_tn(pi, d_o + i * t * hd, dv + i * t * hd, t, hd, t, 1.0, 0);
        /* :958-962 the probabilities are staged because ds may alias p */
        memcpy(stage, pi, sizeof(float) * (size_t)(t * t));
        gemm_nt(d_o + i * t * hd, v + i * t * hd, dp, t, t, hd, 1.0, NULL, 0);
        orc_softmax_bwd(dp, stage, ds + i * t * t, t, t);
    }
    free(stage);
    free(dp);
}

void orc_qk_bwd(const float* ds, const float* q, const float* k, float* dq,
                float* dk, int64_t bh, int64_t t, int64_t hd) {
    const double alpha = (double)(float)(1.0 / sqrt((double)hd));
    for (int64_t i = 0; i < bh; i++) {
        gemm_nn(ds + i * t * t, k + i * t * hd, dq + i * t * hd, t, hd, t,
                alpha, 0);
        gemm_tn(ds + i * t * t, q + i * t * hd, dk + i * t * hd, t, hd, t,
                alpha, 0);
    }
}

/* ------------------------------------------------------------ loss head -- */
void orc_last_logits(const float* x, const int32_t* mask, const float* lm_head,
                     float* out, int64_t batch, int64_t tokens, int64_t hidden,
                     int64_t vocab) {
    for (int64_t b = 0; b < batch; b++) {
        const int32_t* m = mask + b * tokens;
        int64_t target = 0; /* stays 0 when no padding follows (:426-432) */
        for (int64_t i = 0; i < tokens - 1; i++) {
            if (m[i + 1] == 0) {
                target = i;
                break;
            }
        }
        gemm_nt(x + (b * tokens + target) * hidden, lm_head, out + b * vocab,
                1, vocab, hidden, 1.0, NULL, 0);
    }
}

int64_t orc_loss_labels(const int32_t* ids, const int32_t* mask, int64_t batch,
                        int64_t tokens, int32_t* labels) {
    int64_t count = 0;
    for (int64_t b = 0; b < batch; b++) {
        const int32_t* m = mask + b * tokens;
        const int32_t* id = ids + b * tokens;
        for (int64_t t = 0; t < tokens; t++) {
            int32_t lab = -100;
            if (t < tokens - 1 && m[t] != 0 && m[t + 1] != 0) {
                lab = id[t + 1];
                count++;
            }
            if (labels) labels[b * tokens + t] = lab;
        }
    }
    return count;
}

int64_t orc_loss_groups(const int32_t* mask, int64_t batch, int64_t tokens,
                        int64_t group_max, int64_t* triples,
                        int64_t max_groups) {
    int64_t ng = 0;
    for (int64_t b = 0; b < batch; b++) {
        const int32_t* m = mask + b * tokens;
        int64_t begin = -1, size = 0;
        for (int64_t t = 0; t < tokens - 1; t++) {
            if (size == 0) begin = t;
            size++;
            if (t == tokens - 2 || size == group_max) {
                while (size > 0 && m[begin + size - 1] == 0) size--;
                if (size > 0) {
                    if (ng < max_groups) {
                        triples[3 * ng + 0] = b;
                        triples[3 * ng + 1] = begin;
                        triples[3 * ng + 2] = size;
                    }
                    ng++;
                }
                size = 0;
            }
        }
    }
    return ng;
}

float orc_logsoftmax_nll(const float* logits, const int32_t* target,
                         const int32_t* keep, float* lse, float* dlogits,
                         int64_t rows, int64_t vocab) {
    int64_t count = 0;
    for (int64_t r = 0; r < rows; r++)
        if (keep[r] != 0) count++;
    const double scale = count > 0 ? 1.0 / (double)count : 0.0;
    double total = 0.0;
#pragma omp parallel for schedule(static) reduction(+ : total)
    for (int64_t r = 0; r < rows; r++) {
        const float* lr = logits + r * vocab;
        double mx = (double)lr[0];
        for (int64_t c = 1; c < vocab; c++)
            if ((double)lr[c] > mx) mx = (double)lr[c];
        double s = 0.0;
        for (int64_t c = 0; c < vocab; c++) s += exp((double)lr[c] - mx);
        const double l = mx + log(s);
        if (lse) lse[r] = (float)l;
        const int valid =
            keep[r] != 0 && target[r] >= 0 && (int64_t)target[r] < vocab;
        if (valid) total += (double)lr[target[r]] - l;
        if (dlogits) {
            float* dr = dlogits + r * vocab;
            if (valid) {
                for (int64_t c = 0; c < vocab; c++)
                    dr[c] = (float)(exp((double)lr[c] - l) * scale);
                dr[target[r]] =
                    (float)((exp((double)lr[target[r]] - l) - 1.0) * scale);
            } else {
                memset(dr, 0, sizeof(float) * (size_t)vocab);
            }
        }
    }
    return (float)(total * scale);
}

float orc_loss_backward(const float* x, const int32_t* ids,
                        const int32_t* mask, const float* lm_head, float* x_g,
                        float* lm_head_g, float* dlogits_out, int64_t batch,
                        int64_t tokens, int64_t hidden, int64_t vocab) {
    const int64_t n = batch * tokens;
    int32_t* labels = (int32_t*)malloc(sizeof(int32_t) * (size_t)n);
    int32_t* keep = (int32_t*)malloc(sizeof(int32_t) * (size_t)n);
    orc_loss_labels(ids, mask, batch, tokens, labels);
    for (int64_t i = 0; i < n; i++) keep[i] = labels[i] >= 0 && labels[i] < vocab;
    float* logits = (float*)malloc(sizeof(float) * (size_t)(n * vocab));
    float* dl = dlogits_out
                    ? dlogits_out
                    : (float*)malloc(sizeof(float) * (size_t)(n * vocab));
    /* vocab_embedding (cuda_tensor.cpp:467-489) */
    gemm_nt(x, lm_head, logits, n, vocab, hidden, 1.0, NULL, 0);
    /* Note: the count that scales the loss is count_loss_tokens (:555-568),
     * which does not look at the label range; labels outside [0,vocab) are
     * skipped by nll_loss.cu:29 but still counted. */
    int64_t count = orc_loss_labels(ids, mask, batch, tokens, NULL);
    const double scale = 1.0 / (double)count;
    double total = 0.0;
#pragma omp parallel for schedule(static) reduction(+ : total)
    for (int64_t r = 0; r < n; r++) {
        const float* lr = logits + r * vocab;
        float* dr = dl + r * vocab;
        if (!keep[r]) {
            memset(dr, 0, sizeof(float) * (size_t)vocab);
            continue;
        }
        double mx = (double)lr[0];
        for (int64_t c = 1; c < vocab; c++)
            if ((double)lr[c] > mx) mx = (double)lr[c];
        double s = 0.0;
        for (int64_t c = 0; c < vocab; c++) s += exp((double)lr[c] - mx);
        const double l = mx + log(s);
        total += (double)lr[labels[r]] - l;
        for (int64_t c = 0; c < vocab; c++)
            dr[c] = (float)(exp((double)lr[c] - l) * scale);
        dr[labels[r]] = (float)((exp((double)lr[labels[r]] - l) - 1.0) * scale);
    }
    /* vocab_grad_x (:491-513): x_g zeroed (:592) then written on covered rows */
    gemm_nn(dl, lm_head, x_g, n, hidden, vocab, 1.0, 0);
    /* vocab_grad_w (:515-533): beta = 1, accumulates */
    gemm_tn(dl, x, lm_head_g, vocab, hidden, n, 1.0, 1);
    free(labels);
    free(keep);
    free(logits);
    if (!dlogits_out) free(dl);
    return (float)(total / (double)count);
}

/* ----------------------------------------------------------- fetch_data -- */
void orc_embedding_gather(const float* vocab, const int32_t* ids, float* out,
                          int64_t n, int64_t hidden) {
    for (int64_t i = 0; i < n; i++)
        memcpy(out + i * hidden, vocab + (int64_t)ids[i] * hidden,
               sizeof(float) * (size_t)hidden);
}

/* Backward of the gather (no counterpart in the reference, whose embedding
 * table is frozen): the plain sequential scatter, which fixes the summation
 * order for repeated ids. */
void orc_embedding_scatter_add(float* grad, const float* dx, const int32_t* ids,
                               int64_t n, int64_t hidden, int64_t vocab) {
    for (int64_t i = 0; i < n; i++) {
        if (ids[i] < 0 || ids[i] >= vocab) continue;
        float* row = grad + (int64_t)ids[i] * hidden;
        for (int64_t c = 0; c < hidden; c++) row[c] += dx[i * hidden + c];
    }
}

void orc_alibi(float* alibi, int64_t heads, int64_t tokens) {
    double base = 3 - log2((double)heads * 1.0);
    base = -1 * pow(2.0, base);
    base = pow(2.0, base);
    for (int64_t j = 0; j < heads; j++) {
        const double slope = pow(base, (double)(j + 1) * 1.0);
        for (int64_t k = 0; k < tokens; k++)
            alibi[j * tokens + k] = (float)((double)k * 1.0 * slope);
    }
}

void orc_xmask(const int32_t* mask, float* xmask, int64_t batch,
               int64_t tokens) {
    const int64_t total = batch * tokens * tokens;
    for (int64_t i = 0; i < total; i++) xmask[i] = -FLT_MAX;
    for (int64_t b = 0; b < batch; b++) {
        const int32_t* ms = mask + b * tokens;
        float* m2d = xmask + b * tokens * tokens;
        for (int64_t m = 0; m < tokens; m++) {
            for (int64_t n = 0; n <= m; n++) {
                if (ms[n] != 0)
                    m2d[m * tokens + n] = 0.0f;
                else
                    break;
            }
        }
    }
}

/* ------------------------------------------------------------ fp16 glue -- */
static uint16_t f32_to_f16_one(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | (absx > 0x7f800000u ? 0x200u : 0));
    if (absx >= 0x477ff000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    if (absx < 0x33000001u) /* below half of the smallest subnormal */
        return (uint16_t)sign;
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x7fffffu) | 0x800000u;
    int shift;
    uint32_t half_exp;
    if (e < -14) { /* subnormal half */
        shift = 13 + (-14 - e);
        half_exp = 0;
    } else {
        shift = 13;
        half_exp = (uint32_t)(e + 15);
    }
    uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    uint32_t out;
    if (half_exp == 0)
        out = q; /* may carry into the normal range, which is correct */
    else
        out = ((half_exp - 1) << 10) + q; /* q carries the implicit bit */
    return (uint16_t)(sign | out);
}

static float f16_to_f32_one(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu;
    const uint32_t m = h & 0x3ffu;
    uint32_t x;
    if (e == 0) {
        if (m == 0) {
            x = sign;
        } else {
            float f = (float)m * 5.9604644775390625e-08f; /* 2^-24 */
            memcpy(&x, &f, 4);
            x |= sign;
        }
    } else if (e == 31) {
        x = sign | 0x7f800000u | (m << 13);
    } else {
        x = sign | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

void orc_f32_to_f16(const float* x, uint16_t* y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) y[i] = f32_to_f16_one(x[i]);
}

void orc_f16_to_f32(const uint16_t* x, float* y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) y[i] = f16_to_f32_one(x[i]);
}
