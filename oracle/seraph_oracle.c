/*
 * seraph_oracle.c - CPU restatement of Seraph's backward / optimizer path.
 * TEST INFRASTRUCTURE ONLY (parity checker and timed CPU baseline); see
 * seraph_oracle.h for the contract and the reference citations.
 *
 * Build: gcc -O3 -march=x86-64-v3 -fopenmp -ffp-contract=off (no -ffast-math).
 */
#include "seraph_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ====================================================================== */
/* cross entropy                                                          */
/* ====================================================================== */

/* One row of shaders/cross_entropy_grad.comp:44-98. `live` = 0 reproduces the
 * "no supervision" branch (zero row, loss 0). */
static void ce_row(const float* x, uint32_t target, float* g, float* loss,
                   int64_t cols, double scale, int live) {
    if (!live || (int64_t)target >= cols) {
        memset(g, 0, (size_t)cols * sizeof(float));
        *loss = 0.0f;
        return;
    }
    float mx = -3.4e38f;
    for (int64_t c = 0; c < cols; c++) mx = x[c] > mx ? x[c] : mx;
    double sum = 0.0;
    for (int64_t c = 0; c < cols; c++) sum += exp((double)x[c] - (double)mx);
    double inv = 1.0 / sum;
    *loss = (float)(-(((double)x[target] - (double)mx) - log(sum)));
    for (int64_t c = 0; c < cols; c++) {
        double p = exp((double)x[c] - (double)mx) * inv;
        if (c == (int64_t)target) p -= 1.0;
        g[c] = (float)(p * scale);
    }
}

void orc_cross_entropy_grad(const float* logits, const uint32_t* targets,
                            float* grad, float* loss_rows,
                            int64_t rows, int64_t cols, int64_t valid_rows) {
    double scale = valid_rows > 0 ? 1.0 / (double)valid_rows : 0.0;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++)
        ce_row(logits + r * cols, targets[r], grad + r * cols, loss_rows + r, cols, scale, 1);
}

static int find_seq(const uint32_t* starts, int batch, int64_t pos) {
    int lo = 0, hi = batch;
    while (lo < hi) {                       /* src/cuda_train_context.cu:641-650 */
        int mid = (lo + hi) / 2;
        if ((int64_t)starts[mid + 1] <= pos) lo = mid + 1; else hi = mid;
    }
    return lo;
}

void orc_cross_entropy_grad_packed(const float* logits, const uint32_t* targets,
                                   float* grad, float* loss_rows,
                                   const uint32_t* seq_starts, int64_t total_tokens,
                                   int batch, int64_t cols, int64_t num_valid) {
    double scale = num_valid > 0 ? 1.0 / (double)num_valid : 0.0;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < total_tokens; r++) {
        int live = 1;
        if (seq_starts) {
            int s = find_seq(seq_starts, batch, r);
            live = r < (int64_t)seq_starts[s + 1] - 1;
        } else {
            live = r < total_tokens - 1;
        }
        ce_row(logits + r * cols, targets[r], grad + r * cols, loss_rows + r, cols, scale, live);
    }
}

void orc_reduce_sum(const float* in, float* out, int64_t count) {
    int64_t groups = (count + 511) / 512;
    for (int64_t g = 0; g < groups; g++) {
        double s = 0.0;
        int64_t end = (g + 1) * 512 < count ? (g + 1) * 512 : count;
        for (int64_t i = g * 512; i < end; i++) s += in[i];
        out[g] = (float)s;
    }
}

/* ====================================================================== */
/* GEMM                                                                   */
/* ====================================================================== */

/* Large products (the step at the benchmark widths) take a cache-blocked form of the same sum: C is cut into
 * MB x NB tiles, K into runs of KB; inside a run the partial dot products are accumulated in FP32 with fused
 * multiply-adds (one rounding per term), and the runs are added up in double, so the result is at least as
 * accurate as an FP32 accumulation over all of K and far closer to the double sum than the tolerance of the
 * parity tests.  orc_matmul_exact is the plain double-accumulated loop nest (every test of small shapes, and
 * the check of the blocked form in tests/test_oracle_pins.py). */
#include <immintrin.h>

enum { GM_MR = 6, GM_NR = 16, GM_MB = 192, GM_NB = 256, GM_KB = 256 };

/* acc[GM_MR][GM_NR] (double) += ap[k][GM_MR] * bp[k][GM_NR] over kb terms */
static void gemm_micro(const float* ap, const float* bp, int kb, double* acc, int ldacc) {
    __m256 c[GM_MR][2];
    for (int i = 0; i < GM_MR; i++) { c[i][0] = _mm256_setzero_ps(); c[i][1] = _mm256_setzero_ps(); }
    for (int k = 0; k < kb; k++) {
        const __m256 b0 = _mm256_loadu_ps(bp + (size_t)k * GM_NR), b1 = _mm256_loadu_ps(bp + (size_t)k * GM_NR + 8);
        for (int i = 0; i < GM_MR; i++) {
            const __m256 a = _mm256_broadcast_ss(ap + (size_t)k * GM_MR + i);
            c[i][0] = _mm256_fmadd_ps(a, b0, c[i][0]);
            c[i][1] = _mm256_fmadd_ps(a, b1, c[i][1]);
        }
    }
    for (int i = 0; i < GM_MR; i++) {
        float t[GM_NR];
        _mm256_storeu_ps(t, c[i][0]); _mm256_storeu_ps(t + 8, c[i][1]);
        for (int j = 0; j < GM_NR; j++) acc[(size_t)i * ldacc + j] += (double)t[j];
    }
}

static void matmul_blocked(const float* A, const float* B, float* C,
                           int64_t M, int64_t N, int64_t K, int tA, int tB, int accumulate) {
    const int64_t sai = tA ? 1 : K, sak = tA ? M : 1;      /* A(i,k) = A[i*sai + k*sak] */
    const int64_t sbk = tB ? 1 : N, sbj = tB ? K : 1;      /* B(k,j) = B[k*sbk + j*sbj] */
    const int64_t mt = (M + GM_MB - 1) / GM_MB, nt = (N + GM_NB - 1) / GM_NB;
#pragma omp parallel
    {
        float* ap = (float*)aligned_alloc(64, sizeof(float) * GM_MB * GM_KB);
        float* bp = (float*)aligned_alloc(64, sizeof(float) * GM_NB * GM_KB);
        double* acc = (double*)malloc(sizeof(double) * GM_MB * GM_NB);
#pragma omp for collapse(2) schedule(dynamic, 1)
        for (int64_t ti = 0; ti < mt; ti++)
            for (int64_t tj = 0; tj < nt; tj++) {
                const int64_t i0 = ti * GM_MB, j0 = tj * GM_NB;
                const int mb = (int)(M - i0 < GM_MB ? M - i0 : GM_MB), nb = (int)(N - j0 < GM_NB ? N - j0 : GM_NB);
                memset(acc, 0, sizeof(double) * GM_MB * GM_NB);
                for (int64_t k0 = 0; k0 < K; k0 += GM_KB) {
                    const int kb = (int)(K - k0 < GM_KB ? K - k0 : GM_KB);
                    /* panels of GM_MR rows of A and GM_NR columns of B, k-major inside a panel, zero padded */
                    for (int pi = 0; pi < GM_MB / GM_MR; pi++) {
                        float* dst = ap + (size_t)pi * GM_MR * GM_KB;
                        if (pi * GM_MR >= mb) break;
                        for (int k = 0; k < kb; k++)
                            for (int i = 0; i < GM_MR; i++) {
                                const int ii = pi * GM_MR + i;
                                dst[(size_t)k * GM_MR + i] = ii < mb ? A[(i0 + ii) * sai + (k0 + k) * sak] : 0.0f;
                            }
                    }
                    for (int pj = 0; pj < GM_NB / GM_NR; pj++) {
                        float* dst = bp + (size_t)pj * GM_NR * GM_KB;
                        if (pj * GM_NR >= nb) break;
                        if (!tB && (pj + 1) * GM_NR <= nb) {
                            for (int k = 0; k < kb; k++) memcpy(dst + (size_t)k * GM_NR, B + (k0 + k) * sbk + (j0 + pj * GM_NR), sizeof(float) * GM_NR);
                        } else {
                            for (int j = 0; j < GM_NR; j++) {
                                const int jj = pj * GM_NR + j;
                                if (jj < nb) { const float* src = B + (j0 + jj) * sbj + k0 * sbk; for (int k = 0; k < kb; k++) dst[(size_t)k * GM_NR + j] = src[(int64_t)k * sbk]; }
                                else for (int k = 0; k < kb; k++) dst[(size_t)k * GM_NR + j] = 0.0f;
                            }
                        }
                    }
                    for (int pi = 0; pi * GM_MR < mb; pi++)
                        for (int pj = 0; pj * GM_NR < nb; pj++)
                            gemm_micro(ap + (size_t)pi * GM_MR * GM_KB, bp + (size_t)pj * GM_NR * GM_KB, kb,
                                       acc + (size_t)pi * GM_MR * GM_NB + pj * GM_NR, GM_NB);
                }
                for (int i = 0; i < mb; i++) {
                    float* crow = C + (i0 + i) * N + j0;
                    const double* arow = acc + (size_t)i * GM_NB;
                    if (accumulate) for (int j = 0; j < nb; j++) crow[j] = (float)((double)crow[j] + arow[j]);
                    else            for (int j = 0; j < nb; j++) crow[j] = (float)arow[j];
                }
            }
        free(ap); free(bp); free(acc);
    }
}

void orc_matmul_exact(const float* A, const float* B, float* C,
                      int64_t M, int64_t N, int64_t K, int tA, int tB, int accumulate) {
    /* Index expressions as shaders/matmul_transpose.comp:60-80. The loop nest
     * is arranged so the innermost stream is contiguous where it can be. */
#pragma omp parallel
    {
        double* acc = (double*)malloc((size_t)N * sizeof(double));
#pragma omp for schedule(static)
        for (int64_t i = 0; i < M; i++) {
            if (!tB) {
                for (int64_t j = 0; j < N; j++) acc[j] = 0.0;
                for (int64_t k = 0; k < K; k++) {
                    double a = tA ? A[k * M + i] : A[i * K + k];
                    const float* brow = B + k * N;
                    for (int64_t j = 0; j < N; j++) acc[j] += a * (double)brow[j];
                }
            } else {
                for (int64_t j = 0; j < N; j++) {
                    const float* bcol = B + j * K;
                    double s = 0.0;
                    if (!tA) {
                        const float* arow = A + i * K;
                        for (int64_t k = 0; k < K; k++) s += (double)arow[k] * (double)bcol[k];
                    } else {
                        for (int64_t k = 0; k < K; k++) s += (double)A[k * M + i] * (double)bcol[k];
                    }
                    acc[j] = s;
                }
            }
            float* crow = C + i * N;
            if (accumulate) for (int64_t j = 0; j < N; j++) crow[j] = (float)((double)crow[j] + acc[j]);
            else            for (int64_t j = 0; j < N; j++) crow[j] = (float)acc[j];
        }
        free(acc);
    }
}

void orc_matmul(const float* A, const float* B, float* C,
                int64_t M, int64_t N, int64_t K, int tA, int tB, int accumulate) {
    if (M >= 32 && N >= 32 && (double)M * (double)N * (double)K >= 33554432.0)
        matmul_blocked(A, B, C, M, N, K, tA, tB, accumulate);
    else
        orc_matmul_exact(A, B, C, M, N, K, tA, tB, accumulate);
}

/* ====================================================================== */
/* attention                                                              */
/* ====================================================================== */

static inline int64_t seq_begin_of(const uint32_t* starts, int batch, int64_t t) {
    if (!starts) return 0;
    return (int64_t)starts[find_seq(starts, batch, t)];
}

void orc_attention_forward(const float* Q, const float* K, const float* V,
                           float* out, float* lse,
                           const uint32_t* seq_starts, int batch, int64_t T,
                           int H, int KVH, int D, float scale) {
    int64_t qw = (int64_t)H * D, kw = (int64_t)KVH * D;
#pragma omp parallel
    {
        double* p = (double*)malloc((size_t)T * sizeof(double));
        double* o = (double*)malloc((size_t)D * sizeof(double));
#pragma omp for collapse(2) schedule(dynamic, 8)
        for (int64_t t = 0; t < T; t++) {
            for (int h = 0; h < H; h++) {
                int kvh = h * KVH / H;
                int64_t j0 = seq_begin_of(seq_starts, batch, t);
                const float* q = Q + t * qw + (int64_t)h * D;
                double mx = -1e300;
                for (int64_t j = j0; j <= t; j++) {
                    const float* k = K + j * kw + (int64_t)kvh * D;
                    double s = 0.0;
                    for (int d = 0; d < D; d++) s += (double)q[d] * (double)k[d];
                    s *= (double)scale;
                    p[j - j0] = s;
                    if (s > mx) mx = s;
                }
                double l = 0.0;
                for (int64_t j = j0; j <= t; j++) { p[j - j0] = exp(p[j - j0] - mx); l += p[j - j0]; }
                for (int d = 0; d < D; d++) o[d] = 0.0;
                for (int64_t j = j0; j <= t; j++) {
                    const float* v = V + j * kw + (int64_t)kvh * D;
                    double pj = p[j - j0] / l;
                    for (int d = 0; d < D; d++) o[d] += pj * (double)v[d];
                }
                float* dst = out + t * qw + (int64_t)h * D;
                for (int d = 0; d < D; d++) dst[d] = (float)o[d];
                if (lse) lse[t * H + h] = (float)(mx + log(l));
            }
        }
        free(p); free(o);
    }
}

void orc_attention_backward(const float* Q, const float* K, const float* V,
                            const float* dO, float* dQ, float* dK, float* dV,
                            const uint32_t* seq_starts, int batch, int64_t T,
                            int H, int KVH, int D, float scale) {
    int64_t qw = (int64_t)H * D, kw = (int64_t)KVH * D;
    /* The shader adds into dK/dV from every (head, query) workgroup with
     * atomics.  Here one thread owns one kv head, so sums need no atomics and
     * are carried in double until the end. */
    double* aK = (double*)calloc((size_t)T * kw, sizeof(double));
    double* aV = (double*)calloc((size_t)T * kw, sizeof(double));
#pragma omp parallel
    {
        double* p  = (double*)malloc((size_t)T * sizeof(double));
        double* dp = (double*)malloc((size_t)T * sizeof(double));
        double* dq = (double*)malloc((size_t)D * sizeof(double));
        /* one (kv head, packed sequence) pair per task: the pairs touch disjoint rows of aK / aV */
        const int nseq = seq_starts ? batch : 1;
#pragma omp for collapse(2) schedule(dynamic, 1)
        for (int kvh = 0; kvh < KVH; kvh++) {
          for (int sq = 0; sq < nseq; sq++) {
            const int64_t t_lo = seq_starts ? (int64_t)seq_starts[sq] : 0;
            const int64_t t_hi = seq_starts ? (int64_t)seq_starts[sq + 1] : T;
            for (int h = 0; h < H; h++) {
                if (h * KVH / H != kvh) continue;    /* batch_attention_backward.comp:58 */
                for (int64_t t = t_lo; t < t_hi && t < T; t++) {
                    int64_t j0 = t_lo;
                    const float* q  = Q  + t * qw + (int64_t)h * D;
                    const float* go = dO + t * qw + (int64_t)h * D;
                    double mx = -1e300;
                    for (int64_t j = j0; j <= t; j++) {
                        const float* k = K + j * kw + (int64_t)kvh * D;
                        double s = 0.0;
                        for (int d = 0; d < D; d++) s += (double)q[d] * (double)k[d];
                        s *= (double)scale;
                        p[j - j0] = s; if (s > mx) mx = s;
                    }
                    double l = 0.0;
                    for (int64_t j = j0; j <= t; j++) { p[j - j0] = exp(p[j - j0] - mx); l += p[j - j0]; }
                    double wsum = 0.0;
                    for (int64_t j = j0; j <= t; j++) {
                        const float* v = V + j * kw + (int64_t)kvh * D;
                        double pj = p[j - j0] / l;
                        p[j - j0] = pj;
                        double dot = 0.0;
                        double* av = aV + j * kw + (int64_t)kvh * D;
                        for (int d = 0; d < D; d++) {
                            dot += (double)go[d] * (double)v[d];
                            av[d] += pj * (double)go[d];          /* dV += p * dO */
                        }
                        dp[j - j0] = dot;
                        wsum += pj * dot;
                    }
                    for (int d = 0; d < D; d++) dq[d] = 0.0;
                    for (int64_t j = j0; j <= t; j++) {
                        double ds = p[j - j0] * (dp[j - j0] - wsum);
                        const float* k = K + j * kw + (int64_t)kvh * D;
                        double* ak = aK + j * kw + (int64_t)kvh * D;
                        for (int d = 0; d < D; d++) {
                            dq[d] += ds * (double)k[d];
                            ak[d] += (ds * (double)scale) * (double)q[d];   /* dK += scale*dS*Q */
                        }
                    }
                    float* dst = dQ + t * qw + (int64_t)h * D;
                    for (int d = 0; d < D; d++) dst[d] = (float)(dq[d] * (double)scale);
                }
            }
          }
        }
        free(p); free(dp); free(dq);
    }
    for (int64_t i = 0; i < T * kw; i++) {
        dK[i] = (float)((double)dK[i] + aK[i]);
        dV[i] = (float)((double)dV[i] + aV[i]);
    }
    free(aK); free(aV);
}

/* ====================================================================== */
/* rmsnorm, rope, qk_norm                                                 */
/* ====================================================================== */

void orc_rmsnorm(const float* x, const float* scale, float* y,
                 int64_t rows, int64_t cols, float eps) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        const float* xr = x + r * cols;
        double ss = 0.0;
        for (int64_t c = 0; c < cols; c++) ss += (double)xr[c] * (double)xr[c];
        double inv = 1.0 / sqrt(ss / (double)cols + (double)eps);
        for (int64_t c = 0; c < cols; c++) y[r * cols + c] = (float)((double)xr[c] * inv * (double)scale[c]);
    }
}

void orc_rmsnorm_backward_batch(const float* x, const float* scale, const float* dy,
                                float* dx, float* grad_scale,
                                int64_t rows, int64_t cols, float eps) {
    double* gs = (double*)calloc((size_t)cols, sizeof(double));
    double denom = cols > 1 ? (double)cols : 1.0;          /* max(1.0, cols) :56 */
#pragma omp parallel
    {
        double* lgs = (double*)calloc((size_t)cols, sizeof(double));
#pragma omp for schedule(static)
        for (int64_t r = 0; r < rows; r++) {
            const float* xr = x + r * cols;
            const float* gr = dy + r * cols;
            double ss = 0.0, cp = 0.0;
            for (int64_t c = 0; c < cols; c++) {
                ss += (double)xr[c] * (double)xr[c];
                cp += (double)gr[c] * (double)scale[c] * (double)xr[c];
            }
            double rms = sqrt(ss / denom + (double)eps);
            if (rms < 0.01) rms = 0.01;                      /* :59 */
            double inv = 1.0 / rms, inv3 = inv * inv * inv;
            double coupled = cp / denom;                     /* :79 */
            for (int64_t c = 0; c < cols; c++) {
                /* each term is rounded to float before it is added, :90 */
                lgs[c] += (double)(float)((double)gr[c] * (double)xr[c] * inv);
                dx[r * cols + c] = (float)((double)gr[c] * (double)scale[c] * inv
                                           - (double)xr[c] * (coupled * inv3));   /* :98 */
            }
        }
#pragma omp critical
        for (int64_t c = 0; c < cols; c++) gs[c] += lgs[c];
        free(lgs);
    }
    for (int64_t c = 0; c < cols; c++) grad_scale[c] = (float)((double)grad_scale[c] + gs[c]);
    free(gs);
}

void orc_rope_inv_freq(float* inv_freq, int D, float theta) {
    for (int i = 0; i < D / 2; i++) {
        float exponent = (float)(2 * i) / (float)D;
        inv_freq[i] = 1.0f / powf(theta, exponent);
    }
}

void orc_rope(const float* in, float* out, const uint32_t* seq_starts, int batch,
              int64_t T, int heads, int D, float theta, int backward) {
    float inv_freq[512];
    orc_rope_inv_freq(inv_freq, D, theta);
    int64_t w = (int64_t)heads * D;
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; t++) {
        int64_t pos = t - seq_begin_of(seq_starts, batch, t);
        for (int i = 0; i < D / 2; i++) {
            float angle = (float)pos * inv_freq[i];          /* FP32 product, :43 */
            double c = cos((double)angle), s = sin((double)angle);
            for (int h = 0; h < heads; h++) {
                int64_t i0 = t * w + (int64_t)h * D + 2 * i;
                double a = in[i0], b = in[i0 + 1];
                if (!backward) { out[i0] = (float)(a * c - b * s); out[i0 + 1] = (float)(a * s + b * c); }
                else           { out[i0] = (float)(a * c + b * s); out[i0 + 1] = (float)(-a * s + b * c); }
            }
        }
    }
}

void orc_qk_norm(float* qk, int64_t T, int heads, int D, float eps) {
    int64_t n = (int64_t)heads * D;
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; t++) {
        float* x = qk + t * n;
        double ss = 0.0;
        for (int64_t i = 0; i < n; i++) ss += (double)x[i] * (double)x[i];
        double rms = sqrt(ss / (double)n);
        if (rms < (double)eps) rms = (double)eps;
        for (int64_t i = 0; i < n; i++) x[i] = (float)((double)x[i] / rms);
    }
}

void orc_qk_norm_backward(const float* x_pre, const float* dy, float* dx,
                          int64_t T, int heads, int D, float eps) {
    int64_t n = (int64_t)heads * D;
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; t++) {
        const float* x = x_pre + t * n;
        const float* g = dy + t * n;
        double ss = 0.0, gx = 0.0;
        for (int64_t i = 0; i < n; i++) { ss += (double)x[i] * (double)x[i]; gx += (double)g[i] * (double)x[i]; }
        double rms = sqrt(ss / (double)n);
        if (rms < (double)eps) {
            /* clamped branch: y = x/eps with eps constant */
            for (int64_t i = 0; i < n; i++) dx[t * n + i] = (float)((double)g[i] / (double)eps);
        } else {
            double inv = 1.0 / rms, k = gx / ((double)n * rms * rms * rms);
            for (int64_t i = 0; i < n; i++) dx[t * n + i] = (float)((double)g[i] * inv - (double)x[i] * k);
        }
    }
}

/* ====================================================================== */
/* element-wise                                                           */
/* ====================================================================== */

void orc_silu(const float* x, float* y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) y[i] = (float)((double)x[i] / (1.0 + exp(-(double)x[i])));
}

void orc_silu_backward(const float* x, const float* dy, float* dx, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        double xv = x[i], s = 1.0 / (1.0 + exp(-xv));
        dx[i] = (float)((double)dy[i] * (s * (1.0 + xv * (1.0 - s))));
    }
}

void orc_mul_backward(const float* A, const float* B, const float* dC,
                      float* dA, float* dB, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        float a = A[i], b = B[i], g = dC[i];
        dA[i] = g * b;
        dB[i] = g * a;
    }
}

void orc_swiglu_backward(const float* gate, const float* up, const float* dH,
                         float* dGate, float* dUp, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        double x = gate[i], s = 1.0 / (1.0 + exp(-x));
        double silu = x * s;
        double g = dH[i];
        dUp[i]   = (float)(g * silu);
        dGate[i] = (float)((g * (double)up[i]) * (s * (1.0 + x * (1.0 - s))));
    }
}

/* ====================================================================== */
/* embedding                                                              */
/* ====================================================================== */

void orc_embed_lookup(const uint32_t* tokens, const float* embed, float* out,
                      int64_t T, int64_t hidden, int64_t vocab) {
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; t++) {
        if ((int64_t)tokens[t] >= vocab) memset(out + t * hidden, 0, (size_t)hidden * sizeof(float));
        else memcpy(out + t * hidden, embed + (int64_t)tokens[t] * hidden, (size_t)hidden * sizeof(float));
    }
}

void orc_embedding_backward(const uint32_t* tokens, const float* dH, float* grad_embed,
                            int64_t T, int64_t hidden, int64_t vocab) {
    /* first[t] = 1 when position t is the first occurrence of its token */
    double* acc = (double*)malloc((size_t)hidden * sizeof(double));
    char* done = (char*)calloc((size_t)T, 1);
    for (int64_t t = 0; t < T; t++) {
        if (done[t] || (int64_t)tokens[t] >= vocab) continue;
        for (int64_t c = 0; c < hidden; c++) acc[c] = 0.0;
        for (int64_t u = t; u < T; u++) {
            if (tokens[u] != tokens[t]) continue;
            done[u] = 1;
            for (int64_t c = 0; c < hidden; c++) acc[c] += (double)dH[u * hidden + c];
        }
        float* row = grad_embed + (int64_t)tokens[t] * hidden;
        for (int64_t c = 0; c < hidden; c++) row[c] = (float)((double)row[c] + acc[c]);
    }
    free(acc); free(done);
}

/* ====================================================================== */
/* AdamW                                                                  */
/* ====================================================================== */

void orc_adamw(float* w, const float* g, float* m, float* v, int64_t n,
               float lr, float beta1, float beta2, float weight_decay, float eps,
               int step, float clip) {
    float bc1 = 1.0f - powf(beta1, (float)step);     /* src/vulkan_backend.c:2151 */
    float bc2 = 1.0f - powf(beta2, (float)step);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        float gi = g[i];
        if (clip > 0.0f) gi = gi > clip ? clip : (gi < -clip ? -clip : gi);
        float wi = w[i];
        float mn = beta1 * m[i] + (1.0f - beta1) * gi;          /* adamw.comp:47 */
        m[i] = mn;
        float vn = beta2 * v[i] + (1.0f - beta2) * gi * gi;     /* :51 */
        v[i] = vn;
        float mh = mn / bc1, vh = vn / bc2;                      /* :55-56 */
        w[i] = wi * (1.0f - lr * weight_decay) - lr * mh / (sqrtf(vh) + eps);   /* :60 */
    }
}

int orc_nan_check(const float* x, int64_t n) {
    int bad = 0;
#pragma omp parallel for reduction(|:bad) schedule(static)
    for (int64_t i = 0; i < n; i++) bad |= (isnan(x[i]) || isinf(x[i])) ? 1 : 0;
    return bad;
}

float orc_lr_schedule(float base_lr, int optimizer_step, int accum_steps) {
    float warmup_steps = 100.0f, lr = base_lr;
    if ((float)optimizer_step < warmup_steps) lr = base_lr * ((float)optimizer_step / warmup_steps);
    if (accum_steps < 1) accum_steps = 1;
    return lr / (float)accum_steps;
}

/* ====================================================================== */
/* whole step                                                             */
/* ====================================================================== */

typedef struct {
    int64_t in_norm, q, k, v, o, post_norm, gate, up, down;
} layer_off_t;

typedef struct {
    int64_t embed, final_norm, layer0, layer_stride;
    layer_off_t rel;   /* offsets relative to the start of a layer */
} layout_t;

static layout_t make_layout(const orc_config_t* c) {
    layout_t L;
    int64_t h = c->hidden, qd = (int64_t)c->heads * c->head_dim, kv = (int64_t)c->kv_heads * c->head_dim, f = c->ffn;
    L.embed = 0;
    L.final_norm = (int64_t)c->vocab * h;
    L.layer0 = L.final_norm + h;
    int64_t o = 0;
    L.rel.in_norm = o; o += h;
    L.rel.q = o; o += qd * h;
    L.rel.k = o; o += kv * h;
    L.rel.v = o; o += kv * h;
    L.rel.o = o; o += h * qd;
    L.rel.post_norm = o; o += h;
    L.rel.gate = o; o += f * h;
    L.rel.up = o; o += f * h;
    L.rel.down = o; o += h * f;
    L.layer_stride = o;
    return L;
}

int64_t orc_param_count(const orc_config_t* c) {
    layout_t L = make_layout(c);
    return L.layer0 + L.layer_stride * c->layers;
}

/* per-layer LoRA block: for each selected projection, A[r,in] then B[out,r] */
typedef struct { int64_t A[7], B[7], in[7], out[7], stride; } lora_layout_t;

static lora_layout_t make_lora_layout(const orc_config_t* c) {
    lora_layout_t L;
    int64_t h = c->hidden, qd = (int64_t)c->heads * c->head_dim, kv = (int64_t)c->kv_heads * c->head_dim;
    int64_t f = c->ffn;
    int64_t ins[7]  = { h, h, h, qd, h, h, f };      /* q k v o gate up down: src/lora.c:372-396 */
    int64_t outs[7] = { qd, kv, kv, h, f, f, h };
    int64_t o = 0;
    for (int p = 0; p < 7; p++) {
        L.in[p] = ins[p]; L.out[p] = outs[p];
        L.A[p] = L.B[p] = -1;
        if (c->lora_rank > 0 && (c->lora_mask >> p) & 1) {
            L.A[p] = o; o += (int64_t)c->lora_rank * ins[p];
            L.B[p] = o; o += outs[p] * (int64_t)c->lora_rank;
        }
    }
    L.stride = o;
    return L;
}

int64_t orc_lora_param_count(const orc_config_t* c) {
    return make_lora_layout(c).stride * c->layers;
}

static float* fnew(int64_t n) { return (float*)calloc((size_t)(n > 0 ? n : 1), sizeof(float)); }

static void add_into(float* dst, const float* a, const float* b, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) dst[i] = a[i] + b[i];
}
static void scale_inplace(float* a, int64_t n, float s) {
    for (int64_t i = 0; i < n; i++) a[i] *= s;
}

/* src/train.c:5778-5796 */
static void lora_forward_add(const float* x, float* out, const float* A, const float* B, float* tmp,
                             int64_t T, int64_t in, int64_t outd, int r, float s) {
    orc_matmul(x, A, tmp, T, r, in, 0, 1, 0);
    scale_inplace(tmp, T * r, s);
    orc_matmul(tmp, B, out, T, outd, r, 0, 1, 1);
}

/* src/train.c:5803-5845 with grad_input == NULL */
static void lora_backward(const float* dY, const float* x, const float* A, const float* B,
                          float* gA, float* gB, float* tmp,
                          int64_t T, int64_t in, int64_t outd, int r, float s) {
    orc_matmul(x, A, tmp, T, r, in, 0, 1, 0);
    scale_inplace(tmp, T * r, s);
    orc_matmul(dY, tmp, gB, outd, r, T, 1, 0, 1);
    orc_matmul(dY, B, tmp, T, r, outd, 0, 0, 0);
    scale_inplace(tmp, T * r, s);
    orc_matmul(tmp, x, gA, r, in, T, 1, 0, 1);
}

static float step_impl(const orc_config_t* c, const float* P, float* G,
                       const float* LP, float* LG,
                       const int32_t* tokens_in, const int32_t* seq_starts_in, int batch, int64_t T) {
    const int lora = LP != NULL;
    layout_t L = make_layout(c);
    lora_layout_t LL = make_lora_layout(c);
    const int64_t h = c->hidden, f = c->ffn, V = c->vocab;
    const int H = c->heads, KVH = c->kv_heads, D = c->head_dim, NL = c->layers;
    const int64_t qd = (int64_t)H * D, kv = (int64_t)KVH * D;
    const float scale = 1.0f / sqrtf((float)D);          /* src/vulkan_backend_backward.c:1168 */
    const float eps = c->rms_eps;
    const int r = c->lora_rank;
    const float ls = r > 0 ? c->lora_alpha / (float)r : 0.0f;

    /* tokens / targets: src/train_cuda.c:2029-2043 (negative ids -> 0) */
    uint32_t* starts = (uint32_t*)malloc((size_t)(batch + 1) * sizeof(uint32_t));
    if (seq_starts_in) for (int b = 0; b <= batch; b++) starts[b] = (uint32_t)seq_starts_in[b];
    else { starts[0] = 0; starts[1] = (uint32_t)T; batch = 1; }
    uint32_t* tok = (uint32_t*)malloc((size_t)T * sizeof(uint32_t));
    uint32_t* tgt = (uint32_t*)malloc((size_t)T * sizeof(uint32_t));
    for (int b = 0; b < batch; b++)
        for (int64_t t = starts[b]; t < (int64_t)starts[b + 1]; t++) {
            tok[t] = tokens_in[t] < 0 ? 0u : (uint32_t)tokens_in[t];
            if (t < (int64_t)starts[b + 1] - 1) tgt[t] = tokens_in[t + 1] < 0 ? 0u : (uint32_t)tokens_in[t + 1];
            else tgt[t] = 0;
        }
    int64_t num_valid = T - batch;

    /* saved activations */
    float **layer_in = calloc(NL, sizeof(float*)), **xn_attn = calloc(NL, sizeof(float*)),
          **cq = calloc(NL, sizeof(float*)), **ck = calloc(NL, sizeof(float*)), **cv = calloc(NL, sizeof(float*)),
          **attn_out = calloc(NL, sizeof(float*)), **post_in = calloc(NL, sizeof(float*)),
          **xn_ffn = calloc(NL, sizeof(float*)), **gate = calloc(NL, sizeof(float*)),
          **up = calloc(NL, sizeof(float*)), **silu_out = calloc(NL, sizeof(float*)),
          **ffn_h = calloc(NL, sizeof(float*)), **pq = calloc(NL, sizeof(float*)), **pk = calloc(NL, sizeof(float*));
    float* hidden = fnew(T * h);
    float* tmp_h = fnew(T * h);
    float* ltmp = fnew(T * (r > 0 ? r : 1));

    orc_embed_lookup(tok, P + L.embed, hidden, T, h, V);
    for (int l = 0; l < NL; l++) {
        const float* W = P + L.layer0 + L.layer_stride * l;
        const float* LW = lora ? LP + LL.stride * l : NULL;
        layer_in[l] = fnew(T * h); memcpy(layer_in[l], hidden, (size_t)(T * h) * 4);
        xn_attn[l] = fnew(T * h);
        orc_rmsnorm(hidden, W + L.rel.in_norm, xn_attn[l], T, h, eps);
        cq[l] = fnew(T * qd); ck[l] = fnew(T * kv); cv[l] = fnew(T * kv);
        orc_matmul(xn_attn[l], W + L.rel.q, cq[l], T, qd, h, 0, 1, 0);
        if (lora && LL.A[0] >= 0) lora_forward_add(xn_attn[l], cq[l], LW + LL.A[0], LW + LL.B[0], ltmp, T, h, qd, r, ls);
        orc_matmul(xn_attn[l], W + L.rel.k, ck[l], T, kv, h, 0, 1, 0);
        if (lora && LL.A[1] >= 0) lora_forward_add(xn_attn[l], ck[l], LW + LL.A[1], LW + LL.B[1], ltmp, T, h, kv, r, ls);
        orc_matmul(xn_attn[l], W + L.rel.v, cv[l], T, kv, h, 0, 1, 0);
        if (lora && LL.A[2] >= 0) lora_forward_add(xn_attn[l], cv[l], LW + LL.A[2], LW + LL.B[2], ltmp, T, h, kv, r, ls);
        orc_rope(cq[l], cq[l], starts, batch, T, H, D, c->rope_theta, 0);
        orc_rope(ck[l], ck[l], starts, batch, T, KVH, D, c->rope_theta, 0);
        if (c->use_qk_norm) {                                    /* src/train.c:4687-4689; the inputs are kept for the derivative */
            pq[l] = fnew(T * qd); memcpy(pq[l], cq[l], (size_t)(T * qd) * 4);
            pk[l] = fnew(T * kv); memcpy(pk[l], ck[l], (size_t)(T * kv) * 4);
            orc_qk_norm(cq[l], T, H, D, eps);
            orc_qk_norm(ck[l], T, KVH, D, eps);
        }
        attn_out[l] = fnew(T * qd);
        orc_attention_forward(cq[l], ck[l], cv[l], attn_out[l], NULL, starts, batch, T, H, KVH, D, scale);
        orc_matmul(attn_out[l], W + L.rel.o, tmp_h, T, h, qd, 0, 1, 0);
        if (lora && LL.A[3] >= 0) lora_forward_add(attn_out[l], tmp_h, LW + LL.A[3], LW + LL.B[3], ltmp, T, qd, h, r, ls);
        add_into(hidden, hidden, tmp_h, T * h);
        post_in[l] = fnew(T * h); memcpy(post_in[l], hidden, (size_t)(T * h) * 4);
        xn_ffn[l] = fnew(T * h);
        orc_rmsnorm(hidden, W + L.rel.post_norm, xn_ffn[l], T, h, eps);
        gate[l] = fnew(T * f); up[l] = fnew(T * f); silu_out[l] = fnew(T * f); ffn_h[l] = fnew(T * f);
        orc_matmul(xn_ffn[l], W + L.rel.gate, gate[l], T, f, h, 0, 1, 0);
        if (lora && LL.A[4] >= 0) lora_forward_add(xn_ffn[l], gate[l], LW + LL.A[4], LW + LL.B[4], ltmp, T, h, f, r, ls);
        orc_matmul(xn_ffn[l], W + L.rel.up, up[l], T, f, h, 0, 1, 0);
        if (lora && LL.A[5] >= 0) lora_forward_add(xn_ffn[l], up[l], LW + LL.A[5], LW + LL.B[5], ltmp, T, h, f, r, ls);
        orc_silu(gate[l], silu_out[l], T * f);
        for (int64_t i = 0; i < T * f; i++) ffn_h[l][i] = silu_out[l][i] * up[l][i];
        orc_matmul(ffn_h[l], W + L.rel.down, tmp_h, T, h, f, 0, 1, 0);
        if (lora && LL.A[6] >= 0) lora_forward_add(ffn_h[l], tmp_h, LW + LL.A[6], LW + LL.B[6], ltmp, T, f, h, r, ls);
        add_into(hidden, hidden, tmp_h, T * h);
    }
    float* final_in = fnew(T * h); memcpy(final_in, hidden, (size_t)(T * h) * 4);
    float* xn_final = fnew(T * h);
    orc_rmsnorm(hidden, P + L.final_norm, xn_final, T, h, eps);
    float* logits = fnew(T * V);
    orc_matmul(xn_final, P + L.embed, logits, T, V, h, 0, 1, 0);     /* tied head, src/train.c:4869-4872 */

    /* loss */
    float* glog = fnew(T * V);
    float* loss_rows = fnew(T);
    orc_cross_entropy_grad_packed(logits, tgt, glog, loss_rows, starts, T, batch, V, num_valid);
    double loss_sum = 0.0;
    for (int64_t t = 0; t < T; t++) loss_sum += loss_rows[t];
    float loss = num_valid > 0 ? (float)(loss_sum / (double)num_valid) : 0.0f;
    free(logits);

    /* backward */
    float* g_hidden = fnew(T * h);
    float* g_tmp = fnew(T * h);
    float* g_xn = fnew(T * h);
    float* scratch_gs = fnew(h);
    orc_matmul(glog, P + L.embed, g_hidden, T, h, V, 0, 0, 0);                      /* LM head dgrad */
    if (!lora) orc_matmul(glog, xn_final, G + L.embed, V, h, T, 1, 0, 1);           /* LM head wgrad */
    free(glog);
    orc_rmsnorm_backward_batch(final_in, P + L.final_norm, g_hidden, g_tmp,
                               lora ? scratch_gs : G + L.final_norm, T, h, eps);
    memcpy(g_hidden, g_tmp, (size_t)(T * h) * 4);

    float* g_ffn = fnew(T * f); float* g_gate = fnew(T * f); float* g_up = fnew(T * f);
    float* g_attn = fnew(T * qd); float* g_q = fnew(T * qd); float* g_k = fnew(T * kv); float* g_v = fnew(T * kv);
    for (int l = NL - 1; l >= 0; l--) {
        const float* W = P + L.layer0 + L.layer_stride * l;
        float* GW = lora ? NULL : G + L.layer0 + L.layer_stride * l;
        const float* LW = lora ? LP + LL.stride * l : NULL;
        float* LGW = lora ? LG + LL.stride * l : NULL;

        if (!lora) orc_matmul(g_hidden, ffn_h[l], GW + L.rel.down, h, f, T, 1, 0, 1);
        orc_matmul(g_hidden, W + L.rel.down, g_ffn, T, f, h, 0, 0, 0);
        if (lora && LL.A[6] >= 0)                                            /* src/train.c:6422-6429 */
            lora_backward(g_hidden, ffn_h[l], LW + LL.A[6], LW + LL.B[6], LGW + LL.A[6], LGW + LL.B[6], ltmp, T, f, h, r, ls);
        orc_mul_backward(silu_out[l], up[l], g_ffn, g_gate, g_up, T * f);
        orc_silu_backward(gate[l], g_gate, g_gate, T * f);
        if (lora && LL.A[4] >= 0)                                            /* src/train.c:6446-6461 */
            lora_backward(g_gate, xn_ffn[l], LW + LL.A[4], LW + LL.B[4], LGW + LL.A[4], LGW + LL.B[4], ltmp, T, h, f, r, ls);
        if (lora && LL.A[5] >= 0)
            lora_backward(g_up, xn_ffn[l], LW + LL.A[5], LW + LL.B[5], LGW + LL.A[5], LGW + LL.B[5], ltmp, T, h, f, r, ls);
        if (!lora) {
            orc_matmul(g_gate, xn_ffn[l], GW + L.rel.gate, f, h, T, 1, 0, 1);
            orc_matmul(g_up, xn_ffn[l], GW + L.rel.up, f, h, T, 1, 0, 1);
        }
        orc_matmul(g_gate, W + L.rel.gate, g_xn, T, h, f, 0, 0, 0);
        orc_matmul(g_up, W + L.rel.up, g_tmp, T, h, f, 0, 0, 0);
        add_into(g_xn, g_xn, g_tmp, T * h);
        orc_rmsnorm_backward_batch(post_in[l], W + L.rel.post_norm, g_xn, g_tmp,
                                   lora ? scratch_gs : GW + L.rel.post_norm, T, h, eps);
        add_into(g_hidden, g_tmp, g_hidden, T * h);

        if (!lora) orc_matmul(g_hidden, attn_out[l], GW + L.rel.o, h, qd, T, 1, 0, 1);
        orc_matmul(g_hidden, W + L.rel.o, g_attn, T, qd, h, 0, 0, 0);
        if (lora && LL.A[3] >= 0)
            lora_backward(g_hidden, attn_out[l], LW + LL.A[3], LW + LL.B[3], LGW + LL.A[3], LGW + LL.B[3], ltmp, T, qd, h, r, ls);
        memset(g_k, 0, (size_t)(T * kv) * 4); memset(g_v, 0, (size_t)(T * kv) * 4);
        orc_attention_backward(cq[l], ck[l], cv[l], g_attn, g_q, g_k, g_v, starts, batch, T, H, KVH, D, scale);
        if (c->use_qk_norm) {
            float* tq = fnew(T * qd); float* tk = fnew(T * kv);
            orc_qk_norm_backward(pq[l], g_q, tq, T, H, D, eps);
            orc_qk_norm_backward(pk[l], g_k, tk, T, KVH, D, eps);
            memcpy(g_q, tq, (size_t)(T * qd) * 4); memcpy(g_k, tk, (size_t)(T * kv) * 4);
            free(tq); free(tk);
        }
        orc_rope(g_q, g_q, starts, batch, T, H, D, c->rope_theta, 1);
        orc_rope(g_k, g_k, starts, batch, T, KVH, D, c->rope_theta, 1);
        if (!lora) {
            orc_matmul(g_q, xn_attn[l], GW + L.rel.q, qd, h, T, 1, 0, 1);
            orc_matmul(g_k, xn_attn[l], GW + L.rel.k, kv, h, T, 1, 0, 1);
            orc_matmul(g_v, xn_attn[l], GW + L.rel.v, kv, h, T, 1, 0, 1);
        } else {
            if (LL.A[0] >= 0) lora_backward(g_q, xn_attn[l], LW + LL.A[0], LW + LL.B[0], LGW + LL.A[0], LGW + LL.B[0], ltmp, T, h, qd, r, ls);
            if (LL.A[1] >= 0) lora_backward(g_k, xn_attn[l], LW + LL.A[1], LW + LL.B[1], LGW + LL.A[1], LGW + LL.B[1], ltmp, T, h, kv, r, ls);
            if (LL.A[2] >= 0) lora_backward(g_v, xn_attn[l], LW + LL.A[2], LW + LL.B[2], LGW + LL.A[2], LGW + LL.B[2], ltmp, T, h, kv, r, ls);
        }
        orc_matmul(g_q, W + L.rel.q, g_xn, T, h, qd, 0, 0, 0);
        orc_matmul(g_k, W + L.rel.k, g_tmp, T, h, kv, 0, 0, 0);
        add_into(g_xn, g_xn, g_tmp, T * h);
        orc_matmul(g_v, W + L.rel.v, g_tmp, T, h, kv, 0, 0, 0);
        add_into(g_xn, g_xn, g_tmp, T * h);
        orc_rmsnorm_backward_batch(layer_in[l], W + L.rel.in_norm, g_xn, g_tmp,
                                   lora ? scratch_gs : GW + L.rel.in_norm, T, h, eps);
        add_into(g_hidden, g_tmp, g_hidden, T * h);
    }
    if (!lora) orc_embedding_backward(tok, g_hidden, G + L.embed, T, h, V);

    for (int l = 0; l < NL; l++) {
        free(layer_in[l]); free(xn_attn[l]); free(cq[l]); free(ck[l]); free(cv[l]); free(attn_out[l]);
        free(post_in[l]); free(xn_ffn[l]); free(gate[l]); free(up[l]); free(silu_out[l]); free(ffn_h[l]);
        free(pq[l]); free(pk[l]);
    }
    free(pq); free(pk);
    free(layer_in); free(xn_attn); free(cq); free(ck); free(cv); free(attn_out); free(post_in);
    free(xn_ffn); free(gate); free(up); free(silu_out); free(ffn_h);
    free(hidden); free(tmp_h); free(ltmp); free(final_in); free(xn_final); free(loss_rows);
    free(g_hidden); free(g_tmp); free(g_xn); free(scratch_gs); free(g_ffn); free(g_gate); free(g_up);
    free(g_attn); free(g_q); free(g_k); free(g_v); free(starts); free(tok); free(tgt);
    return loss;
}

float orc_step_full(const orc_config_t* c, const float* params, float* grads,
                    const int32_t* tokens, const int32_t* seq_starts, int batch, int64_t T) {
    return step_impl(c, params, grads, NULL, NULL, tokens, seq_starts, batch, T);
}

float orc_step_lora(const orc_config_t* c, const float* params, const float* lora,
                    float* lora_grads, const int32_t* tokens,
                    const int32_t* seq_starts, int batch, int64_t T) {
    return step_impl(c, params, NULL, lora, lora_grads, tokens, seq_starts, batch, T);
}
