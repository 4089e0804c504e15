/*
 * dwconv_oracle.c -- TEST INFRASTRUCTURE ONLY (never linked into or called by the product).
 *
 * A CPU restatement, straight from the definition, of the varlen depthwise 1-D convolution that
 * libnplm_dwconv computes on the GPU. Inputs are fp32 (bf16 test data is upcast before the call),
 * every sum is accumulated in double and returned in double.
 *
 * What it follows: the reference snapshot (peymanvahidi/nanoplm 0.1.6) contains no convolution, so
 * there is no reference function to restate. The definition is the one the reference path named
 * for this op computes -- torch.nn.functional.conv1d(x_i.T[None], w[:,None,:], b,
 * padding=(K-1)//2, groups=C) applied to each sequence i of the packed tensor (torch >= 2.8.0,
 * /root/reference/pyproject.toml:39) -- i.e. cross-correlation, zero padding at both ends of each
 * sequence, no kernel flip. The packed layout and cu_seqlens convention are those of
 * /root/reference/src/nanoplm/pretraining/collator.py:308-325 (int32 cumulative lengths,
 * cu[0] = 0) and modeling.py:339 ((total_tokens, hidden) activations).
 *
 * Parity status: pinned. tests/test_oracle.py checks these functions against the library routine
 * (per-sequence F.conv1d and its autograd, fp64), closed forms (K = 1, delta kernel, all-ones
 * kernel = clipped window sums, length-1 sequences), the adjoint/bilinear identities, finite
 * differences and the committed golden vectors under tests/golden/.
 *
 * Build: see oracle/Makefile (gcc -O2 -fopenmp -shared).
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* returns 0, or 1 if cu violates cu[0] == 0, non-decreasing, cu[S] == T, or K is even */
static int check_inputs(const int32_t* cu, int64_t T, int32_t K, int32_t S) {
    if (K < 1 || (K % 2) == 0 || S < 0) return 1;
    if (cu[0] != 0 || (int64_t)cu[S] != T) return 1;
    for (int32_t i = 0; i < S; ++i)
        if (cu[i + 1] < cu[i]) return 1;
    return 0;
}

/* y[t,c] = b[c] + sum_k w[c,k] * x[t+k-P, c] over taps that stay inside t's sequence */
int nplm_oracle_dwconv_fwd(const float* x, const int32_t* cu, const float* w, const float* b, double* y,
                           int64_t T, int32_t C, int32_t K, int32_t S) {
    if (check_inputs(cu, T, K, S)) return 1;
    const int P = (K - 1) / 2;
#pragma omp parallel for schedule(dynamic, 1)
    for (int32_t i = 0; i < S; ++i) {
        const int64_t s = cu[i], e = cu[i + 1];
        for (int64_t t = s; t < e; ++t) {
            for (int32_t c = 0; c < C; ++c) {
                double acc = b ? (double)b[c] : 0.0;
                for (int32_t k = 0; k < K; ++k) {
                    const int64_t j = t + k - P;
                    if (j >= s && j < e) acc += (double)w[(size_t)c * K + k] * (double)x[(size_t)j * C + c];
                }
                y[(size_t)t * C + c] = acc;
            }
        }
    }
    return 0;
}

/*
 * dx[t,c] = sum_k w[c,k] * dy[t-k+P, c]   (taps inside t's sequence)
 * dw[c,k] = sum_t dy[t,c] * x[t+k-P, c]   (taps inside t's sequence)
 * db[c]   = sum_t dy[t,c]
 * Any of dx / dw / db may be NULL to skip it.
 */
int nplm_oracle_dwconv_bwd(const float* x, const float* dy, const int32_t* cu, const float* w, double* dx,
                           double* dw, double* db, int64_t T, int32_t C, int32_t K, int32_t S) {
    if (check_inputs(cu, T, K, S)) return 1;
    const int P = (K - 1) / 2;
    if (dx) {
#pragma omp parallel for schedule(dynamic, 1)
        for (int32_t i = 0; i < S; ++i) {
            const int64_t s = cu[i], e = cu[i + 1];
            for (int64_t t = s; t < e; ++t)
                for (int32_t c = 0; c < C; ++c) {
                    double acc = 0.0;
                    for (int32_t k = 0; k < K; ++k) {
                        const int64_t j = t - k + P;
                        if (j >= s && j < e) acc += (double)w[(size_t)c * K + k] * (double)dy[(size_t)j * C + c];
                    }
                    dx[(size_t)t * C + c] = acc;
                }
        }
    }
    if (dw) memset(dw, 0, sizeof(double) * (size_t)C * K);
    if (db) memset(db, 0, sizeof(double) * (size_t)C);
    if (dw || db) {
#pragma omp parallel
        {
            double* lw = (double*)calloc((size_t)C * K, sizeof(double));
            double* lb = (double*)calloc((size_t)C, sizeof(double));
#pragma omp for schedule(dynamic, 1)
            for (int32_t i = 0; i < S; ++i) {
                const int64_t s = cu[i], e = cu[i + 1];
                for (int64_t t = s; t < e; ++t)
                    for (int32_t c = 0; c < C; ++c) {
                        const double g = (double)dy[(size_t)t * C + c];
                        lb[c] += g;
                        for (int32_t k = 0; k < K; ++k) {
                            const int64_t j = t + k - P;
                            if (j >= s && j < e) lw[(size_t)c * K + k] += g * (double)x[(size_t)j * C + c];
                        }
                    }
            }
#pragma omp critical
            {
                if (dw) for (size_t n = 0; n < (size_t)C * K; ++n) dw[n] += lw[n];
                if (db) for (size_t n = 0; n < (size_t)C; ++n) db[n] += lb[n];
            }
            free(lw);
            free(lb);
        }
    }
    return 0;
}
