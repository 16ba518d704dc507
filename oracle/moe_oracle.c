/*
 * Plain-C restatement of the OPMX mixture-of-experts operators.
 * TEST INFRASTRUCTURE ONLY: this file is the checker for the HIP kernels and
 * an independent second opinion on moe_oracle.py.  The product library never
 * links or loads it.
 *
 * Everything works on float32 buffers (callers up-cast fp16/bf16 exactly) and
 * accumulates in double, so results are "as exact as float32 inputs allow";
 * callers round once to the output dtype.
 *
 * Reference files followed (OpenPPL/ppl.pmx):
 *   torch_function/MoeSelect.py:37-64               oracle_moe_select, oracle_expand_rows
 *   torch_function/MoeColumnParallelLinear.py:58-69 oracle_grouped_linear
 *   torch_function/MoeRowParallelLinear.py:44-60    oracle_grouped_linear (bias per expert)
 *   torch_function/SwiGLU.py:15-16                  oracle_swiglu
 *   torch_function/SiLU.py:18-21                    oracle_silu
 *   torch_function/MoeReduce.py:23-25               oracle_moe_reduce
 *   torch_function/Linear.py:32                     oracle_linear
 * Tie rule: among equal scores the LOWER expert id is picked first; NaN ranks
 * above every number; -0.0 equals +0.0.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* "a ranks strictly before b": value descending, NaN first. Ids break ties
 * because candidates are scanned in ascending id and only a strict win
 * replaces the incumbent. */
static int ranks_before(float a, float b)
{
    int an = isnan(a), bn = isnan(b);
    if (an || bn) return an && !bn;
    return a > b;              /* -0.0 > +0.0 is false both ways: equal */
}

/* MoeSelect.py:40-60.  scores [T,E]; outputs idx [T,k], w [T,k] (softmax of
 * the k picked values, MoeSelect.py:41), inv [T*k], off [E+1]. Returns 0. */
int oracle_moe_select(const float *scores, int64_t T, int E, int k,
                      int64_t *idx, float *w, int64_t *inv, int64_t *off)
{
    if (E <= 0 || k <= 0 || k > E) return -1;
    char *taken = (char *)malloc((size_t)E);
    int64_t *cursor = (int64_t *)calloc((size_t)E + 1, sizeof(int64_t));
    if (!taken || !cursor) { free(taken); free(cursor); return -2; }

    for (int64_t t = 0; t < T; ++t) {
        const float *s = scores + t * E;
        memset(taken, 0, (size_t)E);
        for (int j = 0; j < k; ++j) {                 /* k rounds of arg-best */
            int best = -1;
            for (int e = 0; e < E; ++e) {
                if (taken[e]) continue;
                if (best < 0 || ranks_before(s[e], s[best])) best = e;
            }
            taken[best] = 1;
            idx[t * k + j] = best;
        }
        double m = s[idx[t * k]], sum = 0.0;           /* first pick is the max */
        for (int j = 0; j < k; ++j) sum += exp((double)s[idx[t * k + j]] - m);
        for (int j = 0; j < k; ++j)
            w[t * k + j] = (float)(exp((double)s[idx[t * k + j]] - m) / sum);
    }

    /* expert_offset[e] = #{picks with id < e}            MoeSelect.py:54-60 */
    for (int64_t j = 0; j < T * k; ++j) cursor[idx[j] + 1]++;
    off[0] = 0;
    for (int e = 0; e < E; ++e) off[e + 1] = off[e] + cursor[e + 1];
    /* stable sort by expert id == counting sort in flat order; inv[j] is the
     * sorted position of flat element j                  MoeSelect.py:44-52 */
    for (int e = 0; e < E; ++e) cursor[e] = off[e];
    for (int64_t j = 0; j < T * k; ++j) inv[j] = cursor[idx[j]]++;
    free(taken); free(cursor);
    return 0;
}

/* X_expand_permute[inv[t*k+s]] = X[t]                    MoeSelect.py:45-47 */
void oracle_expand_rows(const float *X, int64_t T, int64_t H, int k,
                        const int64_t *inv, float *Xp)
{
    for (int64_t j = 0; j < T * k; ++j)
        memcpy(Xp + inv[j] * H, X + (j / k) * H, (size_t)H * sizeof(float));
}

/* Y[r] = X[r] @ W[e]^T (+ B[e]) for off[e] <= r < off[e+1]; other rows 0. */
void oracle_grouped_linear(const float *X, const int64_t *off, const float *W,
                           const float *B, int E, int64_t R, int64_t K, int64_t N,
                           float *Y)
{
    memset(Y, 0, (size_t)(R * N) * sizeof(float));
    for (int e = 0; e < E; ++e) {
        int64_t lo = off[e], hi = off[e + 1];
        if (hi - lo <= 0) continue;
        const float *We = W + (int64_t)e * N * K;
#pragma omp parallel for collapse(2) schedule(static)
        for (int64_t r = lo; r < hi; ++r)
            for (int64_t n = 0; n < N; ++n) {
                const float *x = X + r * K, *wr = We + n * K;
                double a = 0.0;
                for (int64_t c = 0; c < K; ++c) a += (double)x[c] * (double)wr[c];
                if (B) a += (double)B[(int64_t)e * N + n];
                Y[r * N + n] = (float)a;
            }
    }
}

/* Linear.py:32 */
void oracle_linear(const float *X, const float *W, const float *B, int64_t T,
                   int64_t K, int64_t N, float *Y)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t t = 0; t < T; ++t)
        for (int64_t n = 0; n < N; ++n) {
            double a = 0.0;
            for (int64_t c = 0; c < K; ++c) a += (double)X[t * K + c] * (double)W[n * K + c];
            if (B) a += (double)B[n];
            Y[t * N + n] = (float)a;
        }
}

/* SwiGLU.py:15-16: X [R,2D] -> Y [R,D]; x = first half, g = second half. */
void oracle_swiglu(const float *X, int64_t R, int64_t D, float beta, float *Y)
{
    for (int64_t r = 0; r < R; ++r)
        for (int64_t i = 0; i < D; ++i) {
            double x = X[r * 2 * D + i], g = X[r * 2 * D + D + i];
            Y[r * D + i] = (float)(g * x / (1.0 + exp(-(double)beta * x)));
        }
}

/* SiLU.py:18-21: gate * x * sigmoid(x); gate may be NULL. */
void oracle_silu(const float *X, const float *gate, int64_t n, float *Y)
{
    for (int64_t i = 0; i < n; ++i) {
        double x = X[i], y = x / (1.0 + exp(-x));
        Y[i] = (float)(gate ? (double)gate[i] * y : y);
    }
}

/* MoeReduce.py:23-25: out[t] = sum_s w[t,s] * Y[inv[t,s]] */
void oracle_moe_reduce(const float *Y, const float *w, const int64_t *inv,
                       int64_t T, int k, int64_t N, float *out)
{
    for (int64_t t = 0; t < T; ++t)
        for (int64_t n = 0; n < N; ++n) {
            double a = 0.0;
            for (int s = 0; s < k; ++s)
                a += (double)w[t * k + s] * (double)Y[inv[t * k + s] * N + n];
            out[t * N + n] = (float)a;
        }
}
