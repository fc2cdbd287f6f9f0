/*
 * CPU oracle for the Multiply-And-Max/min (MAM) fully-connected hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the HIP library, the torch
 * binding, the Python package) may link, import or call this file; it exists so
 * that tests, the smoke check and the benchmark's cpu_baseline leg have an
 * independent statement of the algorithm to compare the GPU path against.
 *
 * Each function restates the reference algorithm (SSIGPRO/mamtorch 1.5.2):
 *   forward   : test/reference.py:3-10 (products, max/min along k, sum, + bias)
 *               mamtorch/kernel/v1/csrc/cuda/fullyconnected.cu:126-143 (k ascending,
 *               strict > and <  => the LOWEST k attaining the extreme wins)
 *               mamtorch/nn/v4/fullyconnected.py:197-198 (bias added after max+min)
 *   backward  : test/reference.py:12-25 (beta = 0 branch) and
 *               mamtorch/kernel/v4/csrc/cuda/fullyconnected_backward.cu:54-75
 *               (two scatter-adds per output; argmax == argmin counts twice)
 *   selection : mamtorch/nn/v4/fullyconnected.py:114-129
 *   CSR       : operand layout of mamtorch/sparse/kernel/v1/csrc/cuda/cusparsemm_csr.cu:25-45
 *               (int64 crow/col, fp32 values); MAM semantics over a pruned weight are
 *               "equal to the dense forward on the densified weight", because the
 *               reference prunes by writing literal zeros into dense weights
 *               (examples/vitb16_imagenet1k/pruning_utils.py:107,111).
 *
 *   SpMM      : mamtorch/sparse/kernel/v1/csrc/cuda/cusparsemm_csr.cu:19-77 and
 *               cusparsemm_coo.cu:19-76: C = A_sparse @ B with alpha 1, beta 0 through
 *               cuSPARSE (third party, absent here; the reference's own test only prints
 *               the max-abs error against the dense a@b, test/test_sparse.py:33-44).  The
 *               restatement is the defining sum, accumulated in fp64; it returns the sum of
 *               |terms| as well, which is what a tolerance for any fp32 summation order
 *               is made of.  Pinned against numpy's dense matmul and scipy.sparse.
 *
 * Arithmetic: every product is ONE round-to-nearest fp32 multiply, max+min is one
 * fp32 add, bias one more fp32 add.  Build with -ffp-contract=off.
 *
 * Parity status: all functions are pinned by tests/test_oracle.py (hand-derived
 * known answers, a pure-Python brute force, closed-form special cases, autograd
 * of a gather formulation, fp64 finite differences).  None is "parity unpinned".
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define MAM_W_KM 0 /* w is (K, M) row-major : the operator's "b" operand          */
#define MAM_W_MK 1 /* w is (M, K) row-major : nn.Module weight (out, in) layout   */

static inline float w_at(const float *w, int64_t ldw, int layout, int64_t k, int64_t m)
{
    return layout == MAM_W_MK ? w[m * ldw + k] : w[k * ldw + m];
}

/*
 * y[n,m] = (max_k x[n,k]*w[k,m] + min_k x[n,k]*w[k,m]) + bias[m]; first-index ties.
 * The scan is the reference kernel's (mamtorch/kernel/v1/csrc/cuda/fullyconnected.cu:68-78,132-142): the
 * accumulators start below / above every float with index 0 (the reference starts the max at FLT_MIN, a bug
 * that the build does not reproduce: -inf here), k ascends, and a product replaces an extreme only when an
 * ORDERED compare says it is strictly greater / smaller.  A NaN product therefore never wins and never
 * sticks, wherever it stands; a column of NaN products keeps (-inf, index 0) and (+inf, index 0), and so
 * does an extreme whose only candidates equal the starting infinity.
 */
void mam_oracle_forward(const float *x, int64_t ldx, const float *w, int64_t ldw, int layout,
                        const float *bias, float *c, int32_t *argmax, int32_t *argmin,
                        int64_t N, int64_t K, int64_t M)
{
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        for (int64_t m = 0; m < M; ++m) {
            float vmax = -__builtin_inff(), vmin = __builtin_inff();
            int32_t imax = 0, imin = 0;
            for (int64_t k = 0; k < K; ++k) {
                volatile float p = x[n * ldx + k] * w_at(w, ldw, layout, k, m);
                if (p > vmax) { vmax = p; imax = (int32_t)k; }
                if (p < vmin) { vmin = p; imin = (int32_t)k; }
            }
            volatile float s = vmax + vmin;
            if (bias) s = s + bias[m];
            c[n * M + m] = s;
            if (argmax) argmax[n * M + m] = imax;
            if (argmin) argmin[n * M + m] = imin;
        }
    }
}

/*
 * x_grad[n,k] = sum_m g[n,m] * w[k,m] * ([k==argmax[n,m]] + [k==argmin[n,m]])
 * w_grad[k,m] = sum_n g[n,m] * x[n,k] * (same)
 * Each term is an fp32 product (as the reference's atomicAdd operand); the sums are
 * accumulated in fp64 and rounded once, so the oracle is the order-independent value
 * that any fp32 summation order must approximate.  w_grad uses the layout of w.
 */
void mam_oracle_backward(const float *x, int64_t ldx, const float *w, int64_t ldw, int layout,
                         const float *g, const int32_t *argmax, const int32_t *argmin,
                         float *x_grad, float *w_grad, int64_t N, int64_t K, int64_t M)
{
    double *xa = (double *)calloc((size_t)(N * K), sizeof(double));
    double *wa = (double *)calloc((size_t)(K * M), sizeof(double));
    for (int64_t n = 0; n < N; ++n)
        for (int64_t m = 0; m < M; ++m) {
            const float gv = g[n * M + m];
            const int32_t sel[2] = { argmax[n * M + m], argmin[n * M + m] };
            for (int t = 0; t < 2; ++t) {
                const int64_t k = sel[t];
                volatile float tx = w_at(w, ldw, layout, k, m) * gv;
                volatile float tw = x[n * ldx + k] * gv;
                xa[n * K + k] += (double)tx;
                wa[(layout == MAM_W_MK) ? m * K + k : k * M + m] += (double)tw;
            }
        }
    for (int64_t i = 0; i < N * K; ++i) x_grad[i] = (float)xa[i];
    for (int64_t i = 0; i < K * M; ++i) w_grad[i] = (float)wa[i];
    free(xa); free(wa);
}

/*
 * counts are (M, K) int32, added to in place.
 * mode 0 "reference": literal behaviour of update_selection_count -- an advanced-index
 *   "+= 1" does not accumulate duplicates, and both statements write max_count:
 *   max_count[m,k] += [some n has argmax[n,m]==k] + [some n has argmin[n,m]==k];
 *   min_count untouched.
 * mode 1 "hits": max_count[m,k] += #{n: argmax[n,m]==k}; min_count likewise with argmin.
 */
void mam_oracle_selection_count(const int32_t *argmax, const int32_t *argmin,
                                int32_t *max_count, int32_t *min_count,
                                int64_t N, int64_t M, int64_t K, int mode)
{
    if (mode == 1) {
        for (int64_t n = 0; n < N; ++n)
            for (int64_t m = 0; m < M; ++m) {
                max_count[m * K + argmax[n * M + m]] += 1;
                min_count[m * K + argmin[n * M + m]] += 1;
            }
        return;
    }
    unsigned char *seen = (unsigned char *)malloc((size_t)(M * K));
    for (int pass = 0; pass < 2; ++pass) {
        const int32_t *arg = pass == 0 ? argmax : argmin;
        memset(seen, 0, (size_t)(M * K));
        for (int64_t n = 0; n < N; ++n)
            for (int64_t m = 0; m < M; ++m) seen[m * K + arg[n * M + m]] = 1;
        for (int64_t i = 0; i < M * K; ++i) max_count[i] += seen[i];
    }
    free(seen);
}

/* Densify one CSR row of the pruned weight (M, K) into dst[K]. */
static void csr_row_to_dense(const int64_t *crow, const int64_t *col, const float *val,
                             int64_t m, int64_t K, float *dst)
{
    for (int64_t k = 0; k < K; ++k) dst[k] = 0.0f;
    for (int64_t e = crow[m]; e < crow[m + 1]; ++e) dst[col[e]] = val[e];
}

/* CSR forward == dense forward on the densified weight (implicit zeros take part). */
void mam_oracle_csr_forward(const float *x, int64_t ldx, const int64_t *crow, const int64_t *col,
                            const float *val, const float *bias, float *c, int32_t *argmax,
                            int32_t *argmin, int64_t N, int64_t K, int64_t M)
{
    float *dense = (float *)malloc((size_t)(M * K) * sizeof(float));
    for (int64_t m = 0; m < M; ++m) csr_row_to_dense(crow, col, val, m, K, dense + m * K);
    mam_oracle_forward(x, ldx, dense, K, MAM_W_MK, bias, c, argmax, argmin, N, K, M);
    free(dense);
}

/*
 * CSR backward: the dense scatter rule restricted to stored positions.
 * x_grad (N,K) dense; val_grad (nnz).  A selected index that is not stored in the
 * row (an implicit zero won) contributes g*0 to x_grad and has no weight gradient.
 */
void mam_oracle_csr_backward(const float *x, int64_t ldx, const int64_t *crow, const int64_t *col,
                             const float *val, const float *g, const int32_t *argmax,
                             const int32_t *argmin, float *x_grad, float *val_grad,
                             int64_t N, int64_t K, int64_t M)
{
    const int64_t nnz = crow[M];
    double *xa = (double *)calloc((size_t)(N * K), sizeof(double));
    double *va = (double *)calloc((size_t)(nnz > 0 ? nnz : 1), sizeof(double));
    for (int64_t n = 0; n < N; ++n)
        for (int64_t m = 0; m < M; ++m) {
            const float gv = g[n * M + m];
            const int32_t sel[2] = { argmax[n * M + m], argmin[n * M + m] };
            for (int t = 0; t < 2; ++t) {
                const int64_t k = sel[t];
                int64_t found = -1;
                for (int64_t e = crow[m]; e < crow[m + 1]; ++e)
                    if (col[e] == k) { found = e; break; }
                if (found < 0) continue;
                volatile float tx = val[found] * gv;
                volatile float tv = x[n * ldx + k] * gv;
                xa[n * K + k] += (double)tx;
                va[found] += (double)tv;
            }
        }
    for (int64_t i = 0; i < N * K; ++i) x_grad[i] = (float)xa[i];
    for (int64_t i = 0; i < nnz; ++i) val_grad[i] = (float)va[i];
    free(xa); free(va);
}

/*
 * SpMM in COO form (a CSR caller expands crow): c (R,C) = sum over entries e of
 * val[e] * b[col[e], :] added to row row[e]; entries in any order, duplicates add up.
 * c and, when abs_sum != NULL, the sum of |val*b| per cell are fp64 sums rounded to fp32.
 */
void mam_oracle_coo_spmm(const int64_t *row, const int64_t *col, const float *val, int64_t nnz,
                         const float *b, int64_t ldb, float *c, float *abs_sum, int64_t R, int64_t C)
{
    double *acc = (double *)calloc((size_t)(R * C > 0 ? R * C : 1), sizeof(double));
    double *aab = (double *)calloc((size_t)(R * C > 0 ? R * C : 1), sizeof(double));
    for (int64_t e = 0; e < nnz; ++e) {
        const double v = (double)val[e];
        const float *br = b + col[e] * ldb;
        double *cr = acc + row[e] * C, *ar = aab + row[e] * C;
        for (int64_t j = 0; j < C; ++j) {
            const double t = v * (double)br[j];
            cr[j] += t;
            ar[j] += t < 0 ? -t : t;
        }
    }
    for (int64_t i = 0; i < R * C; ++i) {
        c[i] = (float)acc[i];
        if (abs_sum) abs_sum[i] = (float)aab[i];
    }
    free(acc); free(aab);
}
