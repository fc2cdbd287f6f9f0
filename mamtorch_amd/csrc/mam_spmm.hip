// Sum-of-products SpMM for gfx950: c (R, C) = A (R, K) sparse @ b (K, C) dense row-major, fp32.
// Stands behind mamtorch_kernel_sparsev1::cusparsemm, which the reference implements with cuSPARSE
// (CSR: mamtorch/sparse/kernel/v1/csrc/cuda/cusparsemm_csr.cu:19-77, CUSPARSE_SPMM_CSR_ALG2;
//  COO: mamtorch/sparse/kernel/v1/csrc/cuda/cusparsemm_coo.cu, same call on a COO descriptor),
// int64 indices, alpha = 1, beta = 0, and a cudaMalloc per call that is never freed (:60).
// Here nothing is allocated.
//
// Lanes are output columns: a stored entry (r, k, v) adds v * b[k, :] to c[r, :], and b[k, c0..c0+255]
// is one coalesced 1 KiB load for a wave (4 columns per lane).
//   CSR: a wave owns one row for one tile of 256 columns; column indices and values are wave-uniform
//        scalar loads; the loads of the next 8 entries are in flight while 8 are consumed; the row of c
//        is written once, no atomics, no zero fill.
//   COO: entries may come in any order and may repeat, so c is cleared first; a wave takes 64
//        consecutive entries, keeps a run of equal row indices in registers and flushes it with
//        atomic adds when the row changes.  On row-sorted input (what Tensor.to_sparse() and
//        coalesce() produce) that is about one flush per row and wave.
// Products are fused multiply-adds in ascending entry order within a wave; sums that span waves
// (COO only) are combined in no fixed order.
#include "mam_common.h"

namespace mam {
namespace spmm {

constexpr int NT = 256;
constexpr int EG = 8;          // entries whose loads are issued together
constexpr int COO_CHUNK = 64;  // entries per wave and pass

typedef const __attribute__((address_space(4))) int64_t const_i64;
typedef const __attribute__((address_space(4))) float const_f32;

template <int TI> struct Vec;
template <> struct Vec<1> { typedef float type; };
template <> struct Vec<4> { typedef float4 type; };

__device__ __forceinline__ void axpy(float (&acc)[1], float v, const float &b) { acc[0] = __builtin_fmaf(v, b, acc[0]); }
__device__ __forceinline__ void axpy(float (&acc)[4], float v, const float4 &b)
{
    acc[0] = __builtin_fmaf(v, b.x, acc[0]);
    acc[1] = __builtin_fmaf(v, b.y, acc[1]);
    acc[2] = __builtin_fmaf(v, b.z, acc[2]);
    acc[3] = __builtin_fmaf(v, b.w, acc[3]);
}

// TI = 4: b rows and c rows are 16-byte aligned and C is a multiple of 4; TI = 1 otherwise.
template <int TI>
__global__ __launch_bounds__(NT) void csr_spmm_kernel(const int64_t *__restrict__ crow,
                                                      const int64_t *__restrict__ col,
                                                      const float *__restrict__ val,
                                                      const float *__restrict__ b, int64_t ldb,
                                                      float *__restrict__ c, int R, int C)
{
    typedef typename Vec<TI>::type vec;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = blockIdx.x * (NT / 64) + wave;
    if (r >= R) return;
    const int c0 = blockIdx.y * 64 * TI + lane * TI;
    const bool live = c0 < C;
    const int cl = live ? c0 : 0;  // lanes past the last column read column 0 and store nothing

    const_i64 *ccol = (const_i64 *)col;
    const_f32 *cval = (const_f32 *)val;
    const int64_t beg = ((const_i64 *)crow)[r], end = ((const_i64 *)crow)[r + 1];
    const int nnz = (int)(end - beg);
    const float *bl = b + cl;

    float acc[TI];
#pragma unroll
    for (int t = 0; t < TI; ++t) acc[t] = 0.0f;

    const int ng = nnz / EG;
    vec xa[EG], xb[EG];
    float wa[EG], wb[EG];
    auto issue = [&](int g, vec (&xv)[EG], float (&wv)[EG]) {
#pragma unroll
        for (int u = 0; u < EG; ++u) {
            xv[u] = *reinterpret_cast<const vec *>(bl + ccol[beg + g * EG + u] * ldb);
            wv[u] = cval[beg + g * EG + u];
        }
    };
    auto consume = [&](const vec (&xv)[EG], const float (&wv)[EG]) {
#pragma unroll
        for (int u = 0; u < EG; ++u) axpy(acc, wv[u], xv[u]);
    };
    if (ng > 0) issue(0, xa, wa);
    for (int g = 0; g < ng; g += 2) {
        if (g + 1 < ng) issue(g + 1, xb, wb);
        __builtin_amdgcn_sched_barrier(0);
        consume(xa, wa);
        __builtin_amdgcn_sched_barrier(0);
        if (g + 1 >= ng) break;
        if (g + 2 < ng) issue(g + 2, xa, wa);
        __builtin_amdgcn_sched_barrier(0);
        consume(xb, wb);
        __builtin_amdgcn_sched_barrier(0);
    }
    for (int i = ng * EG; i < nnz; ++i) {
        const vec xv = *reinterpret_cast<const vec *>(bl + ccol[beg + i] * ldb);
        axpy(acc, cval[beg + i], xv);
    }
    if (live) {
        float *dst = c + (int64_t)r * C + c0;
        if (TI == 4) {
            *reinterpret_cast<float4 *>(dst) = make_float4(acc[0], acc[TI > 1 ? 1 : 0], acc[TI > 2 ? 2 : 0], acc[TI > 3 ? 3 : 0]);
        } else {
            dst[0] = acc[0];
        }
    }
}

template <int TI>
__device__ __forceinline__ void flush_row(float *__restrict__ c, int64_t row, int C, int c0, bool live,
                                          float (&acc)[TI])
{
    if (live) {
        float *dst = c + row * C + c0;
#pragma unroll
        for (int t = 0; t < TI; ++t) {
            unsafeAtomicAdd(dst + t, acc[t]);
            acc[t] = 0.0f;
        }
    }
}

template <int TI>
__global__ __launch_bounds__(NT) void coo_spmm_kernel(const int64_t *__restrict__ row,
                                                      const int64_t *__restrict__ col,
                                                      const float *__restrict__ val, int64_t nnz,
                                                      const float *__restrict__ b, int64_t ldb,
                                                      float *__restrict__ c, int C)
{
    typedef typename Vec<TI>::type vec;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t e0 = ((int64_t)blockIdx.x * (NT / 64) + wave) * COO_CHUNK;
    if (e0 >= nnz) return;
    const int n = (int)((nnz - e0) < COO_CHUNK ? (nnz - e0) : COO_CHUNK);
    const int c0 = blockIdx.y * 64 * TI + lane * TI;
    const bool live = c0 < C;
    const float *bl = b + (live ? c0 : 0);

    const_i64 *crow = (const_i64 *)row;
    const_i64 *ccol = (const_i64 *)col;
    const_f32 *cval = (const_f32 *)val;
    float acc[TI];
#pragma unroll
    for (int t = 0; t < TI; ++t) acc[t] = 0.0f;
    int64_t cur = crow[e0];
    for (int i = 0; i < n; i += EG) {
        // loads of up to EG entries first; entries past the end repeat the last one with weight 0
        vec xv[EG];
        float wv[EG];
        int64_t rv[EG];
#pragma unroll
        for (int u = 0; u < EG; ++u) {
            const bool ok = i + u < n;
            const int64_t e = e0 + (ok ? i + u : n - 1);
            xv[u] = *reinterpret_cast<const vec *>(bl + ccol[e] * ldb);
            wv[u] = ok ? cval[e] : 0.0f;
            rv[u] = crow[e];
        }
#pragma unroll
        for (int u = 0; u < EG; ++u) {
            if (rv[u] != cur) {  // wave-uniform
                flush_row<TI>(c, cur, C, c0, live, acc);
                cur = rv[u];
            }
            axpy(acc, wv[u], xv[u]);
        }
    }
    flush_row<TI>(c, cur, C, c0, live, acc);
}

static int check_common(const float *b, int64_t ldb, float *c, int64_t R, int64_t K, int64_t C)
{
    if (R < 0 || K < 0 || C < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (R > INT32_MAX / 2 || K > INT32_MAX / 2 || C > INT32_MAX / 2)
        return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    if (R == 0 || C == 0) return MAM_OK;
    if (!c || (K > 0 && !b)) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (ldb < C) return fail(MAM_ERR_INVALID_ARGUMENT, "ldb smaller than the number of columns");
    return MAM_OK;
}

// Scatter of a sparse matrix into a cleared dense one (repeated coordinates add up).  CSR: a wave per row.
// These kernels WRITE at the coordinates they are given, so an entry whose column (or row) lies outside the
// matrix is skipped: nothing is ever written outside `dense`.
__global__ __launch_bounds__(NT) void csr_to_dense_kernel(const int64_t *__restrict__ crow, const int64_t *__restrict__ col,
                                                          const float *__restrict__ val, float *__restrict__ dense,
                                                          int64_t ld, int R, int K)
{
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * (NT / 64) + (threadIdx.x >> 6);
    if (r >= R) return;
    const int64_t beg = crow[r], end = crow[r + 1];
    float *row = dense + (int64_t)r * ld;
    for (int64_t e = beg + lane; e < end; e += 64) {
        const int64_t cc = col[e];
        if ((uint64_t)cc < (uint64_t)K)
            __hip_atomic_fetch_add(row + cc, val[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

__global__ __launch_bounds__(256) void coo_to_dense_kernel(const int64_t *__restrict__ row, const int64_t *__restrict__ col,
                                                           const float *__restrict__ val, int64_t nnz,
                                                           float *__restrict__ dense, int64_t ld, int R, int K)
{
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < nnz; e += stride) {
        const int64_t rr = row[e], cc = col[e];
        if ((uint64_t)rr < (uint64_t)R && (uint64_t)cc < (uint64_t)K)
            __hip_atomic_fetch_add(dense + rr * ld + cc, val[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

static int check_dense(const float *dense, int64_t ld, int64_t R, int64_t K)
{
    if (R < 0 || K < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (R > INT32_MAX / 2 || K > INT32_MAX / 2) return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    if (R == 0 || K == 0) return MAM_OK;
    if (!dense) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (ld < K) return fail(MAM_ERR_INVALID_ARGUMENT, "ld smaller than the number of columns");
    return MAM_OK;
}

// rows of `dense` may be strided: cleared row by row when they are
static int clear_dense(float *dense, int64_t ld, int64_t R, int64_t K, hipStream_t st)
{
    if (ld == K) return fill_zero(dense, R * K, st);
    for (int64_t r = 0; r < R; ++r) {
        const int rc = fill_zero(dense + r * ld, K, st);
        if (rc != MAM_OK) return rc;
    }
    return MAM_OK;
}

static bool wide(const float *b, int64_t ldb, const float *c, int64_t C)
{
    return C % 4 == 0 && ldb % 4 == 0 && (uintptr_t)b % 16 == 0 && (uintptr_t)c % 16 == 0;
}

}  // namespace spmm
}  // namespace mam

extern "C" int mam_csr_spmm(const int64_t *crow, const int64_t *col, const float *val, const float *b,
                            int64_t ldb, float *c, int64_t R, int64_t K, int64_t C, void *stream)
{
    using namespace mam;
    int rc = spmm::check_common(b, ldb, c, R, K, C);
    if (rc != MAM_OK || R == 0 || C == 0) return rc;
    if (!crow) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const unsigned gx = (unsigned)ceil_div(R, spmm::NT / 64);
    if (spmm::wide(b, ldb, c, C)) {
        const int64_t gy = ceil_div(C, 256);
        if (gy > 65535) return fail(MAM_ERR_UNSUPPORTED, "too many columns for the SpMM grid");
        hipLaunchKernelGGL((spmm::csr_spmm_kernel<4>), dim3(gx, (unsigned)gy), dim3(spmm::NT), 0, st, crow, col,
                           val, b, ldb, c, (int)R, (int)C);
    } else {
        const int64_t gy = ceil_div(C, 64);
        if (gy > 65535) return fail(MAM_ERR_UNSUPPORTED, "too many columns for the SpMM grid");
        hipLaunchKernelGGL((spmm::csr_spmm_kernel<1>), dim3(gx, (unsigned)gy), dim3(spmm::NT), 0, st, crow, col,
                           val, b, ldb, c, (int)R, (int)C);
    }
    return check_launch("csr_spmm_kernel");
}

extern "C" int mam_coo_spmm(const int64_t *row, const int64_t *col, const float *val, int64_t nnz,
                            const float *b, int64_t ldb, float *c, int64_t R, int64_t K, int64_t C,
                            void *stream)
{
    using namespace mam;
    if (nnz < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    int rc = spmm::check_common(b, ldb, c, R, K, C);
    if (rc != MAM_OK || R == 0 || C == 0) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    rc = fill_zero(c, R * C, st);
    if (rc != MAM_OK || nnz == 0) return rc;
    if (!row || !col || !val) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    const int64_t gx = ceil_div(nnz, (int64_t)spmm::COO_CHUNK * (spmm::NT / 64));
    if (gx > INT32_MAX) return fail(MAM_ERR_UNSUPPORTED, "too many entries for the SpMM grid");
    if (spmm::wide(b, ldb, c, C)) {
        const int64_t gy = ceil_div(C, 256);
        if (gy > 65535) return fail(MAM_ERR_UNSUPPORTED, "too many columns for the SpMM grid");
        hipLaunchKernelGGL((spmm::coo_spmm_kernel<4>), dim3((unsigned)gx, (unsigned)gy), dim3(spmm::NT), 0, st,
                           row, col, val, nnz, b, ldb, c, (int)C);
    } else {
        const int64_t gy = ceil_div(C, 64);
        if (gy > 65535) return fail(MAM_ERR_UNSUPPORTED, "too many columns for the SpMM grid");
        hipLaunchKernelGGL((spmm::coo_spmm_kernel<1>), dim3((unsigned)gx, (unsigned)gy), dim3(spmm::NT), 0, st,
                           row, col, val, nnz, b, ldb, c, (int)C);
    }
    return check_launch("coo_spmm_kernel");
}

extern "C" int mam_csr_to_dense(const int64_t *crow, const int64_t *col, const float *val, float *dense, int64_t ld,
                                int64_t R, int64_t K, void *stream)
{
    using namespace mam;
    int rc = spmm::check_dense(dense, ld, R, K);
    if (rc != MAM_OK || R == 0 || K == 0) return rc;
    if (!crow) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    rc = spmm::clear_dense(dense, ld, R, K, st);
    if (rc != MAM_OK) return rc;
    hipLaunchKernelGGL(spmm::csr_to_dense_kernel, dim3((unsigned)ceil_div(R, spmm::NT / 64)), dim3(spmm::NT), 0, st, crow,
                       col, val, dense, ld, (int)R, (int)K);
    return check_launch("csr_to_dense_kernel");
}

extern "C" int mam_coo_to_dense(const int64_t *row, const int64_t *col, const float *val, int64_t nnz, float *dense,
                                int64_t ld, int64_t R, int64_t K, void *stream)
{
    using namespace mam;
    if (nnz < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    int rc = spmm::check_dense(dense, ld, R, K);
    if (rc != MAM_OK || R == 0 || K == 0) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    rc = spmm::clear_dense(dense, ld, R, K, st);
    if (rc != MAM_OK || nnz == 0) return rc;
    if (!row || !col || !val) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    int64_t blocks = ceil_div(nnz, 256);
    if (blocks > 64 * kNumCU) blocks = 64 * kNumCU;
    hipLaunchKernelGGL(spmm::coo_to_dense_kernel, dim3((unsigned)blocks), dim3(256), 0, st, row, col, val, nnz, dense, ld,
                       (int)R, (int)K);
    return check_launch("coo_to_dense_kernel");
}
