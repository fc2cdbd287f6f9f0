// CSR-sparse MAM forward / backward over a pruned weight (M, K) on gfx950.
//
// The reference has no sparse MAM operator; its sparse module only wraps a sum-of-products SpMM
// whose operand convention is kept here: CSR with int64 crow / col and fp32 values
// (mamtorch/sparse/kernel/v1/csrc/cuda/cusparsemm_csr.cu:25-45).  The MAM result is defined as
// the dense MAM forward on the densified weight, because the reference prunes by writing literal
// zeros into dense weights (examples/vitb16_imagenet1k/pruning_utils.py:107,111): an absent
// entry is a zero weight whose product x*0 takes part in the max / min and in the first-index
// tie-break.
//
// Forward: a lane owns one CSR row (output neuron) and walks its entries in ascending column
// order; NB batch rows are register-blocked per lane and their x values are gathered from an LDS
// copy of the x tile, so HBM sees every (col, val) pair once per batch tile and x once per
// neuron tile.  While walking, the lane also finds the lowest column missing from its row; the
// implicit-zero candidate x[n, missing] * 0 is compared last under the dense rule (greater wins,
// equal -> lower index wins).
//
// Backward: one workgroup per batch row; selected columns are located in the CSR row by binary
// search, x_grad is accumulated in an LDS histogram and stored once, val_grad takes global
// atomic adds (at most N contenders per entry).
#include "mam_common.h"

namespace mam {
namespace csr {

constexpr int NT = 256;
constexpr int NB = 8;      // batch rows per lane
constexpr int NT_B = 512;  // backward workgroup

__global__ __launch_bounds__(NT) void csr_fwd_kernel(
    const float *__restrict__ x, int64_t ldx, const int64_t *__restrict__ crow,
    const int64_t *__restrict__ col, const float *__restrict__ val, const float *__restrict__ bias,
    float *__restrict__ c, int32_t *__restrict__ argmax, int32_t *__restrict__ argmin, int N, int K,
    int M, int kc)
{
    extern __shared__ float xs[];  // [NB][kc]
    const int tid = threadIdx.x;
    const int m = blockIdx.x * NT + tid;
    const int n0 = blockIdx.y * NB;
    const bool valid = m < M;
    int64_t e = valid ? crow[m] : 0;
    const int64_t e_end = valid ? crow[m + 1] : 0;
    const int64_t row_nnz = e_end - e;

    float vmax[NB], vmin[NB];
    int imax[NB], imin[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        vmax[b] = -__builtin_inff();
        vmin[b] = __builtin_inff();
        imax[b] = -1;
        imin[b] = -1;
    }
    int missing = 0;  // lowest column not stored in this row (valid once the walk is over)

    for (int k0 = 0; k0 < K; k0 += kc) {
        const int kn = (K - k0) < kc ? (K - k0) : kc;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int n = (n0 + b) < N ? (n0 + b) : (N - 1);
            const float *src = x + (int64_t)n * ldx + k0;
            for (int kk = tid; kk < kn; kk += NT) xs[b * kc + kk] = src[kk];
        }
        __syncthreads();
        while (e < e_end) {
            const int64_t cidx = col[e];
            if (cidx >= (int64_t)k0 + kn) break;
            const float v = val[e];
            const int ci = (int)cidx;
            if (ci == missing) ++missing;
            const int kk = ci - k0;
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const float p = xs[b * kc + kk] * v;
                if (p > vmax[b]) { vmax[b] = p; imax[b] = ci; }
                if (p < vmin[b]) { vmin[b] = p; imin[b] = ci; }
            }
            ++e;
        }
        __syncthreads();
    }
    if (!valid) return;

    const bool has_zero = row_nnz < (int64_t)K;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int n = n0 + b;
        if (n >= N) break;
        float hi = vmax[b], lo = vmin[b];
        int ih = imax[b], il = imin[b];
        if (has_zero) {
            const float z = x[(int64_t)n * ldx + missing] * 0.0f;
            if (ih < 0 || z > hi || (z == hi && missing < ih)) { hi = z; ih = missing; }
            if (il < 0 || z < lo || (z == lo && missing < il)) { lo = z; il = missing; }
        }
        float s = hi + lo;
        if (bias) s = s + bias[m];
        const int64_t o = (int64_t)n * M + m;
        c[o] = s;
        argmax[o] = ih;
        argmin[o] = il;
    }
}

__device__ __forceinline__ int64_t find_col(const int64_t *__restrict__ col, int64_t lo, int64_t hi,
                                            int64_t key)
{
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        const int64_t cv = col[mid];
        if (cv < key) lo = mid + 1; else hi = mid;
    }
    return lo;
}

__global__ __launch_bounds__(NT_B) void csr_bwd_kernel(
    const float *__restrict__ x, int64_t ldx, const int64_t *__restrict__ crow,
    const int64_t *__restrict__ col, const float *__restrict__ val, const float *__restrict__ grad,
    const int32_t *__restrict__ argmax, const int32_t *__restrict__ argmin,
    float *__restrict__ x_grad, float *__restrict__ val_grad, int K, int M, int kc)
{
    extern __shared__ float hist[];
    const int n = blockIdx.x;
    const int tid = threadIdx.x;
    const float *xr = x + (int64_t)n * ldx;
    for (int k0 = 0; k0 < K; k0 += kc) {
        const int kn = (K - k0) < kc ? (K - k0) : kc;
        for (int i = tid; i < kn; i += NT_B) hist[i] = 0.0f;
        __syncthreads();
        for (int m = tid; m < M; m += NT_B) {
            const int64_t o = (int64_t)n * M + m;
            const float g = grad[o];
            const int sel[2] = {argmax[o], argmin[o]};
            const int64_t lo = crow[m], hi = crow[m + 1];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int a = sel[t] - k0;
                if ((unsigned)a >= (unsigned)kn) continue;
                const int64_t e = find_col(col, lo, hi, sel[t]);
                if (e >= hi || col[e] != sel[t]) continue;  // an implicit zero was selected
                __hip_atomic_fetch_add(&hist[a], val[e] * g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                if (val_grad) unsafeAtomicAdd(&val_grad[e], xr[sel[t]] * g);
            }
        }
        __syncthreads();
        if (x_grad) {
            float *dst = x_grad + (int64_t)n * K + k0;
            for (int i = tid; i < kn; i += NT_B) dst[i] = hist[i];
        }
        __syncthreads();
    }
}

static int lds_budget_floats(const void *kernel)
{
    constexpr int kWant = 128 * 1024;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kWant) == hipSuccess)
        return kWant / 4;
    (void)hipGetLastError();
    return 64 * 1024 / 4;
}

}  // namespace csr
}  // namespace mam

extern "C" size_t mam_csr_fc_forward_workspace(int64_t, int64_t, int64_t) { return 0; }

extern "C" int mam_csr_fc_forward(const float *x, int64_t ldx, const int64_t *crow, const int64_t *col,
                                  const float *val, const float *bias, float *c, int32_t *argmax,
                                  int32_t *argmin, int64_t N, int64_t K, int64_t M, void *workspace,
                                  size_t workspace_bytes, void *stream)
{
    using namespace mam;
    (void)workspace; (void)workspace_bytes;
    if (N < 0 || K < 0 || M < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (N == 0 || M == 0) return MAM_OK;
    if (K == 0) return fail(MAM_ERR_INVALID_ARGUMENT, "K == 0: max/min over an empty set");
    if (!x || !crow || !c || !argmax || !argmin) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (ldx < K) return fail(MAM_ERR_INVALID_ARGUMENT, "ldx smaller than K");
    if (N > INT32_MAX / 2 || K > INT32_MAX / 2 || M > INT32_MAX / 2)
        return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    static const int budget = csr::lds_budget_floats((const void *)csr::csr_fwd_kernel);
    int kc = budget / csr::NB;
    if (K < kc) kc = (int)K;
    const int64_t gy = ceil_div(N, csr::NB);
    if (gy > 65535) return fail(MAM_ERR_UNSUPPORTED, "N too large for the CSR forward grid");
    hipLaunchKernelGGL(csr::csr_fwd_kernel, dim3((unsigned)ceil_div(M, csr::NT), (unsigned)gy),
                       dim3(csr::NT), (size_t)csr::NB * kc * sizeof(float),
                       static_cast<hipStream_t>(stream), x, ldx, crow, col, val, bias, c, argmax, argmin,
                       (int)N, (int)K, (int)M, kc);
    return check_launch("csr_fwd_kernel");
}

extern "C" int mam_csr_fc_backward(const float *x, int64_t ldx, const int64_t *crow, const int64_t *col,
                                   const float *val, const float *grad, const int32_t *argmax,
                                   const int32_t *argmin, float *x_grad, float *val_grad, int64_t N,
                                   int64_t K, int64_t M, int64_t nnz, void *stream)
{
    using namespace mam;
    if (N < 0 || K < 0 || M < 0 || nnz < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (N > INT32_MAX / 2 || K > INT32_MAX / 2 || M > INT32_MAX / 2)
        return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    hipStream_t st = static_cast<hipStream_t>(stream);
    int rc = MAM_OK;
    if (val_grad) rc = fill_zero(val_grad, nnz, st);
    if (rc != MAM_OK) return rc;
    if (N == 0 || K == 0) return MAM_OK;
    if (M == 0) return x_grad ? fill_zero(x_grad, N * K, st) : MAM_OK;
    if (!x || !crow || !grad || !argmax || !argmin) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (ldx < K) return fail(MAM_ERR_INVALID_ARGUMENT, "ldx smaller than K");
    static const int budget = csr::lds_budget_floats((const void *)csr::csr_bwd_kernel);
    const int kc = (int)(K < budget ? K : budget);
    hipLaunchKernelGGL(csr::csr_bwd_kernel, dim3((unsigned)N), dim3(csr::NT_B), (size_t)kc * sizeof(float),
                       st, x, ldx, crow, col, val, grad, argmax, argmin, x_grad, val_grad, (int)K, (int)M,
                       kc);
    return check_launch("csr_bwd_kernel");
}
