// Pruning of a dense weight (M, K) and its compaction to CSR, on gfx950.
//
// The reference prunes by writing zeros into dense weights: an entry goes when its score is not
// above a threshold, `w[score.abs() <= threshold] = 0`, with score = w (magnitude pruning,
// examples/vitb16_imagenet1k/pruning_utils.py:103-111, 152-160) or score = w * w.grad (gradient
// pruning, :190-203, 252-263); the threshold is a quantile of |score|.  The selection counts of
// the MAM layer (mamtorch/nn/v4/fullyconnected.py:107-131) are the third score: a weight that was
// never (or rarely) selected as max or min can go.  What the reference then multiplies is still the
// dense matrix; here the survivors are compacted to CSR (int64 crow / col, fp32 val, the operand
// convention of mamtorch/sparse/kernel/v1/csrc/cuda/cusparsemm_csr.cu:37-41) for the sparse kernels.
//
// All three passes stream the matrix once with one wave per row and are bound by HBM:
//   count : kept entries per row (ballot + popcount)                      reads 4*M*K (+ the score operand)
//   scan  : exclusive prefix sum of the M row counts, one workgroup       M words
//   fill  : ascending columns and values of the kept entries, positions
//           from the lane's rank among the kept lanes of its 64 columns   reads 4*M*K, writes 12*nnz
// and `apply` is the reference's in-place form (pruned entries become 0.0f).
#include "mam_common.h"

namespace mam {
namespace prune {

constexpr int NT = 256;

// keep <=> !(|score| <= threshold): a NaN score is kept, as by the reference's masked assignment
template <int MODE>
__device__ __forceinline__ bool keep_entry(float w, const void *aux, const void *aux2, int64_t idx, float threshold)
{
    float score;
    if (MODE == MAM_PRUNE_MAGNITUDE) {
        score = __builtin_fabsf(w);
    } else if (MODE == MAM_PRUNE_WEIGHT_TIMES) {
        score = __builtin_fabsf(w * static_cast<const float *>(aux)[idx]);
    } else {
        int cnt = static_cast<const int32_t *>(aux)[idx];
        if (aux2) cnt += static_cast<const int32_t *>(aux2)[idx];
        score = (float)cnt;
    }
    return !(score <= threshold);
}

// Four consecutive columns of one lane: which of them survive (bit j = column k + j).
template <int MODE>
__device__ __forceinline__ int keep_quad(const float *__restrict__ w, int64_t ldw, const void *aux, const void *aux2,
                                         int64_t ld_aux, float threshold, int m, int k, int K, float4 &v)
{
    v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (k >= K) return 0;      // K is a multiple of 4 on this path
    v = *reinterpret_cast<const float4 *>(w + (int64_t)m * ldw + k);
    const int64_t a = (int64_t)m * ld_aux + k;
    int bits = 0;
    if (MODE == MAM_PRUNE_MAGNITUDE) {
        bits |= !(__builtin_fabsf(v.x) <= threshold) ? 1 : 0;
        bits |= !(__builtin_fabsf(v.y) <= threshold) ? 2 : 0;
        bits |= !(__builtin_fabsf(v.z) <= threshold) ? 4 : 0;
        bits |= !(__builtin_fabsf(v.w) <= threshold) ? 8 : 0;
    } else if (MODE == MAM_PRUNE_WEIGHT_TIMES) {
        const float4 f = *reinterpret_cast<const float4 *>(static_cast<const float *>(aux) + a);
        bits |= !(__builtin_fabsf(v.x * f.x) <= threshold) ? 1 : 0;
        bits |= !(__builtin_fabsf(v.y * f.y) <= threshold) ? 2 : 0;
        bits |= !(__builtin_fabsf(v.z * f.z) <= threshold) ? 4 : 0;
        bits |= !(__builtin_fabsf(v.w * f.w) <= threshold) ? 8 : 0;
    } else {
        int4 cnt = *reinterpret_cast<const int4 *>(static_cast<const int32_t *>(aux) + a);
        if (aux2) {
            const int4 c2 = *reinterpret_cast<const int4 *>(static_cast<const int32_t *>(aux2) + a);
            cnt.x += c2.x; cnt.y += c2.y; cnt.z += c2.z; cnt.w += c2.w;
        }
        bits |= !((float)cnt.x <= threshold) ? 1 : 0;
        bits |= !((float)cnt.y <= threshold) ? 2 : 0;
        bits |= !((float)cnt.z <= threshold) ? 4 : 0;
        bits |= !((float)cnt.w <= threshold) ? 8 : 0;
    }
    return bits;
}

// `vec`: rows of w (and of the score operands) are 16-byte aligned and K is a multiple of 4; a lane then
// takes 4 consecutive columns per trip (256 per wave), four trips in flight.
template <int MODE>
__global__ __launch_bounds__(NT) void count_kernel(const float *__restrict__ w, int64_t ldw,
                                                   const void *__restrict__ aux, const void *__restrict__ aux2,
                                                   int64_t ld_aux, float threshold,
                                                   int64_t *__restrict__ crow, int M, int K, int vec)
{
    const int lane = threadIdx.x & 63;
    const int m = blockIdx.x * (NT / 64) + (threadIdx.x >> 6);
    if (m >= M) return;
    int kept = 0;
    if (vec) {
        int mine = 0;
        for (int k0 = 0; k0 < K; k0 += 4 * 256) {
            float4 v[4];
            int bits[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                bits[u] = keep_quad<MODE>(w, ldw, aux, aux2, ld_aux, threshold, m, k0 + u * 256 + 4 * lane, K, v[u]);
#pragma unroll
            for (int u = 0; u < 4; ++u) mine += __builtin_popcount(bits[u]);
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mine += __shfl_down(mine, off);
        kept = mine;
    } else {
        for (int k0 = 0; k0 < K; k0 += 64) {
            const int k = k0 + lane;
            const bool keep = k < K && keep_entry<MODE>(w[(int64_t)m * ldw + k], aux, aux2, (int64_t)m * ld_aux + k, threshold);
            kept += __builtin_popcountll(__ballot(keep));
        }
    }
    if (lane == 0) crow[m + 1] = kept;
    if (m == 0 && lane == 0) crow[0] = 0;
}

// crow[1..M] holds row counts on entry and inclusive prefix sums on exit.  One workgroup: a thread
// takes a run of consecutive rows, waves scan their threads' sums with shuffles, one more step
// chains the 16 waves.
__global__ __launch_bounds__(1024) void scan_kernel(int64_t *__restrict__ crow, int M)
{
    __shared__ int64_t wave_total[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int per = (M + 1023) / 1024;
    const int first = tid * per;
    int64_t sum = 0;
    for (int j = 0; j < per; ++j) {
        const int i = first + j;
        if (i < M) sum += crow[i + 1];
    }
    int64_t incl = sum;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int64_t t = __shfl_up(incl, off);
        if (lane >= off) incl += t;
    }
    if (lane == 63) wave_total[wave] = incl;
    __syncthreads();
    int64_t run = incl - sum;
    for (int w2 = 0; w2 < wave; ++w2) run += wave_total[w2];
    for (int j = 0; j < per; ++j) {
        const int i = first + j;
        if (i < M) {
            run += crow[i + 1];
            crow[i + 1] = run;
        }
    }
}

template <int MODE>
__global__ __launch_bounds__(NT) void fill_kernel(const float *__restrict__ w, int64_t ldw,
                                                  const void *__restrict__ aux, const void *__restrict__ aux2,
                                                  int64_t ld_aux, float threshold,
                                                  const int64_t *__restrict__ crow, int64_t *__restrict__ col,
                                                  float *__restrict__ val, int M, int K, int vec)
{
    const int lane = threadIdx.x & 63;
    const int m = blockIdx.x * (NT / 64) + (threadIdx.x >> 6);
    if (m >= M) return;
    int64_t pos = crow[m];
    if (vec) {
        const uint64_t below = (1ull << lane) - 1ull;
        for (int k0 = 0; k0 < K; k0 += 2 * 256) {
            float4 v[2];
            int bits[2];
#pragma unroll
            for (int u = 0; u < 2; ++u)
                bits[u] = keep_quad<MODE>(w, ldw, aux, aux2, ld_aux, threshold, m, k0 + u * 256 + 4 * lane, K, v[u]);
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                // survivors of lower lanes come first, then this lane's own lower columns
                int before = 0, total = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint64_t mask = __ballot((bits[u] >> j) & 1);
                    before += __builtin_popcountll(mask & below);
                    total += __builtin_popcountll(mask);
                }
                const float vals[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
                int r = before;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if ((bits[u] >> j) & 1) {
                        col[pos + r] = k0 + u * 256 + 4 * lane + j;
                        val[pos + r] = vals[j];
                        ++r;
                    }
                pos += total;
            }
        }
        return;
    }
    for (int k0 = 0; k0 < K; k0 += 64) {
        const int k = k0 + lane;
        const float v = k < K ? w[(int64_t)m * ldw + k] : 0.0f;
        const bool keep = k < K && keep_entry<MODE>(v, aux, aux2, (int64_t)m * ld_aux + k, threshold);
        const uint64_t mask = __ballot(keep);
        if (keep) {
            const int rank = __builtin_popcountll(mask & ((1ull << lane) - 1ull));
            col[pos + rank] = k;
            val[pos + rank] = v;
        }
        pos += __builtin_popcountll(mask);
    }
}

template <int MODE>
__global__ __launch_bounds__(NT) void apply_kernel(float *__restrict__ w, int64_t ldw, const void *__restrict__ aux,
                                                   const void *__restrict__ aux2, int64_t ld_aux, float threshold,
                                                   int M, int K)
{
    const int64_t total = (int64_t)M * K;
    for (int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x; i < total; i += (int64_t)gridDim.x * NT) {
        const int64_t m = i / K, k = i - m * K;
        float *p = w + m * ldw + k;
        if (!keep_entry<MODE>(*p, aux, aux2, m * ld_aux + k, threshold)) *p = 0.0f;
    }
}

static int aligned_rows(const float *w, int64_t ldw, int mode, const void *aux, const void *aux2, int64_t ld_aux,
                        int64_t K)
{
    bool ok = K % 4 == 0 && ldw % 4 == 0 && (uintptr_t)w % 16 == 0;
    if (mode != MAM_PRUNE_MAGNITUDE)
        ok = ok && ld_aux % 4 == 0 && (uintptr_t)aux % 16 == 0 && (uintptr_t)aux2 % 16 == 0;
    return ok;
}

static int check(const float *w, int64_t ldw, int mode, const void *aux, int64_t ld_aux, int64_t M, int64_t K)
{
    if (M < 0 || K < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (mode != MAM_PRUNE_MAGNITUDE && mode != MAM_PRUNE_WEIGHT_TIMES && mode != MAM_PRUNE_COUNT)
        return fail(MAM_ERR_INVALID_ARGUMENT, "unknown pruning mode");
    if (M > INT32_MAX / 2 || K > INT32_MAX / 2) return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    if (M == 0 || K == 0) return MAM_OK;
    if (!w || (mode != MAM_PRUNE_MAGNITUDE && !aux)) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (ldw < K || (mode != MAM_PRUNE_MAGNITUDE && ld_aux < K))
        return fail(MAM_ERR_INVALID_ARGUMENT, "leading dimension smaller than the row length");
    return MAM_OK;
}

}  // namespace prune
}  // namespace mam

#define MAM_PRUNE_DISPATCH(KERNEL, GRID, BLOCK, ...)                                                  \
    do {                                                                                              \
        if (mode == MAM_PRUNE_MAGNITUDE)                                                              \
            hipLaunchKernelGGL((prune::KERNEL<MAM_PRUNE_MAGNITUDE>), GRID, BLOCK, 0, st, __VA_ARGS__);   \
        else if (mode == MAM_PRUNE_WEIGHT_TIMES)                                                      \
            hipLaunchKernelGGL((prune::KERNEL<MAM_PRUNE_WEIGHT_TIMES>), GRID, BLOCK, 0, st, __VA_ARGS__); \
        else                                                                                          \
            hipLaunchKernelGGL((prune::KERNEL<MAM_PRUNE_COUNT>), GRID, BLOCK, 0, st, __VA_ARGS__);       \
    } while (0)

extern "C" int mam_prune_row_offsets(const float *w, int64_t ldw, int mode, const void *aux, const void *aux2,
                                     int64_t ld_aux, float threshold, int64_t *crow, int64_t M, int64_t K,
                                     void *stream)
{
    using namespace mam;
    int rc = prune::check(w, ldw, mode, aux, ld_aux, M, K);
    if (rc != MAM_OK) return rc;
    if (!crow) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (M == 0 || K == 0) return fill_zero(crow, 2 * (M + 1), st);   // int64 offsets = 2 words each
    const dim3 grid((unsigned)ceil_div(M, prune::NT / 64)), block(prune::NT);
    MAM_PRUNE_DISPATCH(count_kernel, grid, block, w, ldw, aux, aux2, ld_aux, threshold, crow, (int)M, (int)K,
                       prune::aligned_rows(w, ldw, mode, aux, aux2, ld_aux, K));
    rc = check_launch("prune count_kernel");
    if (rc != MAM_OK) return rc;
    hipLaunchKernelGGL(prune::scan_kernel, dim3(1), dim3(1024), 0, st, crow, (int)M);
    return check_launch("prune scan_kernel");
}

extern "C" int mam_prune_fill_csr(const float *w, int64_t ldw, int mode, const void *aux, const void *aux2,
                                  int64_t ld_aux, float threshold, const int64_t *crow, int64_t *col, float *val,
                                  int64_t M, int64_t K, void *stream)
{
    using namespace mam;
    int rc = prune::check(w, ldw, mode, aux, ld_aux, M, K);
    if (rc != MAM_OK || M == 0 || K == 0) return rc;
    if (!crow) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)ceil_div(M, prune::NT / 64)), block(prune::NT);
    MAM_PRUNE_DISPATCH(fill_kernel, grid, block, w, ldw, aux, aux2, ld_aux, threshold, crow, col, val, (int)M, (int)K,
                       prune::aligned_rows(w, ldw, mode, aux, aux2, ld_aux, K));
    return check_launch("prune fill_kernel");
}

extern "C" int mam_prune_apply(float *w, int64_t ldw, int mode, const void *aux, const void *aux2, int64_t ld_aux,
                               float threshold, int64_t M, int64_t K, void *stream)
{
    using namespace mam;
    int rc = prune::check(w, ldw, mode, aux, ld_aux, M, K);
    if (rc != MAM_OK || M == 0 || K == 0) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int64_t blocks = ceil_div(M * K, prune::NT);
    if (blocks > 16 * kNumCU) blocks = 16 * kNumCU;
    const dim3 grid((unsigned)blocks), block(prune::NT);
    MAM_PRUNE_DISPATCH(apply_kernel, grid, block, w, ldw, aux, aux2, ld_aux, threshold, (int)M, (int)K);
    return check_launch("prune apply_kernel");
}
