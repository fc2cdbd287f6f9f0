// Selection-count accumulation for pruning on gfx950: adds one batch's argmax / argmin picks
// into (M, K) int32 counters.  Replaces FullyConnected.update_selection_count
// (mamtorch/nn/v4/fullyconnected.py:114-129), which runs two advanced-index "+= 1" statements.
//
// MAM_COUNT_REFERENCE reproduces that code literally: an advanced-index "+= 1" does not
// accumulate duplicate indices, and both statements write max_selection_count, so per call a
// cell gains 1 if any batch row picked it as argmax plus 1 if any row picked it as argmin.  A
// workgroup owns R consecutive neurons, marks picks in two LDS bitmaps (ds_or), then walks the
// set bits and applies plain read-modify-writes to its own rows: the counters are touched only
// where something was picked, and no global atomics are needed.
//
// MAM_COUNT_HITS counts every pick (global int atomics; fire-and-forget).
#include "mam_common.h"

namespace mam {
namespace selcount {

constexpr int NT = 256;

__global__ __launch_bounds__(NT) void hits_kernel(const int32_t *__restrict__ argmax,
                                                  const int32_t *__restrict__ argmin,
                                                  int32_t *__restrict__ max_count,
                                                  int32_t *__restrict__ min_count, int64_t NM, int M,
                                                  int K)
{
    const int64_t o = (int64_t)blockIdx.x * NT + threadIdx.x;
    if (o >= NM) return;
    const int m = (int)(o % M);
    const int a1 = argmax[o], a2 = argmin[o];
    if ((unsigned)a1 < (unsigned)K) atomicAdd(&max_count[(int64_t)m * K + a1], 1);
    if ((unsigned)a2 < (unsigned)K) atomicAdd(&min_count[(int64_t)m * K + a2], 1);
}

__global__ __launch_bounds__(NT) void reference_kernel(const int32_t *__restrict__ argmax,
                                                       const int32_t *__restrict__ argmin,
                                                       int32_t *__restrict__ max_count, int N, int M,
                                                       int K, int log2r, int words)
{
    extern __shared__ uint32_t bits[];  // [2][R][words]
    const int tid = threadIdx.x;
    const int R = 1 << log2r;
    const int m0 = xcd_remap(blockIdx.x, gridDim.x) * R;
    const int rn = (M - m0) < R ? (M - m0) : R;
    const int plane = R * words;
    for (int i = tid; i < 2 * plane; i += NT) bits[i] = 0u;
    __syncthreads();
    const int64_t pairs = (int64_t)N << log2r;
    for (int64_t pi = tid; pi < pairs; pi += NT) {
        const int n = (int)(pi >> log2r), r = (int)(pi & (R - 1));
        if (r >= rn) continue;
        const int64_t o = (int64_t)n * M + m0 + r;
        const int a1 = argmax[o], a2 = argmin[o];
        if ((unsigned)a1 < (unsigned)K) atomicOr(&bits[r * words + (a1 >> 5)], 1u << (a1 & 31));
        if ((unsigned)a2 < (unsigned)K) atomicOr(&bits[plane + r * words + (a2 >> 5)], 1u << (a2 & 31));
    }
    __syncthreads();
    for (int e = tid; e < rn * words; e += NT) {
        const int r = e / words, wi = e - r * words;
        const uint32_t b1 = bits[r * words + wi], b2 = bits[plane + r * words + wi];
        uint32_t u = b1 | b2;
        int32_t *row = max_count + (int64_t)(m0 + r) * K + wi * 32;
        while (u) {
            const int b = __builtin_ctz(u);
            u &= u - 1;
            row[b] += (int)((b1 >> b) & 1u) + (int)((b2 >> b) & 1u);
        }
    }
}

}  // namespace selcount
}  // namespace mam

extern "C" int mam_selection_count(const int32_t *argmax, const int32_t *argmin, int32_t *max_count,
                                   int32_t *min_count, int64_t N, int64_t M, int64_t K, int mode,
                                   void *stream)
{
    using namespace mam;
    if (N < 0 || M < 0 || K < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (mode != MAM_COUNT_REFERENCE && mode != MAM_COUNT_HITS)
        return fail(MAM_ERR_INVALID_ARGUMENT, "unknown selection-count mode %d", mode);
    if (N == 0 || M == 0 || K == 0) return MAM_OK;
    if (!argmax || !argmin || !max_count || (mode == MAM_COUNT_HITS && !min_count))
        return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (N > INT32_MAX / 2 || K > INT32_MAX / 2 || M > INT32_MAX / 2)
        return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (mode == MAM_COUNT_HITS) {
        const int64_t nm = N * M;
        hipLaunchKernelGGL(selcount::hits_kernel, dim3((unsigned)ceil_div(nm, selcount::NT)),
                           dim3(selcount::NT), 0, st, argmax, argmin, max_count, min_count, nm, (int)M,
                           (int)K);
        return check_launch("selcount::hits_kernel");
    }
    const int words = (int)ceil_div(K, 32);
    // two bitmaps of R rows in at most 48 KiB of LDS
    int log2r = 5;
    while (log2r > 0 && (int64_t)2 * (1 << log2r) * words * 4 > 48 * 1024) --log2r;
    if ((int64_t)2 * (1 << log2r) * words * 4 > 48 * 1024)
        return fail(MAM_ERR_UNSUPPORTED, "K = %lld exceeds the bitmap capacity (196608)", (long long)K);
    const int R = 1 << log2r;
    hipLaunchKernelGGL(selcount::reference_kernel, dim3((unsigned)ceil_div(M, R)), dim3(selcount::NT),
                       (size_t)2 * R * words * 4, st, argmax, argmin, max_count, (int)N, (int)M, (int)K,
                       log2r, words);
    return check_launch("selcount::reference_kernel");
}
