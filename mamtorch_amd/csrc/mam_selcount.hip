// Selection-count accumulation for pruning on gfx950: adds one batch's argmax / argmin picks
// into (M, K) int32 counters.  Replaces FullyConnected.update_selection_count
// (mamtorch/nn/v4/fullyconnected.py:114-129), which runs two advanced-index "+= 1" statements.
//
// A workgroup owns R = 4 consecutive neurons x kc columns of the counters.  Picks are collected
// in LDS words that hold two 16-bit fields (low: argmax, high: argmin), then the slab is streamed
// back with 16-byte read-modify-writes that skip chunks nothing was picked in.  At training batch
// sizes nearly every cache line of the counters holds a pick, so this is a coalesced pass over
// the slab; at small N*M it degenerates to a sparse update.  No global atomics.
//
// MAM_COUNT_HITS: the fields are counters (LDS atomic add; the batch is walked in chunks of 32768
// rows so that neither field overflows).
// MAM_COUNT_REFERENCE reproduces the module literally: an advanced-index "+= 1" does not
// accumulate duplicate indices, and both statements write max_selection_count, so per call a cell
// gains 1 if any batch row picked it as argmax plus 1 if any row picked it as argmin.  The fields
// are flags (LDS atomic or) and max_count receives flag(max) + flag(min); min_count is untouched.
// MAM_COUNT_FLAGS: the same flags, max and min apart (max_count += flag(max), min_count += flag(min)):
// the literal rule of the retired convolution modules (mamtorch/nn/backup/mamconv1d.txt:84-103), whose two
// advanced-index "+= 1" statements write the two counters.
#include "mam_common.h"
#include "mam_count_stream.h"

namespace mam {
namespace selcount {


#ifndef MAM_SELCOUNT_NT
#define MAM_SELCOUNT_NT 512
#endif
constexpr int NT_H = MAM_SELCOUNT_NT;
#ifndef MAM_SELCOUNT_FU
#define MAM_SELCOUNT_FU 2
#endif
constexpr int FU = MAM_SELCOUNT_FU;   // 16-byte chunks a thread has in flight while the slab is streamed back

template <int MODE>
__device__ __forceinline__ void mark(uint32_t *word, uint32_t field)
{
    if (MODE == MAM_COUNT_HITS) atomicAdd(word, field); else atomicOr(word, field);
}

constexpr int ROWS_PER_PASS = 32768;

template <int MODE>
__global__ __launch_bounds__(NT_H) void count_kernel(const int32_t *__restrict__ argmax,
                                                    const int32_t *__restrict__ argmin,
                                                    int32_t *__restrict__ max_count,
                                                    int32_t *__restrict__ min_count, int N, int M,
                                                    int K, int log2r, int kc, int vec, int vec_in)
{
    extern __shared__ uint32_t cnt[];  // [R][kc]
    const int tid = threadIdx.x;
    const int R = 1 << log2r;
    const int m0 = xcd_remap(blockIdx.x, gridDim.x) * R;
    const int k0 = blockIdx.y * kc;
    const int rn = (M - m0) < R ? (M - m0) : R;
    const int kn = (K - k0) < kc ? (K - k0) : kc;
    const int rows_per_pass = MODE == MAM_COUNT_HITS ? ROWS_PER_PASS : N;   // flags cannot overflow
    for (int n0 = 0; n0 < N; n0 += rows_per_pass) {
        const int nn = (N - n0) < rows_per_pass ? (N - n0) : rows_per_pass;
        for (int i = tid; i < R * kc; i += NT_H) cnt[i] = 0u;
        __syncthreads();
        if (vec_in && rn == R && R >= 4) {
            const int qpr = R >> 2;
            const int items = nn * qpr;
            for (int it = tid; it < items; it += NT_H) {
                const int n = n0 + it / qpr, r0 = (it % qpr) * 4;
                const int64_t o = (int64_t)n * M + m0 + r0;
                const int4 i1 = *reinterpret_cast<const int4 *>(argmax + o);
                const int4 i2 = *reinterpret_cast<const int4 *>(argmin + o);
                const int a1[4] = {i1.x - k0, i1.y - k0, i1.z - k0, i1.w - k0};
                const int a2[4] = {i2.x - k0, i2.y - k0, i2.z - k0, i2.w - k0};
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if ((unsigned)a1[u] < (unsigned)kn) mark<MODE>(&cnt[(r0 + u) * kc + a1[u]], 1u);
                    if ((unsigned)a2[u] < (unsigned)kn) mark<MODE>(&cnt[(r0 + u) * kc + a2[u]], 0x10000u);
                }
            }
        } else {
            const int pairs = nn << log2r;
            for (int pi = tid; pi < pairs; pi += NT_H) {
                const int n = n0 + (pi >> log2r), r = pi & (R - 1);
                if (r >= rn) continue;
                const int64_t o = (int64_t)n * M + m0 + r;
                const int a1 = argmax[o] - k0, a2 = argmin[o] - k0;
                if ((unsigned)a1 < (unsigned)kn) mark<MODE>(&cnt[r * kc + a1], 1u);
                if ((unsigned)a2 < (unsigned)kn) mark<MODE>(&cnt[r * kc + a2], 0x10000u);
            }
        }
        __syncthreads();
        // Stream the slab back: 4 cells per lane, whole 16-byte chunks skipped when nothing in
        // them was hit.  At training batch sizes nearly every cache line holds a hit, so this is
        // a coalesced read-modify-write of the slab; at small N*M it degenerates to a sparse one.
        if (vec) {
            stream_counts<MODE, NT_H, FU>(cnt, max_count, min_count, tid, m0, k0, rn, kn, kc, K);
        } else {
            for (int e = tid; e < rn * kn; e += NT_H) {
                const int r = e / kn, kk = e - r * kn;
                uint32_t v = cnt[r * kc + kk];
                if (MODE == MAM_COUNT_REFERENCE) v = (v & 1u) + (v >> 16);
                if (v) {
                    const int64_t cell = (int64_t)(m0 + r) * K + k0 + kk;
                    if (v & 0xffffu) max_count[cell] += (int)(v & 0xffffu);
                    if (v >> 16) min_count[cell] += (int)(v >> 16);
                }
            }
        }
        __syncthreads();
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
    if (mode != MAM_COUNT_REFERENCE && mode != MAM_COUNT_HITS && mode != MAM_COUNT_FLAGS)
        return fail(MAM_ERR_INVALID_ARGUMENT, "unknown selection-count mode %d", mode);
    if (N == 0 || M == 0 || K == 0) return MAM_OK;
    if (!argmax || !argmin || !max_count || (mode != MAM_COUNT_REFERENCE && !min_count))
        return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (N > INT32_MAX / 2 || K > INT32_MAX / 2 || M > INT32_MAX / 2)
        return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    hipStream_t st = static_cast<hipStream_t>(stream);
    // 4 whole-K rows of packed fields in 64 KiB: two workgroups per CU
    const int budget = 64 * 1024 / 4;
    const int log2r = 2;
    const int R = 1 << log2r;
    int kc = budget / R;
    if (K < kc) kc = (int)((K + 3) / 4 * 4);
    const int64_t ktiles = ceil_div(K, kc);
    if (ktiles > 65535) return fail(MAM_ERR_UNSUPPORTED, "K too large for the selection-count grid");
    const int vec = (K % 4 == 0) && ((uintptr_t)max_count % 16 == 0) &&
                    (mode == MAM_COUNT_REFERENCE || (uintptr_t)min_count % 16 == 0);
    const int vec_in = (M % 4 == 0) && ((uintptr_t)argmax % 16 == 0) && ((uintptr_t)argmin % 16 == 0);
    const dim3 grid((unsigned)ceil_div(M, R), (unsigned)ktiles);
    if (mode == MAM_COUNT_FLAGS)
        hipLaunchKernelGGL(selcount::count_kernel<MAM_COUNT_FLAGS>, grid, dim3(selcount::NT_H),
                           (size_t)R * kc * 4, st, argmax, argmin, max_count, min_count, (int)N, (int)M,
                           (int)K, log2r, kc, vec, vec_in);
    else if (mode == MAM_COUNT_HITS)
        hipLaunchKernelGGL(selcount::count_kernel<MAM_COUNT_HITS>, grid, dim3(selcount::NT_H),
                           (size_t)R * kc * 4, st, argmax, argmin, max_count, min_count, (int)N, (int)M,
                           (int)K, log2r, kc, vec, vec_in);
    else
        hipLaunchKernelGGL(selcount::count_kernel<MAM_COUNT_REFERENCE>, grid, dim3(selcount::NT_H),
                           (size_t)R * kc * 4, st, argmax, argmin, max_count, min_count, (int)N, (int)M,
                           (int)K, log2r, kc, vec, vec_in);
    return check_launch("selcount::count_kernel");
}
