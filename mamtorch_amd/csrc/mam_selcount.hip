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
// MAM_COUNT_HITS counts every pick with the same ownership scheme and LDS counters.
#include "mam_common.h"

namespace mam {
namespace selcount {

constexpr int NT = 256;

// Hit counting: a workgroup owns R neurons x kc columns of both counters.  Picks are counted in
// LDS words holding two 16-bit counters (low half: argmax hits, high half: argmin hits; the batch
// is walked in chunks of 32768 rows so that neither half overflows), then only the cells that
// were hit are read-modify-written in HBM.
constexpr int NT_H = 512;
constexpr int ROWS_PER_PASS = 32768;

__global__ __launch_bounds__(NT_H) void hits_kernel(const int32_t *__restrict__ argmax,
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
    for (int n0 = 0; n0 < N; n0 += ROWS_PER_PASS) {
        const int nn = (N - n0) < ROWS_PER_PASS ? (N - n0) : ROWS_PER_PASS;
        for (int i = tid; i < R * kc; i += NT_H) cnt[i] = 0u;
        __syncthreads();
        if (vec_in && rn == R) {
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
                    if ((unsigned)a1[u] < (unsigned)kn) atomicAdd(&cnt[(r0 + u) * kc + a1[u]], 1u);
                    if ((unsigned)a2[u] < (unsigned)kn) atomicAdd(&cnt[(r0 + u) * kc + a2[u]], 0x10000u);
                }
            }
        } else {
            const int pairs = nn << log2r;
            for (int pi = tid; pi < pairs; pi += NT_H) {
                const int n = n0 + (pi >> log2r), r = pi & (R - 1);
                if (r >= rn) continue;
                const int64_t o = (int64_t)n * M + m0 + r;
                const int a1 = argmax[o] - k0, a2 = argmin[o] - k0;
                if ((unsigned)a1 < (unsigned)kn) atomicAdd(&cnt[r * kc + a1], 1u);
                if ((unsigned)a2 < (unsigned)kn) atomicAdd(&cnt[r * kc + a2], 0x10000u);
            }
        }
        __syncthreads();
        // Stream the slab back: 4 cells per lane, whole 16-byte chunks skipped when nothing in
        // them was hit.  At training batch sizes nearly every cache line holds a hit, so this is
        // a coalesced read-modify-write of the slab; at small N*M it degenerates to a sparse one.
        if (vec) {
            const int q = kn >> 2;
            const int total = rn * q;
            for (int eb = tid; eb < total; eb += 4 * NT_H) {
                uint4 v[4];
                int4 amx[4], amn[4];
                int64_t cell[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int e = eb + u * NT_H;
                    v[u] = make_uint4(0u, 0u, 0u, 0u);
                    cell[u] = 0;
                    if (e < total) {
                        const int r = e / q, c4 = e - r * q;
                        v[u] = *reinterpret_cast<const uint4 *>(&cnt[r * kc + c4 * 4]);
                        cell[u] = (int64_t)(m0 + r) * K + k0 + c4 * 4;
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t any = v[u].x | v[u].y | v[u].z | v[u].w;
                    if (any & 0xffffu) amx[u] = *reinterpret_cast<const int4 *>(max_count + cell[u]);
                    if (any >> 16) amn[u] = *reinterpret_cast<const int4 *>(min_count + cell[u]);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t any = v[u].x | v[u].y | v[u].z | v[u].w;
                    if (any & 0xffffu) {
                        amx[u].x += (int)(v[u].x & 0xffffu); amx[u].y += (int)(v[u].y & 0xffffu);
                        amx[u].z += (int)(v[u].z & 0xffffu); amx[u].w += (int)(v[u].w & 0xffffu);
                        *reinterpret_cast<int4 *>(max_count + cell[u]) = amx[u];
                    }
                    if (any >> 16) {
                        amn[u].x += (int)(v[u].x >> 16); amn[u].y += (int)(v[u].y >> 16);
                        amn[u].z += (int)(v[u].z >> 16); amn[u].w += (int)(v[u].w >> 16);
                        *reinterpret_cast<int4 *>(min_count + cell[u]) = amn[u];
                    }
                }
            }
        } else {
            for (int e = tid; e < rn * kn; e += NT_H) {
                const int r = e / kn, kk = e - r * kn;
                const uint32_t v = cnt[r * kc + kk];
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
        // 4 whole-K rows of packed counters in 64 KiB: two workgroups per CU
        const int budget = 64 * 1024 / 4;
        const int log2r = 2;
        const int R = 1 << log2r;
        int kc = budget / R;
        if (K < kc) kc = (int)((K + 3) / 4 * 4);
        const int64_t ktiles = ceil_div(K, kc);
        const int vec = (K % 4 == 0) && ((uintptr_t)max_count % 16 == 0) && ((uintptr_t)min_count % 16 == 0);
        const int vec_in = (M % 4 == 0) && ((uintptr_t)argmax % 16 == 0) && ((uintptr_t)argmin % 16 == 0);
        if (ktiles > 65535) return fail(MAM_ERR_UNSUPPORTED, "K too large for the selection-count grid");
        hipLaunchKernelGGL(selcount::hits_kernel, dim3((unsigned)ceil_div(M, R), (unsigned)ktiles),
                           dim3(selcount::NT_H), (size_t)R * kc * 4, st, argmax, argmin, max_count,
                           min_count, (int)N, (int)M, (int)K, log2r, kc, vec, vec_in);
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
