// The pruning threshold on the device (gfx950): the element of a given rank among the absolute scores of
// one or several weight matrices, without sorting them.
//
// The reference finds its thresholds with torch.quantile over one layer's |scores|
// (examples/vitb16_imagenet1k/pruning_utils.py:103-104) or by sorting the concatenated |scores| of every
// layer and taking the element of rank int(p * n) (:139-143): a full sort of 16.8 M (one 4096 x 4096 layer)
// to hundreds of millions of floats for ONE number.  Here the number is found by a radix select over the
// bit patterns of the scores: a non-negative fp32 orders like its bit pattern (NaN above infinity, where
// torch.sort puts it too), so three histogram passes over the 31 key bits (11 + 11 + 9 bits, 2048-bin
// histograms in LDS, flushed to a global histogram with integer atomics) narrow the bins down to the one
// key that holds the rank; a one-workgroup step after each pass walks the histogram and fixes the digit.
// One or two ranks are followed at once (torch.quantile interpolates between two neighbours), and the
// passes take any number of tensors, so the global rule needs no concatenated copy.  Every pass streams
// the scores once: 3 x 4 bytes per element (plus the second operand of a product or count score).
//
// Scores are those of the pruning kernels (mam_prune.hip): |w|, |w * aux| or aux (+ aux2) selection counts.
#include "mam_common.h"

namespace mam {
namespace selectk {

constexpr int NT = 256;        // begin / advance
constexpr int NT_H = 1024;     // histogram passes
constexpr int BINS = 2048;
constexpr int MAX_RANKS = 2;
constexpr int PASSES = 3;

struct State {
    uint32_t prefix[MAX_RANKS];     // digits fixed so far, right-aligned
    uint32_t nranks, pad;
    int64_t rank[MAX_RANKS];        // rank still to go within the elements that share the prefix
};
// workspace: State, then hist[PASSES][MAX_RANKS][BINS] of 64-bit counts (the tensors of one selection may hold
// more than 2^32 elements together; a workgroup's own LDS bins are 32 bits)
typedef unsigned long long count_t;
constexpr size_t kHistWords = (size_t)PASSES * MAX_RANKS * BINS;
constexpr size_t kWorkspaceBytes = 256 + kHistWords * sizeof(count_t);

// keys are 31 bits wide (absolute values: the sign bit is clear): digits of 11, 11 and 9 bits
__host__ __device__ constexpr int pass_shift(int pass) { return pass == 0 ? 20 : pass == 1 ? 9 : 0; }
__host__ __device__ constexpr int pass_bits(int pass) { return pass == 2 ? 9 : 11; }

template <int MODE>
__device__ __forceinline__ uint32_t key_of(float w, const void *aux, const void *aux2, int64_t idx)
{
    if (MODE == MAM_PRUNE_MAGNITUDE) return __float_as_uint(w) & 0x7fffffffu;
    if (MODE == MAM_PRUNE_WEIGHT_TIMES) return __float_as_uint(w * static_cast<const float *>(aux)[idx]) & 0x7fffffffu;
    int cnt = static_cast<const int32_t *>(aux)[idx];
    if (aux2) cnt += static_cast<const int32_t *>(aux2)[idx];
    return (uint32_t)(cnt < 0 ? -cnt : cnt);
}

__global__ __launch_bounds__(NT) void begin_kernel(State *st, count_t *hist, int64_t r0, int64_t r1, int nranks)
{
    for (size_t i = (size_t)blockIdx.x * NT + threadIdx.x; i < kHistWords; i += (size_t)gridDim.x * NT) hist[i] = 0ull;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        st->prefix[0] = st->prefix[1] = 0u;
        st->nranks = (uint32_t)nranks;
        st->pad = 0u;
        st->rank[0] = r0;
        st->rank[1] = r1;
    }
}

// One histogram pass over one matrix.  vec: 16-byte loads (K a multiple of 4, aligned rows).
template <int MODE>
__global__ __launch_bounds__(NT_H) void hist_kernel(const float *__restrict__ w, int64_t ldw, const void *aux,
                                                  const void *aux2, int64_t ld_aux, int64_t M, int64_t K, int vec,
                                                  const State *__restrict__ st, count_t *__restrict__ hist, int pass)
{
    __shared__ uint32_t bins[MAX_RANKS][BINS];
    const int tid = threadIdx.x;
    for (int i = tid; i < MAX_RANKS * BINS; i += NT_H) (&bins[0][0])[i] = 0u;
    const int nr = (int)st->nranks;
    const int shift = pass_shift(pass), nb = pass_bits(pass);
    const uint32_t mask = (1u << nb) - 1u;
    const uint32_t p0 = st->prefix[0], p1 = st->prefix[1];
    const bool one = nr < 2 || p0 == p1;     // both ranks still in the same bin: one histogram serves both
    __syncthreads();
    // Scores crowd into few bins (the first pass looks at the exponent and three mantissa bits), and an
    // LDS atomic costs per lane that shares an address: a thread keeps a run of equal digits in registers
    // and adds it when the digit changes.
    uint32_t run_digit[MAX_RANKS] = {0u, 0u}, run_count[MAX_RANKS] = {0u, 0u};
    auto bump = [&](int s, uint32_t digit) {
        if (digit == run_digit[s]) {
            ++run_count[s];
        } else {
            if (run_count[s]) atomicAdd(&bins[s][run_digit[s]], run_count[s]);
            run_digit[s] = digit;
            run_count[s] = 1u;
        }
    };
    auto take = [&](uint32_t key) {
        const uint32_t hi = pass == 0 ? 0u : key >> (shift + nb);
        const uint32_t digit = (key >> shift) & mask;
        if (hi == p0) bump(0, digit);
        if (!one && hi == p1) bump(1, digit);
    };
    const int64_t stride = (int64_t)gridDim.x * NT_H;
    if (vec) {
        const int64_t q = K >> 2, items = M * q;
        for (int64_t it = (int64_t)blockIdx.x * NT_H + tid; it < items; it += stride) {
            const int64_t r = it / q, c = (it - r * q) * 4;
            const int64_t a = r * ld_aux + c;
            if (MODE == MAM_PRUNE_COUNT) {
                int4 cnt = *reinterpret_cast<const int4 *>(static_cast<const int32_t *>(aux) + a);
                if (aux2) {
                    const int4 c2 = *reinterpret_cast<const int4 *>(static_cast<const int32_t *>(aux2) + a);
                    cnt.x += c2.x; cnt.y += c2.y; cnt.z += c2.z; cnt.w += c2.w;
                }
                take((uint32_t)(cnt.x < 0 ? -cnt.x : cnt.x)); take((uint32_t)(cnt.y < 0 ? -cnt.y : cnt.y));
                take((uint32_t)(cnt.z < 0 ? -cnt.z : cnt.z)); take((uint32_t)(cnt.w < 0 ? -cnt.w : cnt.w));
            } else {
                float4 v = *reinterpret_cast<const float4 *>(w + r * ldw + c);
                if (MODE == MAM_PRUNE_WEIGHT_TIMES) {
                    const float4 f = *reinterpret_cast<const float4 *>(static_cast<const float *>(aux) + a);
                    v.x *= f.x; v.y *= f.y; v.z *= f.z; v.w *= f.w;
                }
                take(__float_as_uint(v.x) & 0x7fffffffu); take(__float_as_uint(v.y) & 0x7fffffffu);
                take(__float_as_uint(v.z) & 0x7fffffffu); take(__float_as_uint(v.w) & 0x7fffffffu);
            }
        }
    } else {
        const int64_t items = M * K;
        for (int64_t it = (int64_t)blockIdx.x * NT_H + tid; it < items; it += stride) {
            const int64_t r = it / K, c = it - r * K;
            const float wv = MODE == MAM_PRUNE_COUNT ? 0.0f : w[r * ldw + c];
            take(key_of<MODE>(wv, aux, aux2, r * ld_aux + c));
        }
    }
#pragma unroll
    for (int s = 0; s < MAX_RANKS; ++s)
        if (run_count[s]) atomicAdd(&bins[s][run_digit[s]], run_count[s]);
    __syncthreads();
    count_t *out = hist + (size_t)pass * MAX_RANKS * BINS;
    for (int i = tid; i < (one ? 1 : MAX_RANKS) * BINS; i += NT_H) {
        const uint32_t v = (&bins[0][0])[i];
        if (v) atomicAdd(&out[i], (count_t)v);
    }
}

// After every tensor has been through pass `pass`: walk the histogram(s) and fix the digit of each rank.
__global__ __launch_bounds__(NT) void advance_kernel(State *st, const count_t *__restrict__ hist, int pass)
{
    __shared__ int64_t partial[NT];
    const int tid = threadIdx.x;
    const int nr = (int)st->nranks;
    const bool one = nr < 2 || st->prefix[0] == st->prefix[1];
    const int nbins = 1 << pass_bits(pass);
    const int per = BINS / NT;     // 8 bins per thread
    uint32_t digit[MAX_RANKS] = {0u, 0u};
    int64_t rest[MAX_RANKS] = {0, 0};
    for (int s = 0; s < nr; ++s) {
        const count_t *h = hist + ((size_t)pass * MAX_RANKS + (one ? 0 : s)) * BINS;
        int64_t sum = 0;
        for (int b = 0; b < per; ++b) sum += (tid * per + b) < nbins ? (int64_t)h[tid * per + b] : 0;
        partial[tid] = sum;
        __syncthreads();
        if (tid == 0) {
            int64_t r = st->rank[s], below = 0;
            int t = 0;
            while (t < NT - 1 && below + partial[t] <= r) below += partial[t++];
            int b = t * per;
            while (b < nbins - 1 && below + (int64_t)h[b] <= r) below += (int64_t)h[b++];
            digit[s] = (uint32_t)b;
            rest[s] = r - below;
        }
        __syncthreads();
    }
    if (tid == 0) {
        for (int s = 0; s < nr; ++s) {
            st->prefix[s] = (st->prefix[s] << pass_bits(pass)) | digit[s];
            st->rank[s] = rest[s];
        }
    }
}

__global__ void result_kernel(const State *st, float *out, int as_count)
{
    const int s = threadIdx.x;
    if (s < (int)st->nranks) out[s] = as_count ? (float)(int)st->prefix[s] : __uint_as_float(st->prefix[s]);
}

static count_t *hist_of(void *workspace) { return reinterpret_cast<count_t *>(static_cast<char *>(workspace) + 256); }

}  // namespace selectk
}  // namespace mam

extern "C" size_t mam_select_workspace(void) { return mam::selectk::kWorkspaceBytes; }

extern "C" int mam_select_begin(void *workspace, size_t workspace_bytes, const int64_t *ranks, int nranks, void *stream)
{
    using namespace mam;
    if (!workspace || workspace_bytes < selectk::kWorkspaceBytes || (uintptr_t)workspace % 16 != 0)
        return fail(MAM_ERR_WORKSPACE, "the selection needs %zu workspace bytes, 16-byte aligned", selectk::kWorkspaceBytes);
    if (!ranks || nranks < 1 || nranks > selectk::MAX_RANKS)
        return fail(MAM_ERR_INVALID_ARGUMENT, "one or two ranks");
    if (ranks[0] < 0 || (nranks == 2 && ranks[1] < ranks[0]))
        return fail(MAM_ERR_INVALID_ARGUMENT, "ranks must be non-negative and ascending");
    hipLaunchKernelGGL(selectk::begin_kernel, dim3(24), dim3(selectk::NT), 0, static_cast<hipStream_t>(stream),
                       static_cast<selectk::State *>(workspace), selectk::hist_of(workspace), ranks[0],
                       nranks == 2 ? ranks[1] : ranks[0], nranks);
    return check_launch("select begin_kernel");
}

extern "C" int mam_select_accumulate(void *workspace, const float *w, int64_t ldw, int mode, const void *aux,
                                     const void *aux2, int64_t ld_aux, int64_t M, int64_t K, int pass, void *stream)
{
    using namespace mam;
    if (!workspace) return fail(MAM_ERR_WORKSPACE, "no workspace");
    if (M < 0 || K < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (pass < 0 || pass >= selectk::PASSES) return fail(MAM_ERR_INVALID_ARGUMENT, "pass must be 0, 1 or 2");
    if (mode != MAM_PRUNE_MAGNITUDE && mode != MAM_PRUNE_WEIGHT_TIMES && mode != MAM_PRUNE_COUNT)
        return fail(MAM_ERR_INVALID_ARGUMENT, "unknown score mode %d", mode);
    if (M == 0 || K == 0) return MAM_OK;
    if ((mode != MAM_PRUNE_COUNT && !w) || (mode != MAM_PRUNE_MAGNITUDE && !aux))
        return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if ((mode != MAM_PRUNE_COUNT && ldw < K) || (mode != MAM_PRUNE_MAGNITUDE && ld_aux < K))
        return fail(MAM_ERR_INVALID_ARGUMENT, "leading dimension smaller than the row length");
    const bool vec = K % 4 == 0 && (mode == MAM_PRUNE_COUNT || ((uintptr_t)w % 16 == 0 && ldw % 4 == 0)) &&
                     (mode == MAM_PRUNE_MAGNITUDE || ((uintptr_t)aux % 16 == 0 && (uintptr_t)aux2 % 16 == 0 && ld_aux % 4 == 0));
    const int64_t items = vec ? M * (K / 4) : M * K;
    // few, large workgroups: every workgroup ends by adding its non-empty bins to the global histogram
    int64_t blocks = ceil_div(items, selectk::NT_H * 4);
    const int64_t cap = 2 * (int64_t)num_cus();
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const selectk::State *state = static_cast<const selectk::State *>(workspace);
    selectk::count_t *hist = selectk::hist_of(workspace);
#define MAM_SELECT_LAUNCH(MODE)                                                                                      \
    hipLaunchKernelGGL(selectk::hist_kernel<MODE>, dim3((unsigned)blocks), dim3(selectk::NT_H), 0, st, w, ldw, aux, aux2, \
                       ld_aux, M, K, vec ? 1 : 0, state, hist, pass)
    if (mode == MAM_PRUNE_MAGNITUDE) MAM_SELECT_LAUNCH(MAM_PRUNE_MAGNITUDE);
    else if (mode == MAM_PRUNE_WEIGHT_TIMES) MAM_SELECT_LAUNCH(MAM_PRUNE_WEIGHT_TIMES);
    else MAM_SELECT_LAUNCH(MAM_PRUNE_COUNT);
#undef MAM_SELECT_LAUNCH
    return check_launch("select hist_kernel");
}

extern "C" int mam_select_advance(void *workspace, int pass, void *stream)
{
    using namespace mam;
    if (!workspace) return fail(MAM_ERR_WORKSPACE, "no workspace");
    if (pass < 0 || pass >= selectk::PASSES) return fail(MAM_ERR_INVALID_ARGUMENT, "pass must be 0, 1 or 2");
    hipLaunchKernelGGL(selectk::advance_kernel, dim3(1), dim3(selectk::NT), 0, static_cast<hipStream_t>(stream),
                       static_cast<selectk::State *>(workspace), selectk::hist_of(workspace), pass);
    return check_launch("select advance_kernel");
}

extern "C" int mam_select_result(void *workspace, int mode, float *out, void *stream)
{
    using namespace mam;
    if (!workspace || !out) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    hipLaunchKernelGGL(selectk::result_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                       static_cast<const selectk::State *>(workspace), out, mode == MAM_PRUNE_COUNT ? 1 : 0);
    return check_launch("select result_kernel");
}
