// MAM backward for gfx950: grad flows only through the selected argmax / argmin positions.
// Replaces the reference's one-thread-per-block global-atomic scatter
// (mamtorch/kernel/v4/csrc/cuda/fullyconnected_backward.cu:24-78 and its zero_() fills, :108-109).
//
// Both outputs are dense matrices that are almost entirely zero (at most 2*N*M non-zeros), so
// the work is bandwidth: write every output byte exactly once and read the (grad, argmax, argmin)
// triples as few times as possible.  Each workgroup OWNS a slab of an output, accumulates the
// scattered terms for that slab in an LDS histogram with ds_add_f32, and then streams the slab to
// HBM with coalesced stores -- no zero-fill pass and no global atomics:
//
//   x_grad : one workgroup per batch row n; histogram over k (chunked when K floats exceed LDS).
//   w_grad : one workgroup per R consecutive output neurons x KC consecutive k.  For the (M,K)
//            layout R = 4 so a slab is 4 whole rows of the weight gradient (64 KiB: two
//            workgroups per CU); for the (K,M) layout R = 32 so that every stored row segment is
//            128 bytes.
//
// Each term is one fp32 product (operand of the reference's atomicAdd); only the order of the
// fp32 additions differs from the reference, which is itself unordered.
#include "mam_common.h"

namespace mam {
namespace bwd {

constexpr int NT_X = 1024;
constexpr int NT_W = 512;

__device__ __forceinline__ void lds_add(float *addr, float v)
{
    __hip_atomic_fetch_add(addr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

template <int LAYOUT>
__global__ __launch_bounds__(NT_X) void mam_bwd_x_kernel(
    const float *__restrict__ w, int64_t ldw, const float *__restrict__ grad,
    const int32_t *__restrict__ argmax, const int32_t *__restrict__ argmin,
    const float *__restrict__ w_sel, int64_t nm, float *__restrict__ x_grad, int K, int M, int kc)
{
    extern __shared__ float hist[];
    const int n = blockIdx.x;
    const int tid = threadIdx.x;
    const float *g_row = grad + (int64_t)n * M;
    const int32_t *amax_row = argmax + (int64_t)n * M;
    const int32_t *amin_row = argmin + (int64_t)n * M;
    for (int k0 = 0; k0 < K; k0 += kc) {
        const int kn = (K - k0) < kc ? (K - k0) : kc;
        for (int i = tid; i < kn; i += NT_X) hist[i] = 0.0f;
        __syncthreads();
        // four outputs per thread and trip: all index loads, then all weight gathers, then the
        // LDS adds, so that the gather latencies overlap instead of adding up
        for (int mb = tid; mb < M; mb += 4 * NT_X) {
            float g[4], wv1[4], wv2[4];
            int a1[4], a2[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int m = mb + u * NT_X;
                const bool ok = m < M;
                g[u] = ok ? g_row[m] : 0.0f;
                a1[u] = ok ? amax_row[m] - k0 : -1;
                a2[u] = ok ? amin_row[m] - k0 : -1;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int m = mb + u * NT_X;
                // the forward can hand over the selected weights; otherwise gather them
                if (w_sel) {
                    const bool ok = m < M;
                    wv1[u] = ok ? w_sel[(int64_t)n * M + m] : 0.0f;
                    wv2[u] = ok ? w_sel[nm + (int64_t)n * M + m] : 0.0f;
                } else {
                    wv1[u] = (unsigned)a1[u] < (unsigned)kn ? load_w<LAYOUT>(w, ldw, a1[u] + k0, m) : 0.0f;
                    wv2[u] = (unsigned)a2[u] < (unsigned)kn ? load_w<LAYOUT>(w, ldw, a2[u] + k0, m) : 0.0f;
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if ((unsigned)a1[u] < (unsigned)kn) lds_add(&hist[a1[u]], wv1[u] * g[u]);
                if ((unsigned)a2[u] < (unsigned)kn) lds_add(&hist[a2[u]], wv2[u] * g[u]);
            }
        }
        __syncthreads();
        float *dst = x_grad + (int64_t)n * K + k0;
        for (int i = tid; i < kn; i += NT_X) dst[i] = hist[i];
        __syncthreads();
    }
}

template <int LAYOUT>
__global__ __launch_bounds__(NT_W) void mam_bwd_w_kernel(
    const float *__restrict__ x, int64_t ldx, const float *__restrict__ grad,
    const int32_t *__restrict__ argmax, const int32_t *__restrict__ argmin,
    float *__restrict__ w_grad, int N, int K, int M, int log2r, int kc, int vec_out,
    int vec_in)
{
    extern __shared__ float hist[];
    const int tid = threadIdx.x;
    const int R = 1 << log2r;
    const int mt = xcd_remap(blockIdx.x, gridDim.x);
    const int m0 = mt * R;
    const int k0 = blockIdx.y * kc;
    const int rn = (M - m0) < R ? (M - m0) : R;
    const int kn = (K - k0) < kc ? (K - k0) : kc;

    const int cells = R * kc;
    for (int i = tid * 4; i < cells; i += NT_W * 4)
        *reinterpret_cast<float4 *>(&hist[i]) = make_float4(0.f, 0.f, 0.f, 0.f);
    __syncthreads();

    if (vec_in && rn == R) {
        // a thread takes 4 consecutive neurons of one batch row: three 16-byte loads, then the
        // eight x gathers (all from one 4*K-byte row), then the LDS adds
        const int qpr = R >> 2;   // quads per row
        const int64_t items = (int64_t)N * qpr;
        for (int64_t it = tid; it < items; it += NT_W) {
            const int n = (int)(it / qpr), r0 = (int)(it - (int64_t)n * qpr) * 4;
            const int64_t o = (int64_t)n * M + m0 + r0;
            const float4 g = *reinterpret_cast<const float4 *>(grad + o);
            const int4 i1 = *reinterpret_cast<const int4 *>(argmax + o);
            const int4 i2 = *reinterpret_cast<const int4 *>(argmin + o);
            const float gv[4] = {g.x, g.y, g.z, g.w};
            const int a1[4] = {i1.x - k0, i1.y - k0, i1.z - k0, i1.w - k0};
            const int a2[4] = {i2.x - k0, i2.y - k0, i2.z - k0, i2.w - k0};
            const float *xr = x + (int64_t)n * ldx + k0;
            float x1[4], x2[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                x1[u] = (unsigned)a1[u] < (unsigned)kn ? xr[a1[u]] : 0.0f;
                x2[u] = (unsigned)a2[u] < (unsigned)kn ? xr[a2[u]] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int r = r0 + u;
                if ((unsigned)a1[u] < (unsigned)kn)
                    lds_add(&hist[LAYOUT == MAM_W_MK ? r * kc + a1[u] : (a1[u] << log2r) + r], x1[u] * gv[u]);
                if ((unsigned)a2[u] < (unsigned)kn)
                    lds_add(&hist[LAYOUT == MAM_W_MK ? r * kc + a2[u] : (a2[u] << log2r) + r], x2[u] * gv[u]);
            }
        }
    } else {
        const int64_t pairs = (int64_t)N << log2r;
        for (int64_t pi = tid; pi < pairs; pi += NT_W) {
            const int n = (int)(pi >> log2r), r = (int)(pi & (R - 1));
            if (r >= rn) continue;
            const int64_t o = (int64_t)n * M + m0 + r;
            const float g = grad[o];
            const int a1 = argmax[o] - k0, a2 = argmin[o] - k0;
            const float *xr = x + (int64_t)n * ldx + k0;
            if ((unsigned)a1 < (unsigned)kn)
                lds_add(&hist[LAYOUT == MAM_W_MK ? r * kc + a1 : (a1 << log2r) + r], xr[a1] * g);
            if ((unsigned)a2 < (unsigned)kn)
                lds_add(&hist[LAYOUT == MAM_W_MK ? r * kc + a2 : (a2 << log2r) + r], xr[a2] * g);
        }
    }
    __syncthreads();

    if (LAYOUT == MAM_W_MK) {
        if (vec_out) {  // K, k0 and kc are multiples of 4 and w_grad is 16-byte aligned
            const int q = kn >> 2;
            for (int e = tid; e < rn * q; e += NT_W) {
                const int r = e / q, c4 = e - r * q;
                *reinterpret_cast<float4 *>(w_grad + (int64_t)(m0 + r) * K + k0 + c4 * 4) =
                    *reinterpret_cast<const float4 *>(&hist[r * kc + c4 * 4]);
            }
        } else {
            for (int e = tid; e < rn * kn; e += NT_W) {
                const int r = e / kn, kk = e - r * kn;
                w_grad[(int64_t)(m0 + r) * K + k0 + kk] = hist[r * kc + kk];
            }
        }
    } else {
        for (int e = tid; e < (kn << log2r); e += NT_W) {
            const int kk = e >> log2r, r = e & (R - 1);
            if (r < rn) w_grad[(int64_t)(k0 + kk) * M + m0 + r] = hist[e];
        }
    }
}

// LDS a workgroup may use for a histogram, in floats.  gfx950 has 160 KiB per CU; above
// 64 KiB the kernel attribute has to be raised first.
static int lds_budget_floats(const void *kernel)
{
    constexpr int kWant = 128 * 1024;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kWant) == hipSuccess)
        return kWant / 4;
    (void)hipGetLastError();
    return 64 * 1024 / 4;
}

template <int LAYOUT>
static int launch_layout(const float *x, int64_t ldx, const float *w, int64_t ldw, const float *grad,
                         const int32_t *argmax, const int32_t *argmin, const float *w_sel,
                         float *x_grad, float *w_grad, int64_t N, int64_t K, int64_t M, hipStream_t st)
{
    int rc = MAM_OK;
    if (x_grad) {
        static const int budget = lds_budget_floats((const void *)mam_bwd_x_kernel<LAYOUT>);
        const int kc = (int)(K < budget ? K : budget);
        hipLaunchKernelGGL((mam_bwd_x_kernel<LAYOUT>), dim3((unsigned)N), dim3(NT_X),
                           (size_t)kc * sizeof(float), st, w, ldw, grad, argmax, argmin, w_sel, N * M,
                           x_grad, (int)K, (int)M, kc);
        rc = check_launch("mam_bwd_x_kernel");
        if (rc != MAM_OK) return rc;
    }
    if (w_grad) {
        // (M,K): 4 whole-K rows in 64 KiB, so two workgroups share a CU and one's scatter phase
        // overlaps the other's store phase.  (K,M): 32 columns x 1024 k in 128 KiB.
        static const int big = lds_budget_floats((const void *)mam_bwd_w_kernel<LAYOUT>);
        const int log2r = LAYOUT == MAM_W_MK ? 2 : 5;
        const int R = 1 << log2r;
        const int budget = LAYOUT == MAM_W_MK ? 64 * 1024 / 4 : big;
        int kc = budget / R;
        if (K < kc) kc = (int)((K + 3) / 4 * 4);
        const int64_t mtiles = ceil_div(M, R), ktiles = ceil_div(K, kc);
        if (ktiles > 65535) return fail(MAM_ERR_UNSUPPORTED, "K too large for the w_grad grid");
        const int vec_out = (K % 4 == 0) && ((uintptr_t)w_grad % 16 == 0);
        const int vec_in = (M % 4 == 0) && ((uintptr_t)grad % 16 == 0) && ((uintptr_t)argmax % 16 == 0) &&
                           ((uintptr_t)argmin % 16 == 0);
        hipLaunchKernelGGL((mam_bwd_w_kernel<LAYOUT>), dim3((unsigned)mtiles, (unsigned)ktiles),
                           dim3(NT_W), (size_t)R * kc * sizeof(float), st, x, ldx, grad, argmax,
                           argmin, w_grad, (int)N, (int)K, (int)M, log2r, kc, vec_out, vec_in);
        rc = check_launch("mam_bwd_w_kernel");
    }
    return rc;
}

}  // namespace bwd
}  // namespace mam

extern "C" int mam_fc_backward(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                               const float *grad, const int32_t *argmax, const int32_t *argmin,
                               const float *w_sel, float *x_grad, float *w_grad, int64_t N, int64_t K,
                               int64_t M, void *stream)
{
    using namespace mam;
    if (N < 0 || K < 0 || M < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (w_layout != MAM_W_KM && w_layout != MAM_W_MK)
        return fail(MAM_ERR_INVALID_ARGUMENT, "w_layout must be MAM_W_KM or MAM_W_MK");
    if (K == 0 || (N == 0 && M == 0)) return MAM_OK;
    if (N > INT32_MAX / 2 || K > INT32_MAX / 2 || M > INT32_MAX / 2)
        return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (N == 0 || M == 0) {  // no terms: the gradients are all zero
        int rc = MAM_OK;
        if (x_grad && N > 0) rc = fill_zero(x_grad, N * K, st);
        if (rc == MAM_OK && w_grad && M > 0) rc = fill_zero(w_grad, M * K, st);
        return rc;
    }
    if (!x || !w || !grad || !argmax || !argmin) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (ldx < K || ldw < (w_layout == MAM_W_MK ? K : M))
        return fail(MAM_ERR_INVALID_ARGUMENT, "leading dimension smaller than the row length");
    if (w_layout == MAM_W_MK)
        return bwd::launch_layout<MAM_W_MK>(x, ldx, w, ldw, grad, argmax, argmin, w_sel, x_grad, w_grad, N, K, M, st);
    return bwd::launch_layout<MAM_W_KM>(x, ldx, w, ldw, grad, argmax, argmin, w_sel, x_grad, w_grad, N, K, M, st);
}
