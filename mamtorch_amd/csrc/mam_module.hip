// Module-level helpers around the MAM kernels on gfx950: the vanishing-contribution blend of
// FullyConnected and the window gather / scatter that turns a MAM convolution into the MAM
// fully-connected kernel.  All HBM-bound elementwise or gather work.
//
//  * mam_blend: out = (alpha * mam + beta * mac) + bias, the module's MAC blend
//    (mamtorch/nn/v4/fullyconnected.py:190-198) in one pass and in the reference's rounding order
//    (two products, their sum, then the bias; no fused multiply-add).
//  * mam_apply_keep: the training-time weight dropout (mamtorch/nn/v4/fullyconnected.py:143-148) from a
//    byte mask, one pass over the weight.
//  * mam_im2col / mam_col2im: the reference's retired MAM convolutions
//    (mamtorch/kernel/backup/mamconv1d_forward.txt:26-166, mamconv2d_forward.txt) run the MAM reduction
//    over the window positions and channels of each output position, with the index
//    arg = (j2 * k1 + j1) * C + c (window column j2 outermost, then window row j1, channel innermost;
//    mamconv1d_forward.txt:128, and the decoding in mamtorch/nn/backup/mamconv2d.txt:97-103).  Here the
//    windows are gathered once into a (B * L1 * L2, k2 * k1 * C) operand in exactly that column
//    order, so that mam_fc_forward's argmax / argmin ARE the reference's indices; col2im is the
//    adjoint (gradient with respect to the input), written as a gather so that it needs no atomics.
#include "mam_common.h"

namespace mam {
namespace module {

__global__ __launch_bounds__(256) void blend_kernel(const float *__restrict__ mam, const float *__restrict__ mac,
                                                    const float *__restrict__ bias, float alpha, float beta,
                                                    float *__restrict__ out, int64_t total, int M, int vec)
{
    const int64_t stride = (int64_t)gridDim.x * 256;
    if (vec) {
        const int64_t quads = total >> 2;
        for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < quads; q += stride) {
            const float4 a = reinterpret_cast<const float4 *>(mam)[q];
            const float4 b = reinterpret_cast<const float4 *>(mac)[q];
            float4 r;
            r.x = alpha * a.x + beta * b.x; r.y = alpha * a.y + beta * b.y;
            r.z = alpha * a.z + beta * b.z; r.w = alpha * a.w + beta * b.w;
            if (bias) {
                const float4 c = *reinterpret_cast<const float4 *>(bias + (q * 4) % M);
                r.x = r.x + c.x; r.y = r.y + c.y; r.z = r.z + c.z; r.w = r.w + c.w;
            }
            reinterpret_cast<float4 *>(out)[q] = r;
        }
    } else {
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
            float r = alpha * mam[i] + beta * mac[i];
            if (bias) r = r + bias[i % M];
            out[i] = r;
        }
    }
}

// out[m][k] = w[m][k] * (keep[m][k] ? 1 : 0): the training-time weight dropout of the module
// (mamtorch/nn/v4/fullyconnected.py:143-148: `weight * bernoulli mask`) with the mask as one byte per
// weight.  The product keeps the reference's bits: a dropped weight becomes a zero with the weight's sign,
// and a non-finite one becomes NaN.
__global__ __launch_bounds__(256) void keep_kernel(const float *__restrict__ w, int64_t ldw,
                                                   const unsigned char *__restrict__ keep,
                                                   float *__restrict__ out, int64_t M, int K, int vec)
{
    const int64_t stride = (int64_t)gridDim.x * 256;
    if (vec) {
        const int qpr = K >> 2;                   // quads per row
        const int64_t quads = M * (int64_t)qpr;
        for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < quads; q += stride) {
            const int64_t m = q / qpr;
            const int k = (int)(q - m * qpr) << 2;
            const float4 a = *reinterpret_cast<const float4 *>(w + m * ldw + k);
            const uint32_t kb = *reinterpret_cast<const uint32_t *>(keep + m * K + k);
            float4 r;
            r.x = a.x * ((kb & 0xffu) ? 1.0f : 0.0f);
            r.y = a.y * ((kb & 0xff00u) ? 1.0f : 0.0f);
            r.z = a.z * ((kb & 0xff0000u) ? 1.0f : 0.0f);
            r.w = a.w * ((kb & 0xff000000u) ? 1.0f : 0.0f);
            *reinterpret_cast<float4 *>(out + m * K + k) = r;
        }
    } else {
        const int64_t total = M * (int64_t)K;
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
            const int64_t m = i / K;
            const int k = (int)(i - m * K);
            out[i] = w[m * ldw + k] * (keep[i] ? 1.0f : 0.0f);
        }
    }
}

struct ConvGeom {
    int B, C, H, W;        // input (B, C, H, W), contiguous
    int k1, k2, s1, s2;    // window rows / columns, strides along H / W
    int L1, L2;            // output positions along H / W
    int ctiles, wtiles;    // 32-wide tiles of channels, of the W axis (output positions or input columns)
};

// One workgroup: fixed (b, l1, j1, j2), a tile of 32 channels x 32 output columns l2.  The input is read
// with l2 fastest (contiguous when s2 == 1), the operand is written with the channel fastest.
__global__ __launch_bounds__(256) void im2col_kernel(const float *__restrict__ x, float *__restrict__ cols,
                                                     const ConvGeom g)
{
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    int64_t id = blockIdx.x;
    const int wt = (int)(id % g.wtiles); id /= g.wtiles;
    const int ct = (int)(id % g.ctiles); id /= g.ctiles;
    const int j2 = (int)(id % g.k2); id /= g.k2;
    const int j1 = (int)(id % g.k1); id /= g.k1;
    const int l1 = (int)(id % g.L1);
    const int b = (int)(id / g.L1);
    const int c0 = ct * 32, w0 = wt * 32;
    const int h = l1 * g.s1 + j1;
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const int c = c0 + r, l2 = w0 + tx;
        float v = 0.0f;
        if (c < g.C && l2 < g.L2)
            v = x[(((int64_t)b * g.C + c) * g.H + h) * g.W + (int64_t)l2 * g.s2 + j2];
        tile[r][tx] = v;
    }
    __syncthreads();
    const int64_t K = (int64_t)g.k2 * g.k1 * g.C;
    const int64_t q0 = ((int64_t)j2 * g.k1 + j1) * g.C + c0;
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const int l2 = w0 + r, c = c0 + tx;
        if (l2 < g.L2 && c < g.C) {
            const int64_t row = ((int64_t)b * g.L1 + l1) * g.L2 + l2;
            cols[row * K + q0 + tx] = tile[tx][r];
        }
    }
}

// Adjoint of the gather: one workgroup owns (b, h) and a tile of 32 channels x 32 input columns w, and
// sums, in ascending (j1, j2), the operand-gradient cells of every window that covers each input cell.
__global__ __launch_bounds__(256) void col2im_kernel(const float *__restrict__ cols, float *__restrict__ xg,
                                                     const ConvGeom g)
{
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    int64_t id = blockIdx.x;
    const int wt = (int)(id % g.wtiles); id /= g.wtiles;
    const int ct = (int)(id % g.ctiles); id /= g.ctiles;
    const int h = (int)(id % g.H);
    const int b = (int)(id / g.H);
    const int c0 = ct * 32, w0 = wt * 32;
    const int64_t K = (int64_t)g.k2 * g.k1 * g.C;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};     // cells (w = w0 + ty + 8 i, c = c0 + tx)
    const int c = c0 + tx;
    for (int j1 = 0; j1 < g.k1; ++j1) {
        const int hh = h - j1;
        if (hh < 0 || hh % g.s1 != 0) continue;
        const int l1 = hh / g.s1;
        if (l1 >= g.L1) continue;
        for (int j2 = 0; j2 < g.k2; ++j2) {
            const int64_t q = ((int64_t)j2 * g.k1 + j1) * g.C + c;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int w = w0 + ty + 8 * i;
                const int ww = w - j2;
                if (w < g.W && c < g.C && ww >= 0 && ww % g.s2 == 0 && ww / g.s2 < g.L2) {
                    const int64_t row = ((int64_t)b * g.L1 + l1) * g.L2 + ww / g.s2;
                    acc[i] = acc[i] + cols[row * K + q];
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) tile[ty + 8 * i][tx] = acc[i];
    __syncthreads();
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const int cc = c0 + r, w = w0 + tx;
        if (cc < g.C && w < g.W) xg[(((int64_t)b * g.C + cc) * g.H + h) * g.W + w] = tile[tx][r];
    }
}

static int make_geom(ConvGeom &g, int64_t B, int64_t C, int64_t H, int64_t W, int64_t k1, int64_t k2, int64_t s1,
                     int64_t s2)
{
    if (B < 0 || C < 0 || H < 0 || W < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (k1 < 1 || k2 < 1 || s1 < 1 || s2 < 1) return fail(MAM_ERR_INVALID_ARGUMENT, "window and stride must be positive");
    if (k1 > H || k2 > W) return fail(MAM_ERR_INVALID_ARGUMENT, "the window is larger than the input");
    const int64_t L1 = (H - k1) / s1 + 1, L2 = (W - k2) / s2 + 1;
    if (B * C * H * W > ((int64_t)1 << 40) || B * L1 * L2 > INT32_MAX / 2 || k1 * k2 * C > INT32_MAX / 2 ||
        H > INT32_MAX / 2 || W > INT32_MAX / 2)
        return fail(MAM_ERR_UNSUPPORTED, "convolution geometry too large");
    g.B = (int)B; g.C = (int)C; g.H = (int)H; g.W = (int)W;
    g.k1 = (int)k1; g.k2 = (int)k2; g.s1 = (int)s1; g.s2 = (int)s2;
    g.L1 = (int)L1; g.L2 = (int)L2;
    g.ctiles = (int)ceil_div(C, 32);
    return MAM_OK;
}

}  // namespace module
// Column sums of grad (N, M): the gradient of the bias that the layer adds after max + min
// (mamtorch/nn/v4/fullyconnected.py:197-198; the reference leaves this sum to autograd).  A workgroup owns 64
// columns and a slab of the batch rows: its four waves take every fourth row of the slab (a row piece of 64
// columns is one coalesced 256-byte load, eight of them in flight per wave), add in row order, and the four
// partial sums are added in wave order -- the result does not depend on timing.  With several slabs the
// partial rows go to the workspace and a second launch adds them in slab order.
__global__ __launch_bounds__(256) void col_sum_kernel(const float *__restrict__ grad, int64_t ld,
                                                      float *__restrict__ out, int N, int M, int rows_per_slab)
{
    __shared__ float part[4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = blockIdx.x * 64 + lane;
    const int n_begin = blockIdx.y * rows_per_slab;
    const int n_end = (n_begin + rows_per_slab) < N ? (n_begin + rows_per_slab) : N;
    float acc = 0.0f;
    if (m < M) {
        const float *col = grad + m;
        int n = n_begin + wave;
        for (; n + 28 < n_end; n += 32) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = col[(int64_t)(n + 4 * u) * ld];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += v[u];
        }
        for (; n < n_end; n += 4) acc += col[(int64_t)n * ld];
    }
    part[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && m < M)
        out[(int64_t)blockIdx.y * M + m] = ((part[0][lane] + part[1][lane]) + part[2][lane]) + part[3][lane];
}

__global__ __launch_bounds__(256) void slab_sum_kernel(const float *__restrict__ partial, float *__restrict__ out,
                                                       int M, int slabs)
{
    const int m = blockIdx.x * 256 + threadIdx.x;
    if (m >= M) return;
    float acc = 0.0f;
    for (int s = 0; s < slabs; ++s) acc += partial[(int64_t)s * M + m];
    out[m] = acc;
}

// slabs of the batch: one up to 512 rows, else slabs of at least 128 rows, at most 64 of them
static int64_t bias_grad_slabs(int64_t N)
{
    if (N <= 512) return 1;
    int64_t s = N / 128;
    return s > 64 ? 64 : s;
}

}  // namespace mam

extern "C" size_t mam_bias_grad_workspace(int64_t N, int64_t M)
{
    if (N <= 0 || M <= 0) return 0;
    const int64_t slabs = mam::bias_grad_slabs(N);
    return slabs > 1 ? (size_t)slabs * (size_t)M * sizeof(float) : 0;
}

extern "C" int mam_bias_grad(const float *grad, int64_t ld, float *bias_grad, int64_t N, int64_t M, void *workspace,
                             size_t workspace_bytes, void *stream)
{
    using namespace mam;
    if (N < 0 || M < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (M == 0) return MAM_OK;
    if (!bias_grad) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (N == 0) return fill_zero(bias_grad, M, st);
    if (!grad) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (ld < M) return fail(MAM_ERR_INVALID_ARGUMENT, "ld smaller than the number of columns");
    if (N > INT32_MAX / 2 || M > INT32_MAX / 2) return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    const int64_t slabs = bias_grad_slabs(N);
    const size_t need = slabs > 1 ? (size_t)slabs * (size_t)M * sizeof(float) : 0;
    if (need > 0 && (!workspace || workspace_bytes < need))
        return fail(MAM_ERR_WORKSPACE, "the bias gradient needs %zu workspace bytes, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    const int64_t rows_per_slab = ceil_div(N, slabs);
    float *first = slabs > 1 ? static_cast<float *>(workspace) : bias_grad;
    hipLaunchKernelGGL(col_sum_kernel, dim3((unsigned)ceil_div(M, 64), (unsigned)slabs), dim3(256), 0, st, grad, ld, first,
                       (int)N, (int)M, (int)rows_per_slab);
    int rc = check_launch("col_sum_kernel");
    if (rc != MAM_OK || slabs == 1) return rc;
    hipLaunchKernelGGL(slab_sum_kernel, dim3((unsigned)ceil_div(M, 256)), dim3(256), 0, st, first, bias_grad, (int)M,
                       (int)slabs);
    return check_launch("slab_sum_kernel");
}

extern "C" int mam_blend(const float *mam_out, const float *mac_out, const float *bias, float alpha, float beta,
                         float *out, int64_t N, int64_t M, void *stream)
{
    using namespace mam;
    if (N < 0 || M < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (N == 0 || M == 0) return MAM_OK;
    if (!mam_out || !mac_out || !out) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (M > INT32_MAX / 2) return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    const int64_t total = N * M;
    const int vec = (M % 4 == 0) && ((uintptr_t)mam_out % 16 == 0) && ((uintptr_t)mac_out % 16 == 0) &&
                    ((uintptr_t)out % 16 == 0) && ((uintptr_t)bias % 16 == 0);
    int64_t blocks = ceil_div(vec ? total / 4 : total, 256);
    if (blocks > 16 * num_cus()) blocks = 16 * num_cus();
    hipLaunchKernelGGL(module::blend_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       mam_out, mac_out, bias, alpha, beta, out, total, (int)M, vec);
    return check_launch("blend_kernel");
}

extern "C" int mam_apply_keep(const float *w, int64_t ldw, const unsigned char *keep, float *out, int64_t M,
                              int64_t K, void *stream)
{
    using namespace mam;
    if (M < 0 || K < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (M == 0 || K == 0) return MAM_OK;
    if (!w || !keep || !out) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (ldw < K) return fail(MAM_ERR_INVALID_ARGUMENT, "leading dimension smaller than the row length");
    if (K > INT32_MAX / 2 || M > INT32_MAX / 2) return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    const int vec = (K % 4 == 0) && (ldw % 4 == 0) && ((uintptr_t)w % 16 == 0) && ((uintptr_t)out % 16 == 0) &&
                    ((uintptr_t)keep % 4 == 0);
    const int64_t total = M * K;
    int64_t blocks = ceil_div(vec ? total / 4 : total, 256);
    if (blocks > 16 * num_cus()) blocks = 16 * num_cus();
    hipLaunchKernelGGL(module::keep_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream), w,
                       ldw, keep, out, M, (int)K, vec);
    return check_launch("keep_kernel");
}

extern "C" int mam_im2col(const float *x, float *cols, int64_t B, int64_t C, int64_t H, int64_t W, int64_t k1,
                          int64_t k2, int64_t s1, int64_t s2, void *stream)
{
    using namespace mam;
    module::ConvGeom g;
    const int rc = module::make_geom(g, B, C, H, W, k1, k2, s1, s2);
    if (rc != MAM_OK) return rc;
    if (B == 0 || C == 0) return MAM_OK;
    if (!x || !cols) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    g.wtiles = (int)ceil_div(g.L2, 32);
    const int64_t blocks = (int64_t)g.B * g.L1 * g.k1 * g.k2 * g.ctiles * g.wtiles;
    if (blocks > INT32_MAX) return fail(MAM_ERR_UNSUPPORTED, "too many tiles");
    hipLaunchKernelGGL(module::im2col_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream), x,
                       cols, g);
    return check_launch("im2col_kernel");
}

extern "C" int mam_col2im(const float *cols, float *x_grad, int64_t B, int64_t C, int64_t H, int64_t W, int64_t k1,
                          int64_t k2, int64_t s1, int64_t s2, void *stream)
{
    using namespace mam;
    module::ConvGeom g;
    const int rc = module::make_geom(g, B, C, H, W, k1, k2, s1, s2);
    if (rc != MAM_OK) return rc;
    if (B == 0 || C == 0) return MAM_OK;
    if (!x_grad || !cols) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    g.wtiles = (int)ceil_div(g.W, 32);
    const int64_t blocks = (int64_t)g.B * g.H * g.ctiles * g.wtiles;
    if (blocks > INT32_MAX) return fail(MAM_ERR_UNSUPPORTED, "too many tiles");
    hipLaunchKernelGGL(module::col2im_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       cols, x_grad, g);
    return check_launch("col2im_kernel");
}
