// MAM backward for gfx950: grad flows only through the selected argmax / argmin positions.
// Replaces the reference's one-thread-per-block global-atomic scatter
// (mamtorch/kernel/v4/csrc/cuda/fullyconnected_backward.cu:24-78 and its zero_() fills, :108-109).
//
// Both outputs are dense matrices that are almost entirely zero (at most 2*N*M non-zeros), so
// the work is bandwidth: write every output byte exactly once and read the (grad, argmax, argmin)
// triples as few times as possible.  Each workgroup OWNS a slab of an output, accumulates the
// scattered terms for that slab in LDS, and then streams the slab to HBM with coalesced stores --
// no zero-fill pass and no global atomics:
//
//   x_grad : one workgroup per batch row n; cells over k (chunked when they exceed LDS).  From 2048
//            batch rows on: 2 to 16 rows per workgroup, the lanes of a wave spread over them.  The cells
//            are 64-bit fixed point (integer LDS atomics, exact sums, see below).
//   w_grad : one workgroup per R consecutive output neurons x KC consecutive k, fp32 cells.  For the (M,K)
//            layout R = 4 so a slab is 4 whole rows of the weight gradient (64 KiB: two
//            workgroups per CU); for the (K,M) layout R = 32 so that every stored row segment is
//            128 bytes.  From 2048 batch rows on, (M,K): up to 16 neurons per slab and the batch shared
//            by several workgroups per slab, which add their shares to the cleared w_grad.
//
// Each term is one fp32 product (operand of the reference's atomicAdd).  x_grad is the exact sum of its
// terms rounded once -- as long as at most QCAP (512) terms of a workgroup's slab fall outside its
// fixed-point window (they are added in fp64 before the rounding); a slab with more of them falls back to
// fp32 LDS atomics and is then a sum in arrival order.  In w_grad only the order of the fp32 additions
// differs from the reference, which is itself unordered; option MAM_OPT_BACKWARD_EXACT accumulates it in
// fixed-point cells as well (mam_bwd_w_exact_kernel).
#include "mam_common.h"
#include "mam_fixed.h"
#include "mam_count_stream.h"

namespace mam {
namespace bwd {

using namespace fixedpoint;

constexpr int NT_X = 1024;
constexpr int NT_W = 512;

// ds_add_f32 costs ~3 cycles per active lane on this chip, ~190 per full 64-lane instruction,
// whatever the addresses (an integer LDS atomic: ~5 per instruction, ~8 for 64 bits).  Only the fp32
// fallback of x_grad still uses it.
__device__ __forceinline__ void lds_add(float *addr, float v)
{
    __hip_atomic_fetch_add(addr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// Where collisions inside one instruction are rare (w_grad: a slab is sparse and its keys spread):
// one compare-and-swap round (~15 cycles per instruction) settles every lane that met no
// contender; only the losers go through the slow float atomic.
__device__ __forceinline__ void lds_add_sparse(float *addr, float v)
{
    int *word = reinterpret_cast<int *>(addr);
    const int seen = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    int expected = seen;
    const bool done = __hip_atomic_compare_exchange_strong(word, &expected, __float_as_int(__int_as_float(seen) + v),
                                                           __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                           __HIP_MEMORY_SCOPE_WORKGROUP);
    if (!done) lds_add(addr, v);
}

// The work of one workgroup of mam_bwd_x_kernel: batch row n, its kc cells in `cells`.
template <int LAYOUT>
__device__ __forceinline__ void bwd_x_body(
    unsigned long long *cells, int n, const float *__restrict__ w, int64_t ldw, const float *__restrict__ grad,
    const int32_t *__restrict__ argmax, const int32_t *__restrict__ argmin,
    const float *__restrict__ w_sel, int64_t nm, float *__restrict__ x_grad, int K, int M, int kc, int planes,
    int span)
{
    // planes > 1 (the module's `splits`): argmax / argmin are [plane][N*M] arrays of absolute k, one pair
    // per K range, w_sel (if any) [plane][2][N*M]; every plane scatters the same grad
    __shared__ FixedQueue q;
    __shared__ uint32_t s_max;
    float *hist = reinterpret_cast<float *>(cells);   // kc cells; the fp32 fallback uses the same bytes
    const int tid = threadIdx.x;
    const float *g_row = grad + (int64_t)n * M;

    // one trip: four outputs per thread; all index loads, then all weight gathers, so that the gather
    // latencies overlap instead of adding up
    float g[4], wv1[4], wv2[4];
    int a1[4], a2[4];
    auto load_trip = [&](int pl, int mb, int k0, int kn) {
        const int32_t *amax_row = argmax + pl * nm + (int64_t)n * M;
        const int32_t *amin_row = argmin + pl * nm + (int64_t)n * M;
        const float *w_sel_pl = w_sel ? w_sel + pl * 2 * nm : nullptr;
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
            if (w_sel_pl) {
                const bool ok = m < M;
                wv1[u] = ok ? w_sel_pl[(int64_t)n * M + m] : 0.0f;
                wv2[u] = ok ? w_sel_pl[nm + (int64_t)n * M + m] : 0.0f;
            } else {
                wv1[u] = (unsigned)a1[u] < (unsigned)kn ? load_w<LAYOUT>(w, ldw, a1[u] + k0, m) : 0.0f;
                wv2[u] = (unsigned)a2[u] < (unsigned)kn ? load_w<LAYOUT>(w, ldw, a2[u] + k0, m) : 0.0f;
            }
        }
    };

    if (tid == 0) {
        s_max = 0u;
        q.count = 0;
    }
    __syncthreads();
    bool fixed = span >= 8;
    bool loaded = false;       // the first trip of chunk 0 is in the registers
    int e_lo = 1;
    if (fixed) {
        const int kn0 = K < kc ? K : kc;
        load_trip(0, tid, 0, kn0);
        loaded = true;
        uint32_t mx = 0u;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t b1 = magnitude_bits(wv1[u] * g[u]), b2 = magnitude_bits(wv2[u] * g[u]);
            mx = mx > b1 ? mx : b1;
            mx = mx > b2 ? mx : b2;
        }
        const bool whole_row = planes == 1 && M <= 4 * NT_X && K <= kc;
        fixed = make_window(workgroup_max(mx, &s_max), whole_row ? 0 : 4, span, e_lo);
    }
    for (int k0 = 0; k0 < K; k0 += kc) {
        const int kn = (K - k0) < kc ? (K - k0) : kc;
        for (int attempt = fixed ? 0 : 1; attempt < 2; ++attempt) {
            const bool fx = attempt == 0;
            if (fx) for (int i = tid; i < kn; i += NT_X) cells[i] = 0ull;
            else for (int i = tid; i < kn; i += NT_X) hist[i] = 0.0f;
            __syncthreads();
            for (int pl = 0; pl < planes; ++pl) {
                for (int mb = tid; mb < M; mb += 4 * NT_X) {
                    if (!loaded) load_trip(pl, mb, k0, kn);
                    loaded = false;
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if ((unsigned)a1[u] < (unsigned)kn) {
                            const float t = wv1[u] * g[u];
                            if (!fx) lds_add(&hist[a1[u]], t);
                            else if (fixed_add(&cells[a1[u]], t, e_lo, span)) queue_push(q, k0 + a1[u], t);
                        }
                        if ((unsigned)a2[u] < (unsigned)kn) {
                            const float t = wv2[u] * g[u];
                            if (!fx) lds_add(&hist[a2[u]], t);
                            else if (fixed_add(&cells[a2[u]], t, e_lo, span)) queue_push(q, k0 + a2[u], t);
                        }
                    }
                }
            }
            __syncthreads();
            const int queued = fx ? q.count : 0;
            __syncthreads();
            if (queued > QCAP) {       // the window was a bad guess: this chunk and the rest with fp32 atomics
                if (tid == 0) q.count = 0;
                fixed = false;
                continue;
            }
            float *dst = x_grad + (int64_t)n * K;
            if (queued > 0) {
                settle_queue<NT_X>(cells, kn, q, queued, e_lo, k0);
                const double *d = reinterpret_cast<const double *>(cells);
                for (int i = tid; i < kn; i += NT_X) dst[k0 + i] = (float)d[i];
                if (tid == 0) q.count = 0;
            } else if (fx) {
                for (int i = tid; i < kn; i += NT_X) dst[k0 + i] = cell_value(cells[i], e_lo);
            } else {
                for (int i = tid; i < kn; i += NT_X) dst[k0 + i] = hist[i];
            }
            __syncthreads();
            break;
        }
    }
}

template <int LAYOUT>
__global__ __launch_bounds__(NT_X) void mam_bwd_x_kernel(
    const float *__restrict__ w, int64_t ldw, const float *__restrict__ grad,
    const int32_t *__restrict__ argmax, const int32_t *__restrict__ argmin,
    const float *__restrict__ w_sel, int64_t nm, float *__restrict__ x_grad, int K, int M, int kc, int planes,
    int span)
{
    extern __shared__ unsigned long long cells[];
    bwd_x_body<LAYOUT>(cells, blockIdx.x, w, ldw, grad, argmax, argmin, w_sel, nm, x_grad, K, M, kc, planes, span);
}

// x_grad for large batches: a workgroup owns R = 2 .. 16 batch rows with their whole K cells in LDS,
// and the lanes of a wave are spread over those rows (64 / R lanes per row, 4 consecutive neurons
// each).  The selections of ONE batch row pile up on the few k where |x| is largest, so in
// mam_bwd_x_kernel most lanes of an instruction meet a contender; here only the 64 / R lanes of the
// same row can, and the loads of a wave are whole 64-byte (R = 16) to 512-byte (R = 2) pieces of R rows.
// Cells are 64-bit fixed point as above; the fp32 fallback settles a term by one compare-and-swap round
// where it can.
template <int LAYOUT>
__global__ __launch_bounds__(NT_W) void mam_bwd_x_rows_kernel(
    const float *__restrict__ w, int64_t ldw, const float *__restrict__ grad,
    const int32_t *__restrict__ argmax, const int32_t *__restrict__ argmin,
    const float *__restrict__ w_sel, int64_t nm, float *__restrict__ x_grad, int N, int K, int M, int log2r,
    int planes, int span)
{
    extern __shared__ unsigned long long cells[];   // [R][K]
    __shared__ FixedQueue q;
    __shared__ uint32_t s_max;
    float *hist = reinterpret_cast<float *>(cells);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int R = 1 << log2r;
    const int lpr = 64 >> log2r;                  // lanes per batch row
    const int r = lane / lpr, j = lane - r * lpr;
    const int n = blockIdx.x * R + r;
    const bool row_ok = n < N;
    const int m_step = (NT_W / 64) * lpr * 4;     // neurons of a row the workgroup covers per trip
    const int trips = (M + m_step - 1) / m_step;     // the same for every thread: lanes past M hold no item

    float4 g = make_float4(0.f, 0.f, 0.f, 0.f), s1 = g, s2 = g;
    int4 i1 = make_int4(-1, -1, -1, -1), i2 = i1;
// (a macro, not a lambda: captured by reference the five vectors end up in scratch memory)
#define MAM_LOAD_ITEM(pl, m)                                                                        \
    do {                                                                                            \
        if (row_ok && (m) < M) {                                                                    \
            const int64_t o_ = (int64_t)n * M + (m);                                                \
            g = *reinterpret_cast<const float4 *>(grad + o_);                                       \
            i1 = *reinterpret_cast<const int4 *>(argmax + (pl) * nm + o_);                          \
            i2 = *reinterpret_cast<const int4 *>(argmin + (pl) * nm + o_);                          \
            if (w_sel) {                                                                            \
                s1 = *reinterpret_cast<const float4 *>(w_sel + (pl) * 2 * nm + o_);                 \
                s2 = *reinterpret_cast<const float4 *>(w_sel + (pl) * 2 * nm + nm + o_);            \
            }                                                                                       \
        } else {                                                                                    \
            i1 = make_int4(-1, -1, -1, -1);                                                         \
            i2 = i1;                                                                                \
        }                                                                                           \
    } while (0)
    const int m_first = (wave * lpr + j) * 4;

    if (tid == 0) {
        s_max = 0u;
        q.count = 0;
    }
    __syncthreads();
    bool fixed = span >= 8;
    int e_lo = 1;
    bool have_first = false;      // the first item of plane 0 is in the registers (loaded for the window)
    if (fixed) {
        MAM_LOAD_ITEM(0, m_first);
        have_first = true;
        uint32_t mx = 0u;
        if (row_ok && m_first < M) {
            if (!w_sel) {     // no hand-over: the first trip's weights are gathered for the window as well
                const int k1[4] = {i1.x, i1.y, i1.z, i1.w}, k2[4] = {i2.x, i2.y, i2.z, i2.w};
                float w1[4], w2[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    w1[u] = (unsigned)k1[u] < (unsigned)K ? load_w<LAYOUT>(w, ldw, k1[u], m_first + u) : 0.0f;
                    w2[u] = (unsigned)k2[u] < (unsigned)K ? load_w<LAYOUT>(w, ldw, k2[u], m_first + u) : 0.0f;
                }
                s1 = make_float4(w1[0], w1[1], w1[2], w1[3]);
                s2 = make_float4(w2[0], w2[1], w2[2], w2[3]);
            }
            const float t[8] = {s1.x * g.x, s1.y * g.y, s1.z * g.z, s1.w * g.w, s2.x * g.x, s2.y * g.y, s2.z * g.z, s2.w * g.w};
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const uint32_t b = magnitude_bits(t[u]);
                mx = mx > b ? mx : b;
            }
        }
        fixed = make_window(workgroup_max(mx, &s_max), 4, span, e_lo);
    }
    const int rows = (N - blockIdx.x * R) < R ? (N - blockIdx.x * R) : R;
    float *dst = x_grad + (int64_t)blockIdx.x * R * K;
    for (int attempt = fixed ? 0 : 1; attempt < 2; ++attempt) {
        const bool fx = attempt == 0;
        if (fx) for (int i = tid; i < R * K; i += NT_W) cells[i] = 0ull;
        else for (int i = tid; i < R * K; i += NT_W) hist[i] = 0.0f;
        __syncthreads();
        for (int pl = 0; pl < planes; ++pl) {            // one (argmax, argmin) pair per K range
            int m = m_first;
            if (!have_first) MAM_LOAD_ITEM(pl, m);
            have_first = false;
            for (int t = 0; t < trips; ++t) {
                const float4 cg = g, c1 = s1, c2 = s2;
                const int4 a1 = i1, a2 = i2;
                const int mc = m;
                m += m_step;
                MAM_LOAD_ITEM(pl, m);         // the next trip's loads are in flight while this one is scattered
                const float gv[4] = {cg.x, cg.y, cg.z, cg.w};
                const int k1[4] = {a1.x, a1.y, a1.z, a1.w}, k2[4] = {a2.x, a2.y, a2.z, a2.w};
                float w1[4] = {c1.x, c1.y, c1.z, c1.w}, w2[4] = {c2.x, c2.y, c2.z, c2.w};
                if (!w_sel) {
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        w1[u] = (unsigned)k1[u] < (unsigned)K ? load_w<LAYOUT>(w, ldw, k1[u], mc + u) : 0.0f;
                        w2[u] = (unsigned)k2[u] < (unsigned)K ? load_w<LAYOUT>(w, ldw, k2[u], mc + u) : 0.0f;
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if ((unsigned)k1[u] < (unsigned)K) {
                        const float tv = w1[u] * gv[u];
                        if (!fx) lds_add_sparse(&hist[r * K + k1[u]], tv);
                        else if (fixed_add(&cells[r * K + k1[u]], tv, e_lo, span)) queue_push(q, r * K + k1[u], tv);
                    }
                    if ((unsigned)k2[u] < (unsigned)K) {
                        const float tv = w2[u] * gv[u];
                        if (!fx) lds_add_sparse(&hist[r * K + k2[u]], tv);
                        else if (fixed_add(&cells[r * K + k2[u]], tv, e_lo, span)) queue_push(q, r * K + k2[u], tv);
                    }
                }
            }
        }
        __syncthreads();
        const int queued = fx ? q.count : 0;
        __syncthreads();
        if (queued > QCAP) continue;      // the window was a bad guess: once more with fp32 atomics
        if (queued > 0) {
            settle_queue<NT_W>(cells, R * K, q, queued, e_lo, 0);
            const double *d = reinterpret_cast<const double *>(cells);
            for (int i = tid; i < rows * K; i += NT_W) dst[i] = (float)d[i];
        } else if (fx) {
            for (int i = tid; i < rows * K; i += NT_W) dst[i] = cell_value(cells[i], e_lo);
        } else {
            for (int i = tid; i < rows * K; i += NT_W) dst[i] = hist[i];
        }
        break;
    }
#undef MAM_LOAD_ITEM
}

// Scatter of one (batch row, 4 consecutive neurons) item into the slab histogram.  COUNT ((M,K) layout): the
// picks are also counted in `cnt`, a second LDS plane of the slab's shape whose words hold two 16-bit fields
// (low: argmax picks, high: argmin picks).
template <int LAYOUT, bool COUNT = false>
__device__ __forceinline__ void scatter_quad(float *hist, const float4 &g, const int4 &i1, const int4 &i2,
                                             const float (&x1)[4], const float (&x2)[4], int r0, int k0,
                                             int kn, int kc, int log2r, uint32_t *cnt = nullptr)
{
    const float gv[4] = {g.x, g.y, g.z, g.w};
    const int a1[4] = {i1.x - k0, i1.y - k0, i1.z - k0, i1.w - k0};
    const int a2[4] = {i2.x - k0, i2.y - k0, i2.z - k0, i2.w - k0};
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int r = r0 + u;
        if ((unsigned)a1[u] < (unsigned)kn) {
            lds_add_sparse(&hist[LAYOUT == MAM_W_MK ? r * kc + a1[u] : (a1[u] << log2r) + r], x1[u] * gv[u]);
            if (COUNT) atomicAdd(&cnt[r * kc + a1[u]], 1u);
        }
        if ((unsigned)a2[u] < (unsigned)kn) {
            lds_add_sparse(&hist[LAYOUT == MAM_W_MK ? r * kc + a2[u] : (a2[u] << log2r) + r], x2[u] * gv[u]);
            if (COUNT) atomicAdd(&cnt[r * kc + a2[u]], 0x10000u);
        }
    }
}

__device__ __forceinline__ void gather_quad(const float *xr, const int4 &i1, const int4 &i2, int k0, int kn,
                                            float (&x1)[4], float (&x2)[4])
{
    const int a1[4] = {i1.x - k0, i1.y - k0, i1.z - k0, i1.w - k0};
    const int a2[4] = {i2.x - k0, i2.y - k0, i2.z - k0, i2.w - k0};
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        x1[u] = (unsigned)a1[u] < (unsigned)kn ? xr[a1[u]] : 0.0f;
        x2[u] = (unsigned)a2[u] < (unsigned)kn ? xr[a2[u]] : 0.0f;
    }
}

// Stores the slab histogram to w_grad (NT threads).
template <int LAYOUT, int NT>
__device__ __forceinline__ void store_slab(const float *hist, float *__restrict__ w_grad, int tid, int m0,
                                           int k0, int rn, int kn, int kc, int log2r, int K, int M,
                                           int vec_out, bool accumulate)
{
    const int R = 1 << log2r;
    if (accumulate) {
        // the batch is split over several workgroups per slab: w_grad was cleared beforehand and
        // every workgroup adds its share (cells it never touched are skipped)
        for (int e = tid; e < (LAYOUT == MAM_W_MK ? rn * kn : (kn << log2r)); e += NT) {
            int r, kk;
            float v;
            if (LAYOUT == MAM_W_MK) { r = e / kn; kk = e - r * kn; v = hist[r * kc + kk]; }
            else { kk = e >> log2r; r = e & (R - 1); v = hist[e]; }
            if (v != 0.0f && r < rn) {
                float *cell = LAYOUT == MAM_W_MK ? w_grad + (int64_t)(m0 + r) * K + k0 + kk
                                                 : w_grad + (int64_t)(k0 + kk) * M + m0 + r;
                __hip_atomic_fetch_add(cell, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        return;
    }
    if (LAYOUT == MAM_W_MK) {
        if (vec_out) {  // K, k0 and kc are multiples of 4 and w_grad is 16-byte aligned
            const int q = kn >> 2;
            for (int e = tid; e < rn * q; e += NT) {
                const int r = e / q, c4 = e - r * q;
                *reinterpret_cast<float4 *>(w_grad + (int64_t)(m0 + r) * K + k0 + c4 * 4) =
                    *reinterpret_cast<const float4 *>(&hist[r * kc + c4 * 4]);
            }
        } else {
            for (int e = tid; e < rn * kn; e += NT) {
                const int r = e / kn, kk = e - r * kn;
                w_grad[(int64_t)(m0 + r) * K + k0 + kk] = hist[r * kc + kk];
            }
        }
    } else {
        for (int e = tid; e < (kn << log2r); e += NT) {
            const int kk = e >> log2r, r = e & (R - 1);
            if (r < rn) w_grad[(int64_t)(k0 + kk) * M + m0 + r] = hist[e];
        }
    }
}

// Fast path (M a multiple of 4, 16-byte aligned grad / argmax / argmin).  A thread's unit of work
// is one batch row x 4 consecutive neurons: three 16-byte loads, eight x gathers from one row,
// eight LDS adds.  A workgroup walks `tiles_per_wg` consecutive slabs and software-pipelines them:
// the index loads of the next slab are issued before the current slab is streamed out, and the x
// gathers are in flight while the histogram is cleared, so the scatter phase's latency chain
// (index load -> gather -> LDS add) overlaps the store phase instead of alternating with it.
// The work of one workgroup (NT threads) of mam_bwd_w_vec_kernel: workgroup `bx` of `nbx` along the slabs,
// k chunk `by`, share `bz` of `nbz` of the batch rows.
// COUNT: the workgroup also owns the slab's selection counters (hits mode, mam_selcount.hip): the picks it
// scatters are counted in a second LDS plane behind the histogram and added to max_count / min_count when the
// slab is streamed out -- the index arrays are read once for both, and one launch serves both.
template <int LAYOUT, int NT, bool COUNT = false>
__device__ __forceinline__ void bwd_w_vec_body(
    float *hist, int bx, int nbx, int by, int bz, int nbz,
    const float *__restrict__ x, int64_t ldx, const float *__restrict__ grad,
    const int32_t *__restrict__ argmax, const int32_t *__restrict__ argmin,
    const float *__restrict__ x_sel, int64_t nm, float *__restrict__ w_grad, int N, int K, int M, int log2r,
    int kc, int vec_out, int mtiles, int tiles_per_wg, int rows_per_split, int planes, int range_len,
    int32_t *__restrict__ max_count = nullptr, int32_t *__restrict__ min_count = nullptr)
{
    uint32_t *cnt = reinterpret_cast<uint32_t *>(hist) + ((size_t)kc << log2r);
    const int tid = threadIdx.x;
    const int R = 1 << log2r;
    const int qpr = R >> 2;
    // bz: which share of the batch rows (one share = the whole batch unless the host split it)
    const int n_begin = bz * rows_per_split;
    const int n_rows = (N - n_begin) < rows_per_split ? (N - n_begin) : rows_per_split;
    const bool accumulate = nbz > 1;
    const int k0 = by * kc;
    const int kn = (K - k0) < kc ? (K - k0) : kc;
    // planes > 1 (the module's `splits`): one (argmax, argmin) pair of absolute k per K range of
    // `range_len`, [plane][N*M]; a slab takes the planes whose ranges meet its k chunk
    const int pl_lo = planes > 1 ? k0 / range_len : 0;
    int pl_hi = planes > 1 ? (k0 + kn - 1) / range_len : 0;
    pl_hi = pl_hi < planes - 1 ? pl_hi : planes - 1;
    const int npl = pl_hi - pl_lo + 1;
    const int64_t per_plane = (int64_t)n_rows * qpr;
    const int64_t items = per_plane * npl;
    const int first = xcd_remap(bx, nbx) * tiles_per_wg;

    // this thread's first item of a slab: plane pl_lo + pf, row n_first, neurons m0 + r_first .. +3
    const int pf = npl > 1 ? (int)(tid / per_plane) : 0;
    const int rem_first = npl > 1 ? (int)(tid - pf * per_plane) : tid;
    const int n_first = n_begin + rem_first / qpr, r_first = (rem_first % qpr) * 4;
    const int64_t po_first = (int64_t)(pl_lo + pf) * nm;
    float4 g = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 s1 = g, s2 = g;      // selected inputs handed over by the forward, if any
    int4 i1 = make_int4(-1, -1, -1, -1), i2 = make_int4(-1, -1, -1, -1);
    bool have = false;
    auto load_first = [&](int m0) {
        have = tid < items && m0 + r_first < M;
        if (have) {
            const int64_t o = (int64_t)n_first * M + m0 + r_first;
            g = *reinterpret_cast<const float4 *>(grad + o);
            i1 = *reinterpret_cast<const int4 *>(argmax + po_first + o);
            i2 = *reinterpret_cast<const int4 *>(argmin + po_first + o);
            if (x_sel) {
                s1 = *reinterpret_cast<const float4 *>(x_sel + 2 * po_first + o);
                s2 = *reinterpret_cast<const float4 *>(x_sel + 2 * po_first + nm + o);
            }
        }
    };
    if (first < mtiles) load_first(first * R);

    for (int t = 0; t < tiles_per_wg; ++t) {
        const int mt = first + t;
        if (mt >= mtiles) break;
        const int m0 = mt * R;
        const int rn = (M - m0) < R ? (M - m0) : R;
        float x1[4] = {s1.x, s1.y, s1.z, s1.w}, x2[4] = {s2.x, s2.y, s2.z, s2.w};
        if (have && !x_sel) gather_quad(x + (int64_t)n_first * ldx + k0, i1, i2, k0, kn, x1, x2);
        for (int i = tid * 4; i < (COUNT ? 2 : 1) * R * kc; i += NT * 4)
            *reinterpret_cast<float4 *>(&hist[i]) = make_float4(0.f, 0.f, 0.f, 0.f);
        __syncthreads();
        if (have) scatter_quad<LAYOUT, COUNT>(hist, g, i1, i2, x1, x2, r_first, k0, kn, kc, log2r, cnt);
        for (int64_t it = tid + NT; it < items; it += NT) {
            const int pl = npl > 1 ? (int)(it / per_plane) : 0;
            const int64_t rem = npl > 1 ? it - pl * per_plane : it;
            const int n = n_begin + (int)(rem / qpr), r0 = (int)(rem % qpr) * 4;
            if (m0 + r0 >= M) continue;
            const int64_t o = (int64_t)n * M + m0 + r0;
            const int64_t po = (int64_t)(pl_lo + pl) * nm;
            const float4 gg = *reinterpret_cast<const float4 *>(grad + o);
            const int4 j1 = *reinterpret_cast<const int4 *>(argmax + po + o);
            const int4 j2 = *reinterpret_cast<const int4 *>(argmin + po + o);
            float y1[4], y2[4];
            if (x_sel) {
                const float4 t1 = *reinterpret_cast<const float4 *>(x_sel + 2 * po + o);
                const float4 t2 = *reinterpret_cast<const float4 *>(x_sel + 2 * po + nm + o);
                y1[0] = t1.x; y1[1] = t1.y; y1[2] = t1.z; y1[3] = t1.w;
                y2[0] = t2.x; y2[1] = t2.y; y2[2] = t2.z; y2[3] = t2.w;
            } else {
                gather_quad(x + (int64_t)n * ldx + k0, j1, j2, k0, kn, y1, y2);
            }
            scatter_quad<LAYOUT, COUNT>(hist, gg, j1, j2, y1, y2, r0, k0, kn, kc, log2r, cnt);
        }
        __syncthreads();
        if (t + 1 < tiles_per_wg && mt + 1 < mtiles) load_first(m0 + R);
        // the counters first: their read-modify-write is the longer chain, the plain stores of w_grad follow it
        // (measured at 256 x 4096 x 4096, x_grad + this kernel: 58.7 us this way round, 61.2 the other)
        if (COUNT)
            selcount::stream_counts<MAM_COUNT_HITS, NT, 2>(cnt, max_count, min_count, tid, m0, k0, rn, kn, kc, K);
        store_slab<LAYOUT, NT>(hist, w_grad, tid, m0, k0, rn, kn, kc, log2r, K, M, vec_out, accumulate);
        __syncthreads();
    }
}

template <int LAYOUT>
__global__ __launch_bounds__(NT_W) void mam_bwd_w_vec_kernel(
    const float *__restrict__ x, int64_t ldx, const float *__restrict__ grad,
    const int32_t *__restrict__ argmax, const int32_t *__restrict__ argmin,
    const float *__restrict__ x_sel, int64_t nm, float *__restrict__ w_grad, int N, int K, int M, int log2r,
    int kc, int vec_out, int mtiles, int tiles_per_wg, int rows_per_split, int planes, int range_len)
{
    extern __shared__ float hist[];
    bwd_w_vec_body<LAYOUT, NT_W>(hist, blockIdx.x, gridDim.x, blockIdx.y, blockIdx.z, gridDim.z, x, ldx, grad, argmax,
                                 argmin, x_sel, nm, w_grad, N, K, M, log2r, kc, vec_out, mtiles, tiles_per_wg,
                                 rows_per_split, planes, range_len);
}

// w_grad and the selection counts (hits) of the same slabs in one launch.
constexpr int NT_C = 1024;   // both LDS planes of a slab are 128 KiB: one workgroup per CU, so twice the threads
__global__ __launch_bounds__(NT_C) void mam_bwd_w_count_kernel(
    const float *__restrict__ x, int64_t ldx, const float *__restrict__ grad,
    const int32_t *__restrict__ argmax, const int32_t *__restrict__ argmin,
    const float *__restrict__ x_sel, int64_t nm, float *__restrict__ w_grad, int32_t *__restrict__ max_count,
    int32_t *__restrict__ min_count, int N, int K, int M, int log2r, int kc, int mtiles, int tiles_per_wg)
{
    extern __shared__ float hist[];
    bwd_w_vec_body<MAM_W_MK, NT_C, true>(hist, blockIdx.x, gridDim.x, blockIdx.y, 0, 1, x, ldx, grad, argmax, argmin,
                                         x_sel, nm, w_grad, N, K, M, log2r, kc, 1, mtiles, tiles_per_wg, N, 1, K,
                                         max_count, min_count);
}

// w_grad as the exact sum of its fp32 terms, rounded once (option MAM_OPT_BACKWARD_EXACT; (M,K) weights, 16-byte
// aligned operands).  A workgroup owns 4 neurons x kc columns in 64-bit fixed-point cells (mam_fixed.h): integer
// adds are exact and commute, so w_grad does not depend on the order in which the lanes arrive and equals the
// correctly rounded sum.  An 8-byte cell halves the columns a 64 KiB slab holds, so a neuron quad with K = 4096
// is covered by two workgroups that each scan the quad's items: 45 against 17 us at 256 x 4096 x 4096 (1.7 to
// 1.8 times the fp32 kernel's time at batch 12608), which is why this is an option and not the default.  Terms outside the window (more than ~2^25 below the largest, inf,
// nan) go through the queue and are added in fp64 before the one rounding; if more than QCAP terms of a
// workgroup fall outside, that workgroup falls back to fp32 LDS atomics (and its cells are then sums in arrival
// order, within the documented tolerance).
constexpr int NT_E = 1024;
__global__ __launch_bounds__(NT_E) void mam_bwd_w_exact_kernel(
    const float *__restrict__ x, int64_t ldx, const float *__restrict__ grad,
    const int32_t *__restrict__ argmax, const int32_t *__restrict__ argmin,
    const float *__restrict__ x_sel, int64_t nm, float *__restrict__ w_grad, int N, int K, int M, int kc, int span)
{
    using namespace fixedpoint;
    extern __shared__ unsigned long long exact_cells[];      // [4][kc]
    __shared__ FixedQueue q;
    __shared__ uint32_t s_max;
    float *hist = reinterpret_cast<float *>(exact_cells);
    const int tid = threadIdx.x;
    const int m0 = xcd_remap(blockIdx.x, gridDim.x) * 4;
    const int k0 = blockIdx.y * kc;
    const int kn = (K - k0) < kc ? (K - k0) : kc;
    const int ncells = 4 * kc;

    // one item: batch row n, neurons m0 .. m0 + 3; cell index per term, -1 = outside this k chunk
    float t1[4], t2[4];
    int c1[4], c2[4];
    auto load_item = [&](int n) {
        const int64_t o = (int64_t)n * M + m0;
        const float4 g = *reinterpret_cast<const float4 *>(grad + o);
        const int4 i1 = *reinterpret_cast<const int4 *>(argmax + o);
        const int4 i2 = *reinterpret_cast<const int4 *>(argmin + o);
        const float gv[4] = {g.x, g.y, g.z, g.w};
        const int a1[4] = {i1.x - k0, i1.y - k0, i1.z - k0, i1.w - k0};
        const int a2[4] = {i2.x - k0, i2.y - k0, i2.z - k0, i2.w - k0};
        float x1[4], x2[4];
        if (x_sel) {
            const float4 s1 = *reinterpret_cast<const float4 *>(x_sel + o);
            const float4 s2 = *reinterpret_cast<const float4 *>(x_sel + nm + o);
            x1[0] = s1.x; x1[1] = s1.y; x1[2] = s1.z; x1[3] = s1.w;
            x2[0] = s2.x; x2[1] = s2.y; x2[2] = s2.z; x2[3] = s2.w;
        } else {
            const float *xr = x + (int64_t)n * ldx + k0;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                x1[u] = (unsigned)a1[u] < (unsigned)kn ? xr[a1[u]] : 0.0f;
                x2[u] = (unsigned)a2[u] < (unsigned)kn ? xr[a2[u]] : 0.0f;
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            c1[u] = (unsigned)a1[u] < (unsigned)kn ? u * kc + a1[u] : -1;
            c2[u] = (unsigned)a2[u] < (unsigned)kn ? u * kc + a2[u] : -1;
            t1[u] = x1[u] * gv[u];
            t2[u] = x2[u] * gv[u];
        }
    };

    if (tid == 0) {
        s_max = 0u;
        q.count = 0;
    }
    __syncthreads();
    bool fixed = span >= 8;
    bool loaded = false;
    int e_lo = 1;
    if (fixed) {
        uint32_t mx = 0u;
        if (tid < N) {
            load_item(tid);
            loaded = true;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (c1[u] >= 0) { const uint32_t b = magnitude_bits(t1[u]); mx = mx > b ? mx : b; }
                if (c2[u] >= 0) { const uint32_t b = magnitude_bits(t2[u]); mx = mx > b ? mx : b; }
            }
        }
        fixed = make_window(workgroup_max(mx, &s_max), N <= NT_E ? 0 : 4, span, e_lo);
    }
    for (int attempt = fixed ? 0 : 1; attempt < 2; ++attempt) {
        const bool fx = attempt == 0;
        if (fx) for (int i = tid; i < ncells; i += NT_E) exact_cells[i] = 0ull;
        else for (int i = tid; i < ncells; i += NT_E) hist[i] = 0.0f;
        __syncthreads();
        for (int n = tid; n < N; n += NT_E) {
            if (!loaded) load_item(n);
            loaded = false;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (c1[u] >= 0) {
                    if (!fx) lds_add_sparse(&hist[c1[u]], t1[u]);
                    else if (fixed_add(&exact_cells[c1[u]], t1[u], e_lo, span)) queue_push(q, c1[u], t1[u]);
                }
                if (c2[u] >= 0) {
                    if (!fx) lds_add_sparse(&hist[c2[u]], t2[u]);
                    else if (fixed_add(&exact_cells[c2[u]], t2[u], e_lo, span)) queue_push(q, c2[u], t2[u]);
                }
            }
        }
        __syncthreads();
        const int queued = fx ? q.count : 0;
        __syncthreads();
        if (queued > QCAP) {
            if (tid == 0) q.count = 0;
            continue;      // the window was a bad guess: once more with fp32 atomics
        }
        if (queued > 0) settle_queue<NT_E>(exact_cells, ncells, q, queued, e_lo, 0);
        const double *d = reinterpret_cast<const double *>(exact_cells);
        const int q4 = kn >> 2;
        for (int e = tid; e < 4 * q4; e += NT_E) {
            const int r = e / q4, c4 = (e - r * q4) * 4;
            if (m0 + r >= M) continue;
            float4 v;
            const int b = r * kc + c4;
            if (queued > 0) v = make_float4((float)d[b], (float)d[b + 1], (float)d[b + 2], (float)d[b + 3]);
            else if (fx) v = make_float4(cell_value(exact_cells[b], e_lo), cell_value(exact_cells[b + 1], e_lo),
                                         cell_value(exact_cells[b + 2], e_lo), cell_value(exact_cells[b + 3], e_lo));
            else v = make_float4(hist[b], hist[b + 1], hist[b + 2], hist[b + 3]);
            *reinterpret_cast<float4 *>(w_grad + (int64_t)(m0 + r) * K + k0 + c4) = v;
        }
        break;
    }
}

// Both gradients in one launch, for the shapes where one launch of each kind fills the chip once: the first
// `x_wgs` workgroups are those of mam_bwd_x_kernel (one batch row each), the rest those of
// mam_bwd_w_vec_kernel with NT_X threads.  Workgroups are dispatched in index order, so every x_grad workgroup
// is resident before the first w_grad one: x_grad is bound by LDS atomics, w_grad by its stream to HBM, and
// side by side they take about as long as w_grad alone.  (Dealt out alternately, the long-running w_grad
// workgroups end up holding every slot.)
struct BothParams {
    const float *x, *w, *grad, *w_sel, *x_sel;
    const int32_t *argmax, *argmin;
    float *x_grad, *w_grad;
    int64_t ldx, ldw, nm;
    int N, K, M, planes, range_len, span, kc_x;
    int log2r, kc_w, vec_out, mtiles, tiles_per_wg, x_wgs;
};
template <int LAYOUT>
__global__ __launch_bounds__(NT_X) void mam_bwd_both_kernel(const BothParams p)
{
    extern __shared__ unsigned long long both_lds[];
    if ((int)blockIdx.x < p.x_wgs) {
        bwd_x_body<LAYOUT>(both_lds, blockIdx.x, p.w, p.ldw, p.grad, p.argmax, p.argmin, p.w_sel, p.nm, p.x_grad, p.K,
                           p.M, p.kc_x, p.planes, p.span);
    } else {
        bwd_w_vec_body<LAYOUT, NT_X>(reinterpret_cast<float *>(both_lds), blockIdx.x - p.x_wgs, gridDim.x - p.x_wgs, 0,
                                     0, 1, p.x, p.ldx, p.grad, p.argmax, p.argmin, p.x_sel, p.nm, p.w_grad, p.N, p.K,
                                     p.M, p.log2r, p.kc_w, p.vec_out, p.mtiles, p.tiles_per_wg, p.N, p.planes,
                                     p.range_len);
    }
}

// Generic path: any M, any alignment; one (batch row, neuron) pair per thread and trip.
template <int LAYOUT>
__global__ __launch_bounds__(NT_W) void mam_bwd_w_kernel(
    const float *__restrict__ x, int64_t ldx, const float *__restrict__ grad,
    const int32_t *__restrict__ argmax, const int32_t *__restrict__ argmin,
    const float *__restrict__ x_sel, int64_t nm, float *__restrict__ w_grad, int N, int K, int M, int log2r,
    int kc, int vec_out, int planes, int range_len)
{
    extern __shared__ float hist[];
    const int tid = threadIdx.x;
    const int R = 1 << log2r;
    const int mt = xcd_remap(blockIdx.x, gridDim.x);
    const int m0 = mt * R;
    const int k0 = blockIdx.y * kc;
    const int rn = (M - m0) < R ? (M - m0) : R;
    const int kn = (K - k0) < kc ? (K - k0) : kc;

    for (int i = tid * 4; i < R * kc; i += NT_W * 4)
        *reinterpret_cast<float4 *>(&hist[i]) = make_float4(0.f, 0.f, 0.f, 0.f);
    __syncthreads();
    const int64_t pairs = (int64_t)N << log2r;
    // one (argmax, argmin) pair of absolute k per K range; only the planes whose ranges meet this k chunk
    const int pl_lo = planes > 1 ? k0 / range_len : 0;
    int pl_hi = planes > 1 ? (k0 + kn - 1) / range_len : 0;
    pl_hi = pl_hi < planes - 1 ? pl_hi : planes - 1;
    for (int pl = pl_lo; pl <= pl_hi; ++pl) {
        const int32_t *amax_pl = argmax + pl * nm, *amin_pl = argmin + pl * nm;
        const float *x_sel_pl = x_sel ? x_sel + pl * 2 * nm : nullptr;
        for (int64_t pi = tid; pi < pairs; pi += NT_W) {
            const int n = (int)(pi >> log2r), r = (int)(pi & (R - 1));
            if (r >= rn) continue;
            const int64_t o = (int64_t)n * M + m0 + r;
            const float g = grad[o];
            const int a1 = amax_pl[o] - k0, a2 = amin_pl[o] - k0;
            const float *xr = x + (int64_t)n * ldx + k0;
            if ((unsigned)a1 < (unsigned)kn)
                lds_add_sparse(&hist[LAYOUT == MAM_W_MK ? r * kc + a1 : (a1 << log2r) + r],
                               (x_sel_pl ? x_sel_pl[o] : xr[a1]) * g);
            if ((unsigned)a2 < (unsigned)kn)
                lds_add_sparse(&hist[LAYOUT == MAM_W_MK ? r * kc + a2 : (a2 << log2r) + r],
                               (x_sel_pl ? x_sel_pl[nm + o] : xr[a2]) * g);
        }
    }
    __syncthreads();
    store_slab<LAYOUT, NT_W>(hist, w_grad, tid, m0, k0, rn, kn, kc, log2r, K, M, vec_out, false);
}

// LDS a workgroup may use for a histogram, in floats, per device.  gfx950 has 160 KiB per CU; above
// 64 KiB the kernel attribute has to be raised first, once per device, which the device's set-up does
// for every kernel of this file.
static int g_lds_floats[kMaxDevices];
#ifndef MAM_BWD_ROWS_LDS
#define MAM_BWD_ROWS_LDS (64 * 1024)
#endif
constexpr int64_t kRowsLdsBytes = MAM_BWD_ROWS_LDS;

static int setup_device(int dev)
{
    constexpr int kWant = 128 * 1024;
    const void *kernels[] = {
        (const void *)mam_bwd_x_rows_kernel<MAM_W_MK>, (const void *)mam_bwd_x_rows_kernel<MAM_W_KM>,
        (const void *)mam_bwd_x_kernel<MAM_W_MK>,      (const void *)mam_bwd_x_kernel<MAM_W_KM>,
        (const void *)mam_bwd_w_kernel<MAM_W_MK>,      (const void *)mam_bwd_w_kernel<MAM_W_KM>,
        (const void *)mam_bwd_w_vec_kernel<MAM_W_MK>,  (const void *)mam_bwd_w_vec_kernel<MAM_W_KM>,
        (const void *)mam_bwd_both_kernel<MAM_W_MK>,   (const void *)mam_bwd_w_count_kernel,
    };
    bool all = true;
    for (const void *k : kernels)
        if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kWant) != hipSuccess) {
            (void)hipGetLastError();
            all = false;
        }
    g_lds_floats[dev] = (all ? kWant : 64 * 1024) / 4;
    return MAM_OK;
}
static DeviceHookRegistration g_registration(setup_device);

template <int LAYOUT>
static int launch_layout(const float *x, int64_t ldx, const float *w, int64_t ldw, const float *grad,
                         const int32_t *argmax, const int32_t *argmin, const float *w_sel, const float *x_sel,
                         float *x_grad, float *w_grad, int64_t N, int64_t K, int64_t M, hipStream_t st,
                         int planes = 1, int range_len = 0)
{
    int rc = MAM_OK;
    if (planes <= 1) range_len = (int)K;
    const int dev = ensure_device(st);
    if (dev < 0) return dev;
    const int lds_cap = g_lds_floats[dev];
    const int cus = num_cus();
    // 64-bit fixed-point cells: room for 2 * M * planes terms of 24 + span - 1 bits each, and one bit to spare
    const int span = window_span(2 * M * planes);
    const bool x_rows = N >= 2048 && K * 16 <= ((int64_t)lds_cap * 4 - 8192 < 64 * 1024 ? (int64_t)lds_cap * 4 - 8192 : 64 * 1024) && (M % 4 == 0) && ((uintptr_t)grad % 16 == 0) &&
                        ((uintptr_t)argmax % 16 == 0) && ((uintptr_t)argmin % 16 == 0) &&
                        ((uintptr_t)w_sel % 16 == 0);
    if (x_grad && x_rows) {
        // as many rows per workgroup (2 to 16) as fit 64 KiB of LDS in 8-byte cells
        // (the queue and the window's scratch are static LDS on top of the cells: 8 KiB kept free for them)
        const int64_t rows_budget = kRowsLdsBytes < (int64_t)lds_cap * 4 - 8192 ? kRowsLdsBytes : (int64_t)lds_cap * 4 - 8192;
        int log2r = 1;
        while (log2r < 4 && ((int64_t)2 << log2r) * K * 8 <= rows_budget) ++log2r;
        const int R = 1 << log2r;
        hipLaunchKernelGGL((mam_bwd_x_rows_kernel<LAYOUT>), dim3((unsigned)ceil_div(N, R)), dim3(NT_W),
                           (size_t)R * K * 8, st, w, ldw, grad, argmax, argmin, w_sel, N * M, x_grad,
                           (int)N, (int)K, (int)M, log2r, planes, span);
        rc = check_launch("mam_bwd_x_rows_kernel");
        if (rc != MAM_OK) return rc;
    } else if (x_grad) {
        const int cells_cap = (lds_cap - 2048) / 2;     // 8-byte cells, 8 KiB kept free for the static LDS
        const int kc = (int)(K < cells_cap ? K : cells_cap);
        hipLaunchKernelGGL((mam_bwd_x_kernel<LAYOUT>), dim3((unsigned)N), dim3(NT_X),
                           (size_t)kc * 8, st, w, ldw, grad, argmax, argmin, w_sel, N * M,
                           x_grad, (int)K, (int)M, kc, planes, span);
        rc = check_launch("mam_bwd_x_kernel");
        if (rc != MAM_OK) return rc;
    }
    if (w_grad) {
        // (M,K): 4 whole-K rows in 64 KiB, so two workgroups share a CU.  (K,M): 32 columns x
        // 1024 k in 128 KiB.
        const int vec_in = (M % 4 == 0) && ((uintptr_t)grad % 16 == 0) && ((uintptr_t)argmax % 16 == 0) &&
                           ((uintptr_t)argmin % 16 == 0) && ((uintptr_t)x_sel % 16 == 0) && (N * M % 4 == 0);
        int log2r = LAYOUT == MAM_W_MK ? 2 : 5;
        // Large batches: a thread reads 16 bytes of a batch row per array, so a slab of 4 neurons uses
        // a quarter of every 64-byte sector it touches.  When K is small enough, 16 neurons (whole
        // sectors) share a slab, and the batch is split over several workgroups per slab to keep the
        // chip filled; they add their shares to the cleared w_grad.
        if (LAYOUT == MAM_W_MK && vec_in && planes == 1 && K % 4 == 0 && (uintptr_t)w_grad % 16 == 0 &&
            option(MAM_OPT_BACKWARD_EXACT) == MAM_BACKWARD_EXACT_ON) {
            // 4 neurons x kc columns of 8-byte cells in 64 KiB
            int kce = 2048;
            if (K < kce) kce = (int)K;
            const int64_t kt = ceil_div(K, kce);
            if (kt <= 65535) {
                hipLaunchKernelGGL(mam_bwd_w_exact_kernel, dim3((unsigned)(M / 4), (unsigned)kt), dim3(NT_E),
                                   (size_t)4 * kce * 8, st, x, ldx, grad, argmax, argmin, x_sel, N * M, w_grad, (int)N,
                                   (int)K, (int)M, kce, window_span(2 * N));
                return check_launch("mam_bwd_w_exact_kernel");
            }
        }
        const bool large_batch = LAYOUT == MAM_W_MK && vec_in && N >= 2048;
        if (large_batch)
            while (log2r < 4 && ((int64_t)2 << log2r) * ((K + 3) / 4 * 4) * 4 <= 64 * 1024) ++log2r;
        const int R = 1 << log2r;
        const int budget = LAYOUT == MAM_W_MK ? (R * 4096 < lds_cap ? R * 4096 : lds_cap) : lds_cap;
        int kc = budget / R;
        if (K < kc) kc = (int)((K + 3) / 4 * 4);
        const int64_t mtiles = ceil_div(M, R), ktiles = ceil_div(K, kc);
        if (ktiles > 65535) return fail(MAM_ERR_UNSUPPORTED, "K too large for the w_grad grid");
        const int vec_out = (K % 4 == 0) && ((uintptr_t)w_grad % 16 == 0);
        if (vec_in) {
            // slabs per workgroup: enough workgroups for two per CU, the rest goes into pipelining
            int tpw = (int)(mtiles * ktiles / (2 * cus));
            if (tpw < 1) tpw = 1;
            if (tpw > 8) tpw = 8;
            // shares of the batch per slab: two rounds of as many workgroups as fit the chip (LDS, threads)
            int64_t shares = 1;
            if (large_batch) {
                int64_t per_cu = (160 * 1024) / ((int64_t)R * kc * 4);
                if (per_cu > 2048 / NT_W) per_cu = 2048 / NT_W;
                if (per_cu < 1) per_cu = 1;
                shares = (2 * per_cu * cus + mtiles * ktiles / 2) / (mtiles * ktiles);
                // a share adds a whole slab to w_grad with atomics: worth it only against >= K rows of work
                if (shares > N / (K > 512 ? K : 512)) shares = N / (K > 512 ? K : 512);
                if (shares > 65535) shares = 65535;
                if (shares < 1) shares = 1;
            }
            const int64_t rows_per_share = ceil_div(N, shares);
            shares = ceil_div(N, rows_per_share);
            if (shares > 1) {
                rc = fill_zero(w_grad, M * K, st);
                if (rc != MAM_OK) return rc;
            }
            hipLaunchKernelGGL((mam_bwd_w_vec_kernel<LAYOUT>),
                               dim3((unsigned)ceil_div(mtiles, tpw), (unsigned)ktiles, (unsigned)shares), dim3(NT_W),
                               (size_t)R * kc * sizeof(float), st, x, ldx, grad, argmax, argmin, x_sel, N * M,
                               w_grad, (int)N, (int)K, (int)M, log2r, kc, vec_out, (int)mtiles, tpw,
                               (int)rows_per_share, planes, range_len);
        } else {
            hipLaunchKernelGGL((mam_bwd_w_kernel<LAYOUT>), dim3((unsigned)mtiles, (unsigned)ktiles),
                               dim3(NT_W), (size_t)R * kc * sizeof(float), st, x, ldx, grad, argmax,
                               argmin, x_sel, N * M, w_grad, (int)N, (int)K, (int)M, log2r, kc, vec_out, planes,
                               range_len);
        }
        rc = check_launch("mam_bwd_w_kernel");
    }
    return rc;
}

// Both gradients in one launch (mam_bwd_both_kernel) where the shape allows it: (M,K) weights, the 16-byte
// paths of both kernels, a batch small enough that the x_grad workgroups (one per batch row) are all resident
// at once, K in one chunk of either kernel -- and, unless the option forces it, at most 2^16 outputs.
// Returns MAM_OK after launching, 1 when the shape is not served.
static int launch_both(const float *x, int64_t ldx, const float *w, int64_t ldw, const float *grad,
                       const int32_t *argmax, const int32_t *argmin, const float *w_sel, const float *x_sel,
                       float *x_grad, float *w_grad, int64_t N, int64_t K, int64_t M, hipStream_t st, int planes,
                       int range_len, bool auto_mode)
{
    if (planes <= 1) range_len = (int)K;
    const int dev = ensure_device(st);
    if (dev < 0) return dev;
    const int cus = num_cus();
    const bool vec_in = (M % 4 == 0) && (N * M % 4 == 0) && ((uintptr_t)grad % 16 == 0) &&
                        ((uintptr_t)argmax % 16 == 0) && ((uintptr_t)argmin % 16 == 0) &&
                        ((uintptr_t)x_sel % 16 == 0);
    constexpr int64_t kLds = 64 * 1024;               // dynamic LDS of the launch: two workgroups per CU
    const int log2r = 2, R = 4;
    const int64_t kc_w = (K + 3) / 4 * 4;
    // Worth it only where the launches themselves are what a call costs (config 1: 10 -> 7 us).  At
    // 256 x 4096 x 4096 one launch took 35.6 us against 29.2 us for two, with one slab or two per w_grad
    // workgroup: the x_grad workgroups hold one of the two slots of every CU for as long as they run.
    const bool small = (auto_mode ? N * M <= (1 << 16) : true);
    if (!small || !vec_in || N >= 2048 || N > 2 * cus || K * 8 > kLds || R * kc_w * 4 > kLds ||
        g_lds_floats[dev] * 4 < (int)kLds + 8192)
        return 1;
    const int64_t mtiles = ceil_div(M, R);
    int tpw = (int)(mtiles / (2 * cus));
    if (tpw < 1) tpw = 1;
    if (tpw > 8) tpw = 8;
    const int64_t w_wgs = ceil_div(mtiles, tpw);
    if (N + w_wgs > INT32_MAX) return 1;
    BothParams p;
    p.x = x; p.w = w; p.grad = grad; p.w_sel = w_sel; p.x_sel = x_sel;
    p.argmax = argmax; p.argmin = argmin; p.x_grad = x_grad; p.w_grad = w_grad;
    p.ldx = ldx; p.ldw = ldw; p.nm = N * M;
    p.N = (int)N; p.K = (int)K; p.M = (int)M; p.planes = planes; p.range_len = range_len;
    p.span = window_span(2 * M * planes); p.kc_x = (int)K;
    p.log2r = log2r; p.kc_w = (int)kc_w; p.vec_out = (K % 4 == 0) && ((uintptr_t)w_grad % 16 == 0);
    p.mtiles = (int)mtiles; p.tiles_per_wg = tpw; p.x_wgs = (int)N;
    const size_t lds = (size_t)(K * 8 > R * kc_w * 4 ? K * 8 : R * kc_w * 4);
    hipLaunchKernelGGL((mam_bwd_both_kernel<MAM_W_MK>), dim3((unsigned)(N + w_wgs)), dim3(NT_X), lds, st, p);
    return check_launch("mam_bwd_both_kernel");
}

// w_grad and the hits-mode selection counts in one launch (mam_bwd_w_count_kernel) where the shape allows it:
// (M,K) weights, the 16-byte paths, a batch below the large-batch shapes and below 32768 rows (16-bit count
// fields), both LDS planes of a slab within the device's limit.  Returns 1 when the shape is not served.
static int launch_w_count(const float *x, int64_t ldx, const float *grad, const int32_t *argmax,
                          const int32_t *argmin, const float *x_sel, float *w_grad, int32_t *max_count,
                          int32_t *min_count, int64_t N, int64_t K, int64_t M, hipStream_t st)
{
    const int dev = ensure_device(st);
    if (dev < 0) return dev;
    const bool vec = (M % 4 == 0) && (N * M % 4 == 0) && (K % 4 == 0) && ((uintptr_t)grad % 16 == 0) &&
                     ((uintptr_t)argmax % 16 == 0) && ((uintptr_t)argmin % 16 == 0) && ((uintptr_t)x_sel % 16 == 0) &&
                     ((uintptr_t)w_grad % 16 == 0) && ((uintptr_t)max_count % 16 == 0) &&
                     ((uintptr_t)min_count % 16 == 0);
    // (a count field in LDS is 16 bits wide: at most one pick per batch row and extreme; larger batches go to the
    // large-batch w_grad route and the count kernel's passes anyway)
    if (!vec || N >= 2048) return 1;
    const int log2r = 2, R = 4;
    // histogram + count plane of a slab: 4 neurons x kc columns x 8 bytes
    const int64_t lds_cap_bytes = (int64_t)g_lds_floats[dev] * 4;
    // whole rows of K = 4096 (one workgroup per CU); half rows with two workgroups per CU read the index
    // arrays twice and took 71 against 59 us at 256 x 4096 x 4096
    int64_t kc = 4096;
    while (kc > 64 && (int64_t)R * kc * 8 > lds_cap_bytes) kc /= 2;
    if (K < kc) kc = (K + 3) / 4 * 4;
    if ((int64_t)R * kc * 8 > lds_cap_bytes) return 1;
    const int64_t mtiles = ceil_div(M, R), ktiles = ceil_div(K, kc);
    if (ktiles > 65535) return 1;
    const int cus = num_cus();
    const int64_t per_cu = (160 * 1024) / (R * kc * 8) < 1 ? 1 : (160 * 1024) / (R * kc * 8);
    int tpw = (int)(mtiles * ktiles / (per_cu * cus));
    if (tpw < 1) tpw = 1;
    if (tpw > 8) tpw = 8;
    hipLaunchKernelGGL(mam_bwd_w_count_kernel, dim3((unsigned)ceil_div(mtiles, tpw), (unsigned)ktiles), dim3(NT_C),
                       (size_t)R * kc * 8, st, x, ldx, grad, argmax, argmin, x_sel, N * M, w_grad, max_count, min_count,
                       (int)N, (int)K, (int)M, log2r, (int)kc, (int)mtiles, tpw);
    return check_launch("mam_bwd_w_count_kernel");
}

// x_grad from selected weights handed over by a forward, whatever that forward read them from.
int x_grad_from_selected(const float *grad, const int32_t *argmax, const int32_t *argmin, const float *w_sel,
                         float *x_grad, int64_t N, int64_t K, int64_t M, hipStream_t st)
{
    const int dev = ensure_device(st);
    if (dev < 0) return dev;
    const int cells_cap = (g_lds_floats[dev] - 2048) / 2;
    const int kc = (int)(K < cells_cap ? K : cells_cap);
    hipLaunchKernelGGL((mam_bwd_x_kernel<MAM_W_MK>), dim3((unsigned)N), dim3(NT_X), (size_t)kc * 8,
                       st, (const float *)nullptr, (int64_t)0, grad, argmax, argmin, w_sel, N * M, x_grad, (int)K,
                       (int)M, kc, 1, window_span(2 * M));
    return check_launch("mam_bwd_x_kernel");
}

}  // namespace bwd
}  // namespace mam

static int backward_impl(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                         const float *grad, const int32_t *argmax, const int32_t *argmin,
                         const float *w_sel, const float *x_sel, float *x_grad, float *w_grad,
                         int64_t N, int64_t K, int64_t M, int planes, int range_len, void *stream)
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
    auto launch = [&](float *xg, float *wg, hipStream_t on) {
        if (w_layout == MAM_W_MK)
            return bwd::launch_layout<MAM_W_MK>(x, ldx, w, ldw, grad, argmax, argmin, w_sel, x_sel, xg, wg, N, K, M, on,
                                                planes, range_len);
        return bwd::launch_layout<MAM_W_KM>(x, ldx, w, ldw, grad, argmax, argmin, w_sel, x_sel, xg, wg, N, K, M, on,
                                            planes, range_len);
    };
    // x_grad is bound by LDS atomics and w_grad by memory traffic, and neither depends on the other: one
    // launch that holds both where the shape allows it, else two streams where that pays
    if (x_grad && w_grad && w_layout == MAM_W_MK && option(MAM_OPT_BACKWARD_ONE_LAUNCH) != MAM_BACKWARD_ONE_LAUNCH_OFF &&
        option(MAM_OPT_BACKWARD_FORK) != MAM_BACKWARD_FORK_ON &&
        option(MAM_OPT_BACKWARD_EXACT) != MAM_BACKWARD_EXACT_ON) {
        const int rc = bwd::launch_both(x, ldx, w, ldw, grad, argmax, argmin, w_sel, x_sel, x_grad, w_grad, N, K, M, st,
                                        planes, range_len,
                                        option(MAM_OPT_BACKWARD_ONE_LAUNCH) == MAM_BACKWARD_ONE_LAUNCH_AUTO);
        if (rc != 1) return rc;
    }
    if (x_grad && w_grad) {
        // Between eager launches the fork pays from 2^23 outputs on and with at least 1024 neurons, measured with
        // and without it (us): 12608 x 768 -> 3072 344 / 369, 16384 x 1024 -> 4096 563 / 598, 4096^3 243 / 282,
        // 8192 x 2048 -> 1024 113 / 121, 16384 x 4096 -> 1024 272 / 282; but 4096 x 1024 -> 1024 62 / 56, and with
        // 768 neurons (the rows kernel's workgroups are short and mostly waiting, and hold the LDS the w_grad
        // workgroups need) 12608 x 3072 -> 768 180 / 165, 25216 rows 335 / 316, 8192 rows 116 / 113.
        ForkedStream fork(st, N * M, N * M >= (1 << 23) && M >= 1024);
        if (fork.forked()) {
            const int rc_x = launch(x_grad, nullptr, fork.side());
            fork.join_later();
            const int rc_w = launch(nullptr, w_grad, st);
            const int rc_j = fork.join();
            return rc_x != MAM_OK ? rc_x : (rc_w != MAM_OK ? rc_w : rc_j);
        }
    }
    return launch(x_grad, w_grad, st);
}

extern "C" int mam_fc_backward(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                               const float *grad, const int32_t *argmax, const int32_t *argmin,
                               const float *w_sel, const float *x_sel, float *x_grad, float *w_grad,
                               int64_t N, int64_t K, int64_t M, void *stream)
{
    return backward_impl(x, ldx, w, ldw, w_layout, grad, argmax, argmin, w_sel, x_sel, x_grad, w_grad, N, K, M, 1, 0,
                         stream);
}

extern "C" int mam_fc_backward_count(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                                     const float *grad, const int32_t *argmax, const int32_t *argmin,
                                     const float *w_sel, const float *x_sel, float *x_grad, float *w_grad,
                                     int32_t *max_count, int32_t *min_count, int count_mode, int64_t N, int64_t K,
                                     int64_t M, void *stream)
{
    using namespace mam;
    if (count_mode != MAM_COUNT_REFERENCE && count_mode != MAM_COUNT_HITS && count_mode != MAM_COUNT_FLAGS)
        return fail(MAM_ERR_INVALID_ARGUMENT, "unknown selection-count mode %d", count_mode);
    if (!max_count || (count_mode != MAM_COUNT_REFERENCE && !min_count))
        return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    // the fused kernel: every operand of the plain calls valid, (M,K) weights, hits, w_grad wanted
    const bool fusable = count_mode == MAM_COUNT_HITS && w_layout == MAM_W_MK && w_grad && x && w && grad && argmax &&
                         argmin && N > 0 && M > 0 && K > 0 && N <= INT32_MAX / 2 && K <= INT32_MAX / 2 &&
                         M <= INT32_MAX / 2 && ldx >= K && ldw >= K;
    if (fusable) {
        hipStream_t st = static_cast<hipStream_t>(stream);
        const int rc_w = bwd::launch_w_count(x, ldx, grad, argmax, argmin, x_sel, w_grad, max_count, min_count, N, K, M,
                                             st);
        if (rc_w != 1) {
            if (rc_w != MAM_OK || !x_grad) return rc_w;
            return backward_impl(x, ldx, w, ldw, w_layout, grad, argmax, argmin, w_sel, x_sel, x_grad, nullptr, N, K, M,
                                 1, 0, stream);
        }
    }
    const int rc = backward_impl(x, ldx, w, ldw, w_layout, grad, argmax, argmin, w_sel, x_sel, x_grad, w_grad, N, K, M, 1,
                                 0, stream);
    if (rc != MAM_OK) return rc;
    return mam_selection_count(argmax, argmin, max_count, min_count, N, M, K, count_mode, stream);
}

extern "C" int mam_fc_backward_ranges(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                                      const float *grad, const int32_t *argmax, const int32_t *argmin,
                                      float *x_grad, float *w_grad, int64_t N, int64_t K, int64_t M,
                                      int64_t range_len, void *stream)
{
    if (range_len <= 0) return mam::fail(MAM_ERR_INVALID_ARGUMENT, "range_len must be positive");
    const int64_t planes = K > 0 ? (K + range_len - 1) / range_len : 1;
    if (planes > 65535) return mam::fail(MAM_ERR_UNSUPPORTED, "more than 65535 ranges");
    return backward_impl(x, ldx, w, ldw, w_layout, grad, argmax, argmin, nullptr, nullptr, x_grad, w_grad, N, K, M,
                         (int)planes, (int)(range_len < K ? range_len : K), stream);
}
