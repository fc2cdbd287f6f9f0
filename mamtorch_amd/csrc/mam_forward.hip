// Exact MAM forward for gfx950 (MI355X): c = max_k(x*w) + min_k(x*w) (+ bias), with the
// lowest k attaining each extreme.  Replaces the reference's v1 exact kernel
// (mamtorch/kernel/v1/csrc/cuda/fullyconnected.cu:33-175), serves the v4 operator, and the
// values-only variant replaces v4's fullyconnected_fast kernel
// (mamtorch/kernel/v4/csrc/cuda/fullyconnected_fast_kernel.cu:29-161).
//
// The (max, min, x) semiring has no matrix-core form, so the kernel is FP32-VALU bound and
// is organised to spend as few VALU issue slots per product as possible:
//
//   * One v_mul_f32 per product; v_max3_f32 / v_min3_f32 fold TWO products into the
//     running extreme per issue slot.  That is 2 slots per (multiply, max, min) triple.
//   * Indices are NOT tracked per product.  Products are consumed in groups of G = 16
//     consecutive k; after a group, one compare + one select per extreme records the group
//     id if the running extreme strictly improved.  Because the test is strict, the recorded
//     group is the one holding the FIRST occurrence of the final extreme.
//   * An epilogue re-reads the 16 operands of the recorded group, finds the first k whose
//     product equals the extreme, and recomputes the value from that k.  Recomputing also
//     removes the +0/-0 ambiguity of the hardware max/min, so values and indices are exactly
//     those of a scalar scan in ascending k with strict comparisons.  The selected operands can
//     be handed to the backward (w_sel, x_sel).
//
// Two tilings.  The first one below (mam_fwd_kernel) takes every layout, alignment and ragged
// size: a workgroup of 256 threads owns a 64 x 128 tile of c; X and W tiles of 32 consecutive k
// are staged in LDS as [row][k] (row stride 36 floats: 16-byte aligned and conflict-free for
// ds_read_b128 along k); a thread owns 4 x 8 outputs, strided by 16 in both directions, so that
// a wave's W reads cover all banks and its X reads broadcast.  Ragged edges are handled by
// replicating the last row / column / k on load: a replicated k duplicates an earlier product
// and can never win a strict comparison.  The second one (mam_fwd_sx_kernel, further down)
// serves the module's case -- (out, in) weight, aligned rows, K a multiple of 64 -- with
// wave-uniform batch rows whose x operands come through the scalar cache.
//
// Small N*M (the 256 x 4096 headline shape has only 256 tiles for 256 CUs x 2) is split
// along K; each split writes (value, group) partials and a merge kernel combines them in
// ascending k order with the same strict comparisons before resolving indices.
#include "mam_common.h"
#include "mam_offsets.h"

#include <stdlib.h>
#include <string.h>

namespace mam {
namespace fwd {

constexpr int BN = 64;        // batch rows per workgroup
constexpr int BM = 128;       // output neurons per workgroup
constexpr int KT = 32;        // k extent of one LDS tile
constexpr int LDK = KT + 4;   // LDS row stride in floats
constexpr int G = 16;         // products per index-tracking group
constexpr int TI = 4;         // rows per thread
constexpr int TJ = 8;         // columns per thread
constexpr int NT = 256;       // threads per workgroup
constexpr int GROUP_N = 8;    // row tiles swept together so that W panels are reused from L2
constexpr int MAX_SPLITS = 16;

struct Params {
    const float *x;
    int64_t ldx;
    const float *w;
    int64_t ldw;
    const float *bias;
    float *c;
    int32_t *argmax;
    int32_t *argmin;
    float *wsel;      // optional [2][N*M]: the selected weights w[argmax], w[argmin] (for the backward)
    float *xsel;      // optional [2][N*M]: the selected inputs x[argmax], x[argmin] (for the backward)
    float *part;      // split-K partials: [split][3 or 2][N*M]: max, min, (group ids packed 16:16)
    int *tickets;     // fused merge: one counter per tile, behind the partials, zero at launch
    int N, K, M;
    int tiles_n, tiles_m, splits, k_per_split;
    int vec_x, vec_w;  // 16-byte global loads are legal for x / w
    int fast;          // the k-invariant 32-bit-offset staging path is legal
    int coop;          // the cooperative resolve is legal: (M,K) w, 16-byte rows, K % G == 0
    int group_n;       // row tiles swept under one W panel (tile order of the launch)
    int gt;            // products per recorded group: G, or 2 G on the wave-uniform-rows tiling at large K
};

// An extreme that still holds its initial value (-inf for the max, +inf for the min) was never strictly
// improved: every product was NaN or equal to that infinity.  The ordered compares of a scalar scan
// (mamtorch/kernel/v1/csrc/cuda/fullyconnected.cu:132-142) leave the index at the first k of the range in
// that case, and so does the resolve: it looks for no match then.
__device__ __forceinline__ bool never_improved(float target, bool is_min)
{
    return target == (is_min ? __builtin_inff() : -__builtin_inff());
}

// First k in group g (ascending) whose product equals `target`; value recomputed from it.
// The cost of this step is the number of cache lines each wave touches, not arithmetic, so the
// G operands of each side are fetched with 16-byte loads when the layout allows it.
template <int LAYOUT>
__device__ __forceinline__ void resolve(const Params &p, int n, int m, int kb, int klast, float target, bool is_min,
                                        float &val, int &idx, float &wsel, float &xsel)
{
    // the group is k = kb .. kb + G - 1; k beyond klast (the last k of the scanned range) repeat klast
    idx = kb < klast ? kb : klast;
    val = target;
    const float *xr = p.x + (int64_t)n * p.ldx;
    wsel = load_w<LAYOUT>(p.w, p.ldw, idx, m);
    xsel = xr[idx];
    float xv[G], wv[G];
    const bool whole = kb + G <= klast + 1 && (kb & 3) == 0;
    if (whole && p.vec_x) {
#pragma unroll
        for (int q = 0; q < G / 4; ++q) {
            const float4 a = *reinterpret_cast<const float4 *>(xr + kb + q * 4);
            xv[q * 4 + 0] = a.x; xv[q * 4 + 1] = a.y; xv[q * 4 + 2] = a.z; xv[q * 4 + 3] = a.w;
        }
    } else {
#pragma unroll
        for (int kk = 0; kk < G; ++kk) xv[kk] = xr[(kb + kk) < klast ? (kb + kk) : klast];
    }
    if (LAYOUT == MAM_W_MK && whole && p.vec_w) {
        const float *wr = p.w + (int64_t)m * p.ldw + kb;
#pragma unroll
        for (int q = 0; q < G / 4; ++q) {
            const float4 a = *reinterpret_cast<const float4 *>(wr + q * 4);
            wv[q * 4 + 0] = a.x; wv[q * 4 + 1] = a.y; wv[q * 4 + 2] = a.z; wv[q * 4 + 3] = a.w;
        }
    } else {
#pragma unroll
        for (int kk = 0; kk < G; ++kk)
            wv[kk] = load_w<LAYOUT>(p.w, p.ldw, (kb + kk) < klast ? (kb + kk) : klast, m);
    }
    const bool never = never_improved(target, is_min);
#pragma unroll
    for (int kk = G - 1; kk >= 0; --kk) {
        const float prod = xv[kk] * wv[kk];
        if (prod == target && !never) { idx = (kb + kk) < klast ? (kb + kk) : klast; val = prod; wsel = wv[kk]; xsel = xv[kk]; }
    }
}

// A zero extreme carries the sign of the FIRST zero product; the hardware max/min may have
// kept another zero's sign.  Rare (whole column of products has no positive / no negative
// entry), so a plain scan is enough.
// (Not inlined, and handed plain pointers: a reference to the kernel's parameter block would force a
// copy of the block into every lane's scratch memory.)
template <int LAYOUT>
__device__ __noinline__ float first_zero_product(const float *xr, const float *w, int64_t ldw, int m, int kbegin,
                                                 int kend)
{
    for (int k = kbegin; k < kend; ++k) {
        const float prod = xr[k] * load_w<LAYOUT>(w, ldw, k, m);
        if (prod == 0.0f) return prod;
    }
    return 0.0f;
}

template <int LAYOUT, bool ARGS>
__device__ __forceinline__ void finish(const Params &p, int n, int m, float vmax, float vmin,
                                       int gmax, int gmin)
{
    float hi = vmax, lo = vmin;
    int ih = 0, il = 0;
    float wh = 0.0f, wl = 0.0f, xh = 0.0f, xl = 0.0f;
    if (ARGS) {
        resolve<LAYOUT>(p, n, m, gmax * G, p.K - 1, vmax, false, hi, ih, wh, xh);
        resolve<LAYOUT>(p, n, m, gmin * G, p.K - 1, vmin, true, lo, il, wl, xl);
    } else {
        if (hi == 0.0f) hi = first_zero_product<LAYOUT>(p.x + (int64_t)n * p.ldx, p.w, p.ldw, m, 0, p.K);
        if (lo == 0.0f) lo = first_zero_product<LAYOUT>(p.x + (int64_t)n * p.ldx, p.w, p.ldw, m, 0, p.K);
    }
    float s = hi + lo;
    if (p.bias) s = s + p.bias[m];
    const int64_t o = (int64_t)n * p.M + m;
    p.c[o] = s;
    if (ARGS) {
        p.argmax[o] = ih;
        p.argmin[o] = il;
        if (p.wsel) {
            p.wsel[o] = wh;
            p.wsel[(int64_t)p.N * p.M + o] = wl;
        }
        if (p.xsel) {
            p.xsel[o] = xh;
            p.xsel[(int64_t)p.N * p.M + o] = xl;
        }
    }
}

// Cooperative resolve of the 64 outputs held by one wave (fast layouts only: (M,K) weight,
// 16-byte aligned rows, K a multiple of G).  The cost of resolving is cache-line lookups plus the
// instructions around them, so the G/4 lanes of a task each fetch one 16-byte chunk of x and of w
// (a task touches one contiguous G*4-byte segment per operand), the lanes of a task agree on the
// first match with two DPP min steps (no LDS permutes), only the winning lane writes the task's
// result to LDS, and in a second pass lane s stores output s: whole-wave stores, contiguous where
// consecutive slots are consecutive neurons.  128 tasks (64 outputs x {max, min}), 64/(G/4) per
// round.
//   vals : LDS, [2][64]  running max, running min of the wave's outputs
//   grps : LDS, [2][64]  absolute group id of the max, of the min
//   res  : LDS, [8][64]  scratch of this wave: value, index, weight, input of the max and of the min
//   nm_of(slot, n, m, valid): output coordinates of slot 0..63 (clamped into range when !valid)
constexpr int LPT = G / 4;             // lanes per task
constexpr int TPR = 64 / LPT;          // tasks per round
constexpr int RES_ROUNDS = 128 / TPR;
constexpr int RES_WORDS = 8 * 64;      // LDS words of `res` per wave
static_assert(LPT == 4, "the lane exchange below is written for 4 lanes per task");

__device__ __forceinline__ int quad_min(int v)
{
    // minimum over the 4 lanes of a quad: neighbours (quad_perm [1,0,3,2]), then pairs ([2,3,0,1])
    int o = __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xf, 0xf, true);
    v = o < v ? o : v;
    o = __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xf, 0xf, true);
    return o < v ? o : v;
}

//   operands(r, slot, sub, kb, xp, wp): where the GT/4 x and GT/4 w operands k = kb .. kb+GT/4-1 of the task in
//   round r live.  The addresses are most of the instructions of a round when they are formed in 64 bits per
//   lane, so a caller whose 64 outputs share bases hands in something cheaper.
//   GT: the k loop's tracking span, 16 or 32 products per recorded group; a lane takes GT/4 of them (one or two
//   16-byte loads per operand), and the loads of 8 * 16 / GT rounds are in flight together.
template <int GT, class NM, class OP>
__device__ __forceinline__ void resolve_wave(const Params &p, const float *vals, const int *grps, float *res,
                                             int lane, NM nm_of, OP operands)
{
    static_assert(GT == 16 || GT == 32, "tracking span");
    constexpr int PPL = GT / LPT;             // products per lane
    constexpr int NV = PPL / 4;               // 16-byte loads per operand and lane
    constexpr int BATCH = RES_ROUNDS / NV;    // rounds whose loads are issued before the first use
    float *res_v = res;                                    // [2][64]
    int *res_i = reinterpret_cast<int *>(res + 128);        // [2][64]
    float *res_w = res + 256;                               // [2][64]
    float *res_x = res + 384;                               // [2][64]
#pragma unroll
    for (int r0 = 0; r0 < RES_ROUNDS; r0 += BATCH) {
        // every load of the batch first, then the matching
        float4 xa[BATCH][NV], wa[BATCH][NV];
        float target[BATCH];
        int grp[BATCH];
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            const int r = r0 + b;
            const int task = r * TPR + lane / LPT;
            const int slot = task >> 1, ext = task & 1, sub = lane % LPT;
            target[b] = vals[ext * 64 + slot];
            grp[b] = grps[ext * 64 + slot];
            const float *xp, *wp;
            operands(r, slot, sub, grp[b] * GT + sub * PPL, xp, wp);
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                xa[b][v] = reinterpret_cast<const float4 *>(xp)[v];
                wa[b][v] = reinterpret_cast<const float4 *>(wp)[v];
            }
        }
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            const int r = r0 + b;
            const int task = r * TPR + lane / LPT;
            const int slot = task >> 1, ext = task & 1, sub = lane % LPT;
            // position within the group of this lane's first match (lowest wins), 255 = none
            int key = 255;
            float wsel = wa[b][0].x, xsel = xa[b][0].x;      // kept only by the fallback below
#pragma unroll
            for (int v = NV - 1; v >= 0; --v) {
                const float p0 = xa[b][v].x * wa[b][v].x, p1 = xa[b][v].y * wa[b][v].y, p2 = xa[b][v].z * wa[b][v].z,
                            p3 = xa[b][v].w * wa[b][v].w;
                const int k0 = sub * PPL + v * 4;
                if (p3 == target[b]) { key = k0 + 3; wsel = wa[b][v].w; xsel = xa[b][v].w; }
                if (p2 == target[b]) { key = k0 + 2; wsel = wa[b][v].z; xsel = xa[b][v].z; }
                if (p1 == target[b]) { key = k0 + 1; wsel = wa[b][v].y; xsel = xa[b][v].y; }
                if (p0 == target[b]) { key = k0 + 0; wsel = wa[b][v].x; xsel = xa[b][v].x; }
            }
            if (never_improved(target[b], ext != 0)) key = 255;
            const int best = quad_min(key);
            // no product equals the extreme (NaN operands), or the extreme was never improved: the first k of
            // the group, from lane 0
            const bool fallback = best == 255 && sub == 0;
            if ((key == best && key != 255) || fallback) {
                // the value is recomputed from the selected operands (the sign of a zero follows them)
                res_v[ext * 64 + slot] = fallback ? target[b] : xsel * wsel;
                res_i[ext * 64 + slot] = grp[b] * GT + (fallback ? 0 : key);
                res_w[ext * 64 + slot] = wsel;
                res_x[ext * 64 + slot] = xsel;
            }
        }
    }
    // lane s finishes output s
    int n, m;
    bool valid;
    nm_of(lane, n, m, valid);
    float sum = res_v[lane] + res_v[64 + lane];
    if (p.bias) sum = sum + p.bias[m];
    if (valid) {
        const int64_t o = (int64_t)n * p.M + m;
        p.c[o] = sum;
        p.argmax[o] = res_i[lane];
        p.argmin[o] = res_i[64 + lane];
        if (p.wsel) {
            p.wsel[o] = res_w[lane];
            p.wsel[(int64_t)p.N * p.M + o] = res_w[64 + lane];
        }
        if (p.xsel) {
            p.xsel[o] = res_x[lane];
            p.xsel[(int64_t)p.N * p.M + o] = res_x[64 + lane];
        }
    }
}

// The general case: every output has its own row of x and of w.
template <class NM>
__device__ __forceinline__ void resolve_wave(const Params &p, const float *vals, const int *grps, float *res,
                                             int lane, NM nm_of)
{
    resolve_wave<G>(p, vals, grps, res, lane, nm_of,
                 [&](int, int slot, int, int kb, const float *&xp, const float *&wp) {
                     int n, m;
                     bool valid;
                     nm_of(slot, n, m, valid);
                     xp = p.x + (int64_t)n * p.ldx + kb;
                     wp = p.w + (int64_t)m * p.ldw + kb;
                 });
}

// Stages one k-tile [k0, k0+KT) of X and W into LDS for any alignment and any ragged edge:
// rows, columns and k beyond the problem are replaced by the last valid one.
template <int LAYOUT>
__device__ __forceinline__ void stage_tile_generic(const Params &p, float (*xs)[LDK], float (*ws)[LDK],
                                                   int tid, int row0, int col0, int k0, int ke)
{
    const int kl = ke - 1;
#pragma unroll
    for (int it = 0; it < (BN * KT / 4) / NT; ++it) {
        const int e = tid + it * NT;
        const int r = e >> 3, ch = e & 7;
        const int row = (row0 + r) < p.N ? (row0 + r) : (p.N - 1);
        const int k = k0 + ch * 4;
        const float *src = p.x + (int64_t)row * p.ldx;
        float4 v;
        v.x = src[k < kl ? k : kl];
        v.y = src[k + 1 < kl ? k + 1 : kl];
        v.z = src[k + 2 < kl ? k + 2 : kl];
        v.w = src[k + 3 < kl ? k + 3 : kl];
        *reinterpret_cast<float4 *>(&xs[r][ch * 4]) = v;
    }
    if (LAYOUT == MAM_W_MK) {
#pragma unroll
        for (int it = 0; it < (BM * KT / 4) / NT; ++it) {
            const int e = tid + it * NT;
            const int r = e >> 3, ch = e & 7;
            const int col = (col0 + r) < p.M ? (col0 + r) : (p.M - 1);
            const int k = k0 + ch * 4;
            const float *src = p.w + (int64_t)col * p.ldw;
            float4 v;
            v.x = src[k < kl ? k : kl];
            v.y = src[k + 1 < kl ? k + 1 : kl];
            v.z = src[k + 2 < kl ? k + 2 : kl];
            v.w = src[k + 3 < kl ? k + 3 : kl];
            *reinterpret_cast<float4 *>(&ws[r][ch * 4]) = v;
        }
    } else {
#pragma unroll
        for (int it = 0; it < (BM * KT / 4) / NT; ++it) {
            const int e = tid + it * NT;
            const int c4 = (e & 7) + ((e >> 8) << 3);
            const int kk = (e >> 3) & 31;
            const int k = (k0 + kk) < kl ? (k0 + kk) : kl;
            const int mb = col0 + c4 * 4;
            const int ml = p.M - 1;
            const float *src = p.w + (int64_t)k * p.ldw;
            ws[c4 * 4 + 0][kk] = src[mb < ml ? mb : ml];
            ws[c4 * 4 + 1][kk] = src[mb + 1 < ml ? mb + 1 : ml];
            ws[c4 * 4 + 2][kk] = src[mb + 2 < ml ? mb + 2 : ml];
            ws[c4 * 4 + 3][kk] = src[mb + 3 < ml ? mb + 3 : ml];
        }
    }
}

// Stages one full, 16-byte-aligned k-tile of the (K, M) operand through registers: 8 lanes fetch
// 128 bytes of one k row, and the tile is transposed on the way into LDS.
__device__ __forceinline__ void stage_w_km_fast(const float *wt, float (*ws)[LDK], int tid,
                                                const uint32_t (&wo)[(BM * KT / 4) / NT])
{
    float4 wr[(BM * KT / 4) / NT];
#pragma unroll
    for (int it = 0; it < (BM * KT / 4) / NT; ++it) wr[it] = *reinterpret_cast<const float4 *>(wt + wo[it]);
#pragma unroll
    for (int it = 0; it < (BM * KT / 4) / NT; ++it) {
        const int e = tid + it * NT;
        const int c4 = (e & 7) + ((e >> 8) << 3);
        const int kk = (e >> 3) & 31;
        ws[c4 * 4 + 0][kk] = wr[it].x;
        ws[c4 * 4 + 1][kk] = wr[it].y;
        ws[c4 * 4 + 2][kk] = wr[it].z;
        ws[c4 * 4 + 3][kk] = wr[it].w;
    }
}

// One wave-level direct-to-LDS load moves 64 x 16 bytes into 1 KiB of consecutive LDS.  A tile
// (X rows then W rows, 9 16-byte slots per row: 8 of data, 1 of padding) is exactly 27 such loads,
// the first 9 of them X; wave w issues loads w, w+4, ...  No register holds the data in flight.
constexpr int TILE_FLOATS = (BN + BM) * LDK;
constexpr int DMA_INSTR = TILE_FLOATS / 4 / 64;
constexpr int DMA_X_INSTR = BN * LDK / 4 / 64;
constexpr int DMA_PER_WAVE = (DMA_INSTR + NT / 64 - 1) / (NT / 64);
static_assert(TILE_FLOATS % 256 == 0 && (BN * LDK) % 256 == 0, "tile must be whole wave-level loads");

// Per-lane source offsets of a wave's loads live in LDS ([load][thread]): they are needed once
// per tile, and a register spilled to scratch would be reloaded through the same counter that
// tracks the loads in flight.
__device__ __forceinline__ void dma_tile(const char *xt, const char *wt, float *tile, int wave,
                                         const uint32_t *doff, bool x_only)
{
#pragma unroll
    for (int t = 0; t < DMA_PER_WAVE; ++t) {
        // every wave issues DMA_PER_WAVE loads; the one past the end repeats the last load
        int inst = wave + (NT / 64) * t;
        inst = inst < DMA_INSTR ? inst : DMA_INSTR - 1;
        if (x_only && t * (NT / 64) >= DMA_X_INSTR) break;
        if (x_only) inst = inst < DMA_X_INSTR ? inst : DMA_X_INSTR - 1;
        // uniform 64-bit base + 32-bit lane offset: the scalar-base form of the load, one
        // address register per load
        const char *src = (inst < DMA_X_INSTR ? xt : wt) + (uint64_t)doff[t * NT];
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void *)src,
            (__attribute__((address_space(3))) void *)(tile + inst * 256), 16, 0, 0);
    }
}

// 2 groups of 16 k from one staged tile: 32 outputs x 16 products each.  The two groups are
// unrolled so that the running extremes ping-pong between two register sets: the value before
// the group stays readable for the "did it improve" test without a copy.
template <bool ARGS>
__device__ __forceinline__ void compute_tile(const float *tile, int tx, int ty, int grel0,
                                             float (&vmax)[TI][TJ], float (&vmin)[TI][TJ],
                                             int (&gmax)[TI][TJ], int (&gmin)[TI][TJ])
{
    const float (*xs)[LDK] = reinterpret_cast<const float (*)[LDK]>(tile);
    const float (*ws)[LDK] = reinterpret_cast<const float (*)[LDK]>(tile + BN * LDK);
#pragma unroll
    for (int gg = 0; gg < KT / G; ++gg) {
        const int grel = grel0 + gg;
        float xv[TI][G];
#pragma unroll
        for (int i = 0; i < TI; ++i)
#pragma unroll
            for (int q = 0; q < G / 4; ++q) {
                const float4 t = *reinterpret_cast<const float4 *>(&xs[ty + 16 * i][gg * G + q * 4]);
                xv[i][q * 4 + 0] = t.x; xv[i][q * 4 + 1] = t.y;
                xv[i][q * 4 + 2] = t.z; xv[i][q * 4 + 3] = t.w;
            }
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            float wv[G];
#pragma unroll
            for (int q = 0; q < G / 4; ++q) {
                const float4 t = *reinterpret_cast<const float4 *>(&ws[tx + 16 * j][gg * G + q * 4]);
                wv[q * 4 + 0] = t.x; wv[q * 4 + 1] = t.y;
                wv[q * 4 + 2] = t.z; wv[q * 4 + 3] = t.w;
            }
#pragma unroll
            for (int i = 0; i < TI; ++i) {
                const float om = vmax[i][j], on = vmin[i][j];
                float hi = om, lo = on;
#pragma unroll
                for (int q = 0; q < G; q += 2) {
                    const float a = xv[i][q] * wv[q], b = xv[i][q + 1] * wv[q + 1];
                    hi = __builtin_fmaxf(__builtin_fmaxf(hi, a), b);   // v_max3_f32
                    lo = __builtin_fminf(__builtin_fminf(lo, a), b);   // v_min3_f32
                }
                if (ARGS) {
                    // one compare + one select per extreme and group, left to the compiler to
                    // place: issued back to back they stall on the condition mask
                    gmax[i][j] = (hi > om) ? grel : gmax[i][j];
                    gmin[i][j] = (lo < on) ? grel : gmin[i][j];
                }
                vmax[i][j] = hi;
                vmin[i][j] = lo;
            }
        }
    }
}

template <int LAYOUT, bool ARGS>
__global__ __launch_bounds__(NT, 2) void mam_fwd_kernel(const Params p)
{
    // Two tile buffers as two separate arrays: the compiler can then see that loads in flight
    // into one never alias reads of the other, and lets them overlap.
    __shared__ __attribute__((aligned(16))) float tile_a[TILE_FLOATS];
    __shared__ __attribute__((aligned(16))) float tile_b[TILE_FLOATS];

    const int tid = threadIdx.x;
    const int tx = tid & 15;  // column lane: columns tx + 16*j
    const int ty = tid >> 4;  // row lane:    rows    ty + 16*i
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // ---- which tile: XCD-aware, then row tiles grouped under one W panel ----
    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    const int tiles = p.tiles_n * p.tiles_m;
    const int split = logical / tiles;
    const int l = logical - split * tiles;
    const int per_group = p.group_n * p.tiles_m;
    const int grp = l / per_group;
    const int first_n = grp * p.group_n;
    const int gsize = (p.tiles_n - first_n) < p.group_n ? (p.tiles_n - first_n) : p.group_n;
    const int lin = l - grp * per_group;
    const int tn = first_n + lin % gsize;
    const int tm = lin / gsize;
    const int row0 = tn * BN, col0 = tm * BM;
    const int kb = split * p.k_per_split;
    const int ke = (kb + p.k_per_split) < p.K ? (kb + p.k_per_split) : p.K;
    const int ntiles = (ke - kb + KT - 1) / KT;

    float vmax[TI][TJ], vmin[TI][TJ];
    // groups of the running max / min, counted from the first group of this workgroup's k range
    int gmax[TI][TJ], gmin[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            vmax[i][j] = -__builtin_inff();
            vmin[i][j] = __builtin_inff();
            gmax[i][j] = 0;
            gmin[i][j] = 0;
        }

    // ---- staging ----
    // Full, aligned tiles take a fast path whose per-thread source offsets do not depend on k
    // (rows / columns past the edge re-read the last valid one).  For x and an (M,K) w that
    // path is direct-to-LDS and runs one tile ahead of the arithmetic; a (K,M) w goes through
    // registers because it has to be transposed, and needs a full column tile.  Everything
    // else (ragged k tail, unaligned views) takes the generic path.
    const bool fast = p.fast && (LAYOUT == MAM_W_MK || col0 + BM <= p.M);
    const float *xbase = p.x + (int64_t)row0 * p.ldx;
    const float *wbase = LAYOUT == MAM_W_MK ? p.w + (int64_t)col0 * p.ldw : p.w + col0;
    __shared__ uint32_t doff_s[DMA_PER_WAVE * NT];
    const uint32_t *doff = doff_s + tid;
#pragma unroll
    for (int t = 0; t < DMA_PER_WAVE; ++t) {
        int inst = wave + (NT / 64) * t;
        inst = inst < DMA_INSTR ? inst : DMA_INSTR - 1;
        if (LAYOUT == MAM_W_KM) inst = inst < DMA_X_INSTR ? inst : DMA_X_INSTR - 1;
        const int slot = inst * 64 + (tid & 63);
        const int row = slot / (LDK / 4), pos = slot % (LDK / 4);
        const int ch = pos < KT / 4 ? pos : KT / 4 - 1;   // the padding slot re-reads the last chunk
        uint32_t off;
        if (row < BN) {
            const int r = ((row0 + row) < p.N ? (row0 + row) : (p.N - 1)) - row0;
            off = (uint32_t)(r * (int)p.ldx + ch * 4) * 4u;
        } else {
            const int c = ((col0 + row - BN) < p.M ? (col0 + row - BN) : (p.M - 1)) - col0;
            off = (uint32_t)(c * (int)p.ldw + ch * 4) * 4u;
        }
        doff_s[t * NT + tid] = off;
    }
    uint32_t wo[(BM * KT / 4) / NT];   // (K,M) register path only
    if (LAYOUT == MAM_W_KM) {
#pragma unroll
        for (int it = 0; it < (BM * KT / 4) / NT; ++it) {
            const int e = tid + it * NT;
            const int c4 = (e & 7) + ((e >> 8) << 3);
            const int kk = (e >> 3) & 31;
            wo[it] = (uint32_t)(kk * (int)p.ldw + c4 * 4);
        }
    }

    // Tiles that take the direct-to-LDS path: double-buffered, loads one tile ahead of the
    // arithmetic, nothing but the running extremes, the operands and three addresses live.
    int t0 = 0;
    if (LAYOUT == MAM_W_MK && fast) {
        const int full = (ke - kb) / KT;
        if (full > 0) {
            const char *xk = reinterpret_cast<const char *>(xbase + kb);
            const char *wk = reinterpret_cast<const char *>(wbase + kb);
            dma_tile(xk, wk, tile_a, wave, doff, false);
            __syncthreads();
            for (int t = 0; t < full; t += 2) {
                xk += KT * sizeof(float);
                wk += KT * sizeof(float);
                if (t + 1 < full) dma_tile(xk, wk, tile_b, wave, doff, false);
                compute_tile<ARGS>(tile_a, tx, ty, t * (KT / G), vmax, vmin, gmax, gmin);
                __syncthreads();
                if (t + 1 >= full) break;
                xk += KT * sizeof(float);
                wk += KT * sizeof(float);
                if (t + 2 < full) dma_tile(xk, wk, tile_a, wave, doff, false);
                compute_tile<ARGS>(tile_b, tx, ty, (t + 1) * (KT / G), vmax, vmin, gmax, gmin);
                __syncthreads();
            }
            t0 = full;
        }
    }
    // Everything else, one tile at a time: the ragged k tail, unaligned views, and the (K,M)
    // layout, whose w goes through registers because it has to be transposed.
#pragma unroll 1
    for (int t = t0; t < ntiles; ++t) {
        const int k0 = kb + t * KT;
        float (*xs)[LDK] = reinterpret_cast<float (*)[LDK]>(tile_a);
        float (*ws)[LDK] = reinterpret_cast<float (*)[LDK]>(tile_a + BN * LDK);
        if (LAYOUT == MAM_W_KM && fast && k0 + KT <= ke) {
            const char *xk = reinterpret_cast<const char *>(xbase + k0);
            dma_tile(xk, xk, tile_a, wave, doff, true);
            stage_w_km_fast(wbase + (int64_t)k0 * p.ldw, ws, tid, wo);
        } else {
            stage_tile_generic<LAYOUT>(p, xs, ws, tid, row0, col0, k0, ke);
        }
        __syncthreads();
        compute_tile<ARGS>(tile_a, tx, ty, t * (KT / G), vmax, vmin, gmax, gmin);
        __syncthreads();
    }

    // ---- epilogue ----
    const int g0 = kb / G;
    if (p.splits == 1 && ARGS && p.coop) {
        // The tiles in LDS are dead (the k loop ended on a barrier).  Row by row, each wave parks
        // its 64 x 8 results in LDS and resolves them cooperatively.
        static_assert(2 * TJ * NT <= TILE_FLOATS, "result stash does not fit a tile buffer");
        const int lane = tid & 63;
        float *vals = tile_a + wave * (TJ * 2 * 64);
        int *grps = reinterpret_cast<int *>(tile_b) + wave * (TJ * 2 * 64);
        static_assert((NT / 64) * (TJ * 2 * 64 + RES_WORDS) <= TILE_FLOATS, "resolve scratch does not fit");
        float *res = tile_a + (NT / 64) * (TJ * 2 * 64) + wave * RES_WORDS;
        // From here on a wave touches only its own corner of LDS, and the LDS operations of one wave
        // complete in issue order: no workgroup barrier between parking and resolving.
        __syncthreads();
#pragma unroll
        for (int i = 0; i < TI; ++i) {
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                vals[(j * 2 + 0) * 64 + lane] = vmax[i][j];
                vals[(j * 2 + 1) * 64 + lane] = vmin[i][j];
                grps[(j * 2 + 0) * 64 + lane] = g0 + gmax[i][j];
                grps[(j * 2 + 1) * 64 + lane] = g0 + gmin[i][j];
            }
            __builtin_amdgcn_wave_barrier();
#pragma unroll 1
            for (int j = 0; j < TJ; ++j) {
                const int nbase = row0 + 16 * i + 4 * wave, mbase = col0 + 16 * j;
                resolve_wave(p, vals + j * 128, grps + j * 128, res, lane,
                             [&](int slot, int &n, int &m, bool &valid) {
                                 n = nbase + (slot >> 4);
                                 m = mbase + (slot & 15);
                                 valid = n < p.N && m < p.M;
                                 n = n < p.N ? n : p.N - 1;
                                 m = m < p.M ? m : p.M - 1;
                             });
            }
        }
    } else if (p.splits == 1) {
        // Generic layouts: each thread parks one row of its results in its own LDS slots so that
        // the index resolution can be a rolled loop over j (one copy of the code per row, and no
        // register array indexed at run time).
        static_assert(3 * TJ * NT <= TILE_FLOATS, "result stash does not fit a tile buffer");
        float *stash = tile_a + tid;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                stash[(0 * TJ + j) * NT] = vmax[i][j];
                stash[(1 * TJ + j) * NT] = vmin[i][j];
                stash[(2 * TJ + j) * NT] = __int_as_float(gmax[i][j] | (gmin[i][j] << 16));
            }
            const int n = row0 + ty + 16 * i;
            if (n < p.N) {
#pragma unroll 1
                for (int j = 0; j < TJ; ++j) {
                    const int m = col0 + tx + 16 * j;
                    if (m < p.M) {
                        const uint32_t gs = __float_as_uint(stash[(2 * TJ + j) * NT]);
                        finish<LAYOUT, ARGS>(p, n, m, stash[(0 * TJ + j) * NT], stash[(1 * TJ + j) * NT],
                                             g0 + (int)(gs & 0xffffu), g0 + (int)(gs >> 16));
                    }
                }
            }
        }
    } else {
        const int64_t nm = (int64_t)p.N * p.M;
        float *base = p.part + (int64_t)split * (ARGS ? 3 : 2) * nm;
#pragma unroll
        for (int i = 0; i < TI; ++i)
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                const int n = row0 + ty + 16 * i, m = col0 + tx + 16 * j;
                if (n < p.N && m < p.M) {
                    const int64_t o = (int64_t)n * p.M + m;
                    base[o] = vmax[i][j];
                    base[nm + o] = vmin[i][j];
                    if (ARGS) base[2 * nm + o] = __int_as_float(gmax[i][j] | (gmin[i][j] << 16));
                }
            }
    }
}

// Combines split-K partials in ascending k order (strict comparisons keep the earliest
// group on ties), then resolves indices / zero signs exactly as the single-pass epilogue.
template <int LAYOUT, bool ARGS, bool COOP, int GT = G>
__global__ __launch_bounds__(256) void mam_fwd_merge_kernel(const Params p)
{
    // A workgroup owns a PR x PC patch of c (16 x 16; with the cooperative resolve 4 x 64: a wave takes one batch
    // row, and its piece of every partial plane and of every output array is two whole 128-byte lines; measured at
    // 256 x 4096 x 4096: 28.4 us with 16 x 16, 27.0 with 8 x 32, 26.6 with 4 x 64).  Resolving re-reads GT
    // weights of row m per output, i.e. random lines of the weight matrix; ordering the patches so that all batch
    // patches of one PC-neuron range run back to back on one XCD keeps those weight rows in that L2.
    constexpr int PC = COOP ? 64 : 16, PR = 256 / PC, LOG2PC = COOP ? 6 : 4;
    __shared__ float vals_s[4][2][64];
    __shared__ int grps_s[4][2][64];
    __shared__ float res_s[4][RES_WORDS];
    const int64_t nm = (int64_t)p.N * p.M;
    const int patches_n = (p.N + PR - 1) / PR;
    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    const int pm = logical / patches_n, pn = logical - pm * patches_n;
    const int n_own = pn * PR + (threadIdx.x >> LOG2PC), m_own = pm * PC + (threadIdx.x & (PC - 1));
    const bool live = n_own < p.N && m_own < p.M;
    const int64_t o = (int64_t)n_own * p.M + m_own;
    const int stride = ARGS ? 3 : 2;
    const int gps = p.k_per_split / GT;   // groups per split
    float vmax = 0.0f, vmin = 0.0f;
    int gmax = 0, gmin = 0;
    if (live) {
        vmax = p.part[o];
        vmin = p.part[nm + o];
        if (ARGS) {
            const int pk = __float_as_int(p.part[2 * nm + o]);
            gmax = pk & 0xffff;
            gmin = (pk >> 16) & 0xffff;
        }
        for (int s = 1; s < p.splits; ++s) {
            const float *base = p.part + (int64_t)s * stride * nm;
            const float hi = base[o], lo = base[nm + o];
            int pk = 0;
            if (ARGS) pk = __float_as_int(base[2 * nm + o]);
            if (hi > vmax) {
                vmax = hi;
                gmax = s * gps + (pk & 0xffff);
            }
            if (lo < vmin) {
                vmin = lo;
                gmin = s * gps + ((pk >> 16) & 0xffff);
            }
        }
    }
    if (COOP) {
        const int lane = threadIdx.x & 63;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        vals_s[wave][0][lane] = vmax;
        vals_s[wave][1][lane] = vmin;
        grps_s[wave][0][lane] = gmax;
        grps_s[wave][1][lane] = gmin;
        __syncthreads();
        const int nbase = pn * PR + (PR / 4) * wave, mbase = pm * PC;
        // slot = 8 r + lane / 8 in round r: batch row nbase + slot / PC (the same for the whole wave) and
        // neuron mbase + slot % PC = mbase + 8 (r % (PC / 8)) + lane / 8, so the operands sit at 32-bit byte
        // offsets from wave-uniform bases (the host checked that PC rows of w span < 4 GiB)
        const int mb = mbase < p.M ? mbase : p.M - 1;
        const char *wrows = reinterpret_cast<const char *>(p.w + (int64_t)mb * p.ldw);
        const uint32_t ldw4 = (uint32_t)p.ldw * 4u;
        const uint32_t last = last_row_offset(p.M, mb, PC, ldw4);
        const uint32_t mine = (uint32_t)(lane >> 3) * ldw4;
        resolve_wave<GT>(p, &vals_s[wave][0][0], &grps_s[wave][0][0], &res_s[wave][0], lane,
                     [&](int slot, int &n, int &m, bool &valid) {
                         n = nbase + (slot >> LOG2PC);
                         m = mbase + (slot & (PC - 1));
                         valid = n < p.N && m < p.M;
                         n = n < p.N ? n : p.N - 1;
                         m = m < p.M ? m : p.M - 1;
                     },
                     [&](int r, int, int, int kb, const float *&xp, const float *&wp) {
                         const int nr = nbase + (r >> (LOG2PC - 3));
                         const int n = nr < p.N ? nr : (p.N - 1);
                         const char *xrow = reinterpret_cast<const char *>(p.x + (int64_t)n * p.ldx);
                         const uint32_t row = mine + (uint32_t)(8 * (r & (PC / 8 - 1))) * ldw4;
                         const uint32_t k4 = (uint32_t)kb * 4u;
                         xp = reinterpret_cast<const float *>(xrow + k4);
                         wp = reinterpret_cast<const float *>(wrows + (clamped_row_offset(row, last) + k4));
                     });
    } else if (live) {
        static_assert(COOP || GT == G, "the per-thread resolve scans groups of G");
        finish<LAYOUT, ARGS>(p, n_own, m_own, vmax, vmin, gmax, gmin);
    }
}


// The module's `splits` (mamtorch/nn/v4/fullyconnected.py:163-176): K is cut into consecutive ranges of
// `k_per_split` inputs (the last one shorter), every range is a MAM neuron of its own, and the layer's
// output is the sum of the ranges' (max + min) in ascending range order, then the bias -- the rounding
// order of the reference's `C_flat += ...` statements.  The forward kernels above run once with the ranges
// as their K ranges and leave (max, min, group) partials per range; this kernel resolves every range's
// extremes exactly (first index, sign of a zero) and adds them up.  argmax / argmin, when asked for, are
// [range][N*M] planes of ABSOLUTE k.
template <int LAYOUT, bool ARGS>
__global__ __launch_bounds__(256) void mam_fwd_range_sum_kernel(const Params p)
{
    const int64_t nm = (int64_t)p.N * p.M;
    const int patches_n = (p.N + 15) / 16;
    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    const int pm = logical / patches_n, pn = logical - pm * patches_n;
    const int n = pn * 16 + (threadIdx.x >> 4), m = pm * 16 + (threadIdx.x & 15);
    if (n >= p.N || m >= p.M) return;
    const int64_t o = (int64_t)n * p.M + m;
    const int stride = ARGS ? 3 : 2;
    float total = 0.0f;
    for (int s = 0; s < p.splits; ++s) {
        const float *base = p.part + (int64_t)s * stride * nm;
        float hi = base[o], lo = base[nm + o];
        const int kb = s * p.k_per_split;
        const int ke = (kb + p.k_per_split) < p.K ? (kb + p.k_per_split) : p.K;
        if (ARGS) {
            const int pk = __float_as_int(base[2 * nm + o]);
            int ih, il;
            float w_unused, x_unused;
            resolve<LAYOUT>(p, n, m, kb + (pk & 0xffff) * G, ke - 1, hi, false, hi, ih, w_unused, x_unused);
            resolve<LAYOUT>(p, n, m, kb + ((pk >> 16) & 0xffff) * G, ke - 1, lo, true, lo, il, w_unused, x_unused);
            p.argmax[(int64_t)s * nm + o] = ih;
            p.argmin[(int64_t)s * nm + o] = il;
        } else {
            if (hi == 0.0f) hi = first_zero_product<LAYOUT>(p.x + (int64_t)n * p.ldx, p.w, p.ldw, m, kb, ke);
            if (lo == 0.0f) lo = first_zero_product<LAYOUT>(p.x + (int64_t)n * p.ldx, p.w, p.ldw, m, kb, ke);
        }
        const float v = hi + lo;
        total = s == 0 ? v : total + v;
    }
    if (p.bias) total = total + p.bias[m];
    p.c[o] = total;
}

// ---------------------------------------------------------------------------------------------
// Second tiling for the (M,K) layout with K a multiple of 16 (64-k tiles, the last one may hold one to
// three 16-k groups): batch rows are wave-uniform.
//
// A wave owns 4 batch rows x 128 neurons (lane + 64 j): its x operands are the same for all
// lanes, so they come through the scalar cache into SGPRs (a VALU multiply takes one SGPR
// operand at no cost) and occupy no vector register and no LDS read.  LDS reads per product
// depend only on the rows per wave (one W value serves 4 products), not on the neurons per lane,
// so a thread holds just 8 outputs x (max, min, two group ids) + one W column of 16 k: ~100
// VGPRs, four waves per SIMD, and a wave that waits (LDS, barrier, scalar load) leaves three to
// issue from.  Eight waves = 32 batch rows share one W tile of 128 neurons x 64 k (32 KiB, two of
// them in flight, two workgroups per CU), one barrier per 64 k.  The tile is stored [neuron][k]
// without padding; 16-byte chunk c of neuron r sits at chunk c ^ (r & 15), which spreads a
// ds_read_b128 of 16 consecutive neurons over all banks, and since direct-to-LDS loads write LDS
// linearly the permutation is applied to the global addresses instead.
// Measured against the first tiling: 194 us against 216 us at the headline shape, 3.9 ms against
// 4.9 ms for the two ViT MLP layers.  Neurons per lane / tile depth of 4 / 32 gave the same
// headline time and 6 % more on the other shapes; reading the next W column ahead of its use
// changed nothing.
namespace sx {
constexpr int BN = 32;    // batch rows per workgroup
constexpr int NT = 512;   // threads per workgroup
constexpr int TI = 4;     // batch rows per wave
constexpr int KT = 64;    // k extent of one W tile
constexpr int CHUNKS = KT / 4;    // 16-byte chunks per neuron and tile
constexpr int RPB = 64 / KT < 1 ? 1 : 64 / KT;   // neurons per 256 bytes of LDS (all 64 banks)
// TJ = neurons per lane.  2 (128 neurons per workgroup) is what the launch uses.  Measured at the
// 256 x 4096 x 4096 shape: 1 (64 neurons per workgroup, 512 tiles, no split of K and no merge) 0.226 ms
// against 0.217 ms for 2 with K split in two plus the merge -- the k loop with one neuron per lane is 7 %
// slower (twice the scalar loads per product), which costs more than the merge; 4 with 32-k tiles: the
// same time at that shape and 6 % more on the large-batch shapes.
template <int TJ_>
struct Cfg {
    static constexpr int TJ = TJ_;
    static constexpr int BM = 64 * TJ;           // neurons per workgroup
    static constexpr int TILE_FLOATS = BM * KT;
    static constexpr int DMA_INSTR = TILE_FLOATS / 256;          // wave-level 1 KiB loads per tile
    static constexpr int DMA_PER_WAVE = DMA_INSTR / (NT / 64);
    static_assert(DMA_PER_WAVE * (NT / 64) == DMA_INSTR, "tile must split evenly over the waves");
    // the resolve scratch of the epilogue lives in the dead tiles when they are large enough
    static constexpr bool RES_IN_TILES = (NT / 64) * (TJ * 128 + 8 * 64) <= TILE_FLOATS;
};
constexpr int BM_MAX = Cfg<2>::BM;
}  // namespace sx

typedef const __attribute__((address_space(4))) float const_f32;

// TAIL: K (or the last K range) is a multiple of G = 16 but not of 64; the last tile is partial.  A separate
// instantiation, so that the whole-tile kernel stays exactly what it was.
// GT: products per recorded group.  G = 16 costs a compare and a select per extreme and 16 products; with
// GT = 32 the pair is issued after every second group (the running extremes of the first are kept as the
// baseline), which takes 64 of a tile's 1160 instructions off the k loop and doubles what the resolve scans
// per output: taken where the resolve is cheap next to the loop (K >= 2048), whole 64-k tiles only.
// FUSE (with SPLIT and ARGS): no merge kernel.  Every workgroup writes its partials and takes a ticket of its
// tile (an integer in the workspace, zero at launch); the workgroup that draws the last ticket of a tile finds
// all the tile's partials complete, combines them in ascending k with strict compares and resolves in its
// own epilogue, as the unsplit kernel does.
template <int TJ, bool ARGS, bool SPLIT, bool TAIL, int GT = G, bool FUSE = false>
__global__ __launch_bounds__(sx::NT, 4) void mam_fwd_sx_kernel(const Params p)
{
    using C = sx::Cfg<TJ>;
    __shared__ __attribute__((aligned(16))) float tile_a[C::TILE_FLOATS];
    __shared__ __attribute__((aligned(16))) float tile_b[C::TILE_FLOATS];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // ---- which tile: as in the first tiling ----
    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    const int tiles = p.tiles_n * p.tiles_m;
    const int split = logical / tiles;
    const int l = logical - split * tiles;
    const int per_group = p.group_n * p.tiles_m;
    const int grp = l / per_group;
    const int first_n = grp * p.group_n;
    const int gsize = (p.tiles_n - first_n) < p.group_n ? (p.tiles_n - first_n) : p.group_n;
    const int lin = l - grp * per_group;
    const int tn = first_n + lin % gsize;
    const int tm = lin / gsize;
    const int row0 = tn * sx::BN + sx::TI * wave, col0 = tm * C::BM;
    const int kb = split * p.k_per_split;
    const int ke = (kb + p.k_per_split) < p.K ? (kb + p.k_per_split) : p.K;
    const int ntiles = (ke - kb) / sx::KT;    // whole tiles; a rest of whole 16-k groups follows as a partial tile

    static_assert(GT == G || (GT == 2 * G && !TAIL), "tracking span");
    float vmax[sx::TI][TJ], vmin[sx::TI][TJ];
    float bmax[sx::TI][TJ], bmin[sx::TI][TJ];     // GT > G: the extremes before the first group of a span
    int gmax[sx::TI][TJ], gmin[sx::TI][TJ];
#pragma unroll
    for (int i = 0; i < sx::TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            vmax[i][j] = -__builtin_inff();
            vmin[i][j] = __builtin_inff();
            bmax[i][j] = vmax[i][j];
            bmin[i][j] = vmin[i][j];
            gmax[i][j] = 0;
            gmin[i][j] = 0;
        }

    // rows past the batch repeat the last one (never stored)
    const_f32 *xr[sx::TI];
#pragma unroll
    for (int i = 0; i < sx::TI; ++i) {
        const int row = (row0 + i) < p.N ? (row0 + i) : (p.N - 1);
        xr[i] = (const_f32 *)(p.x + (int64_t)row * p.ldx + kb);
    }

    // per-lane byte offsets of this wave's direct-to-LDS loads.  They stay in registers, and the
    // loads take them as the 32-bit offset of the (scalar base + vector offset) addressing form: formed
    // per lane in 64 bits, the addresses were 16 64-bit adds per tile.
    uint32_t doff[C::DMA_PER_WAVE];
#pragma unroll
    for (int t = 0; t < C::DMA_PER_WAVE; ++t) {
        const int inst = wave + (sx::NT / 64) * t;
        const int r = inst * (64 / sx::CHUNKS) + lane / sx::CHUNKS;   // neuron within the tile
        // the k chunk that belongs at this LDS position
        const int chunk = (lane % sx::CHUNKS) ^ ((r / sx::RPB) & (sx::CHUNKS - 1));
        const int rc = ((col0 + r) < p.M ? (col0 + r) : (p.M - 1)) - col0;
        doff[t] = (uint32_t)(rc * (int)p.ldw + chunk * 4) * 4u;
    }
    const int sw = (lane / sx::RPB) & (sx::CHUNKS - 1);   // the same for neurons lane + 64 j
    const int wbase = lane * sx::KT;     // floats; neuron lane + 64 j is 64 j * KT further

    auto dma = [&](const char *wk, float *tile) {
        asm volatile("" : "+s"(wk));     // one scalar base for the loads of this tile
#pragma unroll
        for (int t = 0; t < C::DMA_PER_WAVE; ++t) {
            const int inst = wave + (sx::NT / 64) * t;
            uint32_t off = doff[t];
            asm volatile("" : "+v"(off));    // keeps the zero-extension next to the load (no hoisted 64-bit copy)
            const char *src = wk + (uint64_t)off;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                             (__attribute__((address_space(3))) void *)(tile + inst * 256), 16, 0, 0);
        }
    };
    // The last tile of a K range that is not a multiple of 64 (but of G = 16): only its whole groups are
    // loaded (lanes whose 16-byte chunk lies past the range are switched off, so nothing past the end of a
    // weight row is read) and only they are computed.
    const int tail_groups = TAIL ? ((ke - kb) % sx::KT) / G : 0;
    const int nt_all = ntiles + (tail_groups ? 1 : 0);
    auto compute = [&](const float *tile, int t) {
        const int ng = (TAIL && t == ntiles) ? tail_groups : sx::KT / G;
#pragma unroll
        for (int gg = 0; gg < sx::KT / G; ++gg) {
            if (TAIL && gg >= ng) break;
            const int grel = (t * sx::KT + gg * G) / GT;       // the span this group belongs to
            const bool opens = (gg * G) % GT == 0, closes = ((gg + 1) * G) % GT == 0;
            float xv[sx::TI][G];
#pragma unroll
            for (int i = 0; i < sx::TI; ++i)
#pragma unroll
                for (int q = 0; q < G; ++q) xv[i][q] = xr[i][t * sx::KT + gg * G + q];
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                float wv[G];
#pragma unroll
                for (int q = 0; q < G / 4; ++q) {
                    const float4 v = *reinterpret_cast<const float4 *>(
                        &tile[wbase + 64 * j * sx::KT + (((gg * (G / 4) + q) ^ sw) << 2)]);
                    wv[q * 4 + 0] = v.x; wv[q * 4 + 1] = v.y; wv[q * 4 + 2] = v.z; wv[q * 4 + 3] = v.w;
                }
#pragma unroll
                for (int i = 0; i < sx::TI; ++i) {
                    if (GT > G && opens) { bmax[i][j] = vmax[i][j]; bmin[i][j] = vmin[i][j]; }
                    const float om = GT > G ? bmax[i][j] : vmax[i][j], on = GT > G ? bmin[i][j] : vmin[i][j];
                    float hi = vmax[i][j], lo = vmin[i][j];
#pragma unroll
                    for (int q = 0; q < G; q += 2) {
                        const float a = xv[i][q] * wv[q], b = xv[i][q + 1] * wv[q + 1];
                        hi = __builtin_fmaxf(__builtin_fmaxf(hi, a), b);
                        lo = __builtin_fminf(__builtin_fminf(lo, a), b);
                    }
                    if (ARGS && closes) {
                        gmax[i][j] = (hi > om) ? grel : gmax[i][j];
                        gmin[i][j] = (lo < on) ? grel : gmin[i][j];
                    }
                    vmax[i][j] = hi;
                    vmin[i][j] = lo;
                }
            }
        }
    };
    auto dma_any = [&](const char *wk, float *tile, int t) {
        if (!TAIL || t < ntiles) {
            dma(wk, tile);
        } else {
#pragma unroll
            for (int u = 0; u < C::DMA_PER_WAVE; ++u) {
                const int inst = wave + (sx::NT / 64) * u;
                const int r = inst * (64 / sx::CHUNKS) + lane / sx::CHUNKS;
                const int chunk = (lane % sx::CHUNKS) ^ ((r / sx::RPB) & (sx::CHUNKS - 1));
                if (chunk * 4 < tail_groups * G) {
                    const char *src = wk + (uint64_t)doff[u];
                    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                                     (__attribute__((address_space(3))) void *)(tile + inst * 256), 16, 0, 0);
                }
            }
        }
    };

    const char *wk = reinterpret_cast<const char *>(p.w + (int64_t)col0 * p.ldw + kb);
    if (nt_all > 0) {
        dma_any(wk, tile_a, 0);
        __syncthreads();
        for (int t = 0; t < nt_all; t += 2) {
            wk += sx::KT * sizeof(float);
            if (t + 1 < nt_all) dma_any(wk, tile_b, t + 1);
            compute(tile_a, t);
            __syncthreads();
            if (t + 1 >= nt_all) break;
            wk += sx::KT * sizeof(float);
            if (t + 2 < nt_all) dma_any(wk, tile_a, t + 2);
            compute(tile_b, t + 1);
            __syncthreads();
        }
    }

    // ---- epilogue ----
    // The epilogue's waves issue few instructions between long waits and share the CU with the k loop of the
    // other resident workgroup: served first, they finish sooner and the next workgroup starts its k loop sooner
    // (1.55 -> 1.48 ms at 12608 x 3072 -> 768, 3.13 -> 3.09 ms at 4096^3, no shape slower).
    __builtin_amdgcn_s_setprio(3);
    const int g0 = FUSE ? 0 : kb / GT;
    if (SPLIT) {
        const int64_t nm = (int64_t)p.N * p.M;
        float *base = p.part + (int64_t)split * (ARGS ? 3 : 2) * nm;
#pragma unroll
        for (int i = 0; i < sx::TI; ++i)
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                const int n = row0 + i, m = col0 + lane + 64 * j;
                if (n < p.N && m < p.M) {
                    const int64_t o = (int64_t)n * p.M + m;
                    if (FUSE) {
                        // device-coherent stores (they bypass the XCD's L2, which the other XCDs do not see):
                        // complete once the device can read them, so no cache write-back is needed before
                        // the ticket -- a device-scope release fence per workgroup (a write-back of the whole
                        // L2) made the call 0.385 instead of 0.207 ms
                        __hip_atomic_store(base + o, vmax[i][j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(base + nm + o, vmin[i][j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(base + 2 * nm + o, __int_as_float(gmax[i][j] | (gmin[i][j] << 16)),
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    } else {
                        base[o] = vmax[i][j];
                        base[nm + o] = vmin[i][j];
                        if (ARGS) base[2 * nm + o] = __int_as_float(gmax[i][j] | (gmin[i][j] << 16));
                    }
                }
            }
        if (FUSE) {
            __shared__ int s_last;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");     // every wave's stores have completed ...
            __syncthreads();                                            // ... before the ticket is drawn
            if (tid == 0) {
                const int drawn = __hip_atomic_fetch_add(&p.tickets[l], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                s_last = drawn == p.splits - 1;
            }
            __syncthreads();
            if (!s_last) return;
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            const int gps = p.k_per_split / GT;
#pragma unroll
            for (int i = 0; i < sx::TI; ++i)
#pragma unroll
                for (int j = 0; j < TJ; ++j) {
                    const int n = row0 + i, m = col0 + lane + 64 * j;
                    float hi = -__builtin_inff(), lo = __builtin_inff();
                    int gh = 0, gl = 0;
                    if (n < p.N && m < p.M) {
                        const int64_t o = (int64_t)n * p.M + m;
                        for (int sp = 0; sp < p.splits; ++sp) {
                            const float *b2 = p.part + (int64_t)sp * 3 * nm;
                            const float h2 = __hip_atomic_load(b2 + o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            const float l2 = __hip_atomic_load(b2 + nm + o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            const int pk = __float_as_int(
                                __hip_atomic_load(b2 + 2 * nm + o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                            if (sp == 0 || h2 > hi) { hi = h2; gh = sp * gps + (pk & 0xffff); }
                            if (sp == 0 || l2 < lo) { lo = l2; gl = sp * gps + ((pk >> 16) & 0xffff); }
                        }
                    }
                    vmax[i][j] = hi; vmin[i][j] = lo; gmax[i][j] = gh; gmin[i][j] = gl;
                }
        }
    }
    if (SPLIT && !FUSE) {
    } else if (ARGS) {
        // A wave parks one batch row (4 sets of 64 neurons) in its own corner of the dead tiles
        // and resolves it set by set; the 64 outputs of a set share their x row.
        float *vals = tile_a + wave * (TJ * 128);
        int *grps = reinterpret_cast<int *>(tile_b) + wave * (TJ * 128);
        static_assert((sx::NT / 64) * (TJ * 128) <= C::TILE_FLOATS, "result stash does not fit a tile buffer");
        static_assert(RES_WORDS == 8 * 64, "C::RES_IN_TILES assumes this size");
        __shared__ float res_own[C::RES_IN_TILES ? 1 : (sx::NT / 64) * RES_WORDS];
        float *res = C::RES_IN_TILES ? tile_a + (sx::NT / 64) * (TJ * 128) + wave * RES_WORDS
                                      : res_own + wave * RES_WORDS;
        // From here on a wave touches only its own corner of LDS, and the LDS operations of one wave
        // complete in issue order: no workgroup barrier between parking and resolving.
        __syncthreads();
#pragma unroll
        for (int i = 0; i < sx::TI; ++i) {
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                vals[(j * 2 + 0) * 64 + lane] = vmax[i][j];
                vals[(j * 2 + 1) * 64 + lane] = vmin[i][j];
                grps[(j * 2 + 0) * 64 + lane] = g0 + gmax[i][j];
                grps[(j * 2 + 1) * 64 + lane] = g0 + gmin[i][j];
            }
            __builtin_amdgcn_wave_barrier();
            const int nrow = row0 + i;
            // the 64 outputs of a set share the x row, and their w rows are mbase + slot: 32-bit byte
            // offsets from two wave-uniform bases (the host checked that a tile of w spans < 4 GiB)
            const char *xrow = reinterpret_cast<const char *>(p.x + (int64_t)(nrow < p.N ? nrow : p.N - 1) * p.ldx);
            const uint32_t ldw4 = (uint32_t)p.ldw * 4u;
#pragma unroll 1
            for (int j = 0; j < TJ; ++j) {
                const int mbase = col0 + 64 * j;
                const int mb = mbase < p.M ? mbase : p.M - 1;
                const char *wrows = reinterpret_cast<const char *>(p.w + (int64_t)mb * p.ldw);
                const uint32_t last = last_row_offset(p.M, mb, 64, ldw4);   // neurons past M repeat the last one
                const uint32_t mine = (uint32_t)(lane >> 3) * ldw4;         // slot = 8 r + lane / 8
                resolve_wave<GT>(p, vals + j * 128, grps + j * 128, res, lane,
                             [&](int slot, int &n, int &m, bool &valid) {
                                 n = nrow;
                                 m = mbase + slot;
                                 valid = n < p.N && m < p.M;
                                 n = n < p.N ? n : p.N - 1;
                                 m = m < p.M ? m : p.M - 1;
                             },
                             [&](int r, int, int, int kb, const float *&xp, const float *&wp) {
                                 const uint32_t row = mine + (uint32_t)(8 * r) * ldw4;
                                 const uint32_t k4 = (uint32_t)kb * 4u;
                                 xp = reinterpret_cast<const float *>(xrow + k4);
                                 wp = reinterpret_cast<const float *>(wrows + (clamped_row_offset(row, last) + k4));
                             });
            }
        }
    } else {
        // values only: every thread parks its 16 results in its own LDS slots so that finishing them
        // is one rolled loop (one copy of the code, no register array indexed at run time)
        static_assert(sx::TI * TJ * sx::NT <= C::TILE_FLOATS, "result stash does not fit a tile buffer");
        float *smax = tile_a + tid, *smin = tile_b + tid;
#pragma unroll
        for (int i = 0; i < sx::TI; ++i)
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                smax[(i * TJ + j) * sx::NT] = vmax[i][j];
                smin[(i * TJ + j) * sx::NT] = vmin[i][j];
            }
#pragma unroll 1
        for (int o = 0; o < sx::TI * TJ; ++o) {
            const int n = row0 + o / TJ, m = col0 + lane + 64 * (o % TJ);
            if (n < p.N && m < p.M) {
                float hi = smax[o * sx::NT], lo = smin[o * sx::NT];
                if (hi == 0.0f || lo == 0.0f) {
                    // a zero extreme carries the sign of the first zero product (rare: plain scan)
                    const float *xrow = p.x + (int64_t)n * p.ldx, *wrow = p.w + (int64_t)m * p.ldw;
                    float z = 0.0f;
                    for (int k = 0; k < p.K; ++k) {
                        const float prod = xrow[k] * wrow[k];
                        if (prod == 0.0f) { z = prod; break; }
                    }
                    hi = hi == 0.0f ? z : hi;
                    lo = lo == 0.0f ? z : lo;
                }
                float sum = hi + lo;
                if (p.bias) sum = sum + p.bias[m];
                p.c[(int64_t)n * p.M + m] = sum;
            }
        }
    }
}

// How many K ranges to split into so that at least two workgroups reach every CU.
static int choose_splits(int64_t N, int64_t K, int64_t M, int bn = BN, int bm = BM)
{
    const int64_t tiles = ceil_div(N, bn) * ceil_div(M, bm);
    const int64_t want = 2 * num_cus();
    if (tiles >= want) return 1;
    int64_t s = ceil_div(want, tiles);
    const int64_t max_by_k = K / (8 * KT);  // keep at least 256 k per split
    if (s > max_by_k) {
        // Small calls, where ranges of 256 k leave most CUs idle: ranges of 128 k as long as that puts at most one
        // workgroup on a CU (the call's time is then the length of one workgroup's k loop plus the two launches:
        // 24.4 -> 18.3 us at 64 x 784 x 256, 23.0 -> 20.3 us at 64 x 2048 x 512; beyond one workgroup per CU the
        // extra partials cost more than the shorter loops gain: 29.9 -> 33.5 us at 256 x 1024 x 1024).
        int64_t fine = K / (4 * KT);
        if (fine > s) fine = s;
        if (fine > num_cus() / tiles) fine = num_cus() / tiles;
        s = fine > max_by_k ? fine : max_by_k;
    }
    if (s > MAX_SPLITS) s = MAX_SPLITS;
    if (s < 1) s = 1;
    // partial group ids are 16-bit offsets within a split
    if (s > 1 && ceil_div(ceil_div(K, s), KT) * KT / G > 65536) s = 1;
    return (int)s;
}

static size_t workspace_bytes(int64_t N, int64_t K, int64_t M, bool args)
{
    // whichever tiling the launch picks (it depends on alignment, unknown here): the larger need
    const int s1 = choose_splits(N, K, M), s2 = choose_splits(N, K, M, sx::BN, sx::BM_MAX);
    const int s = s1 > s2 ? s1 : s2;
    if (s == 1) return 0;
    size_t tickets = 0;     // of the fused merge, one per tile of the finer tiling
    if (option(MAM_OPT_FORWARD_TILING) == MAM_FORWARD_TILING_FUSED_MERGE)
        tickets = ((size_t)(ceil_div(N, sx::BN) * ceil_div(M, BM)) * sizeof(int) + 255) / 256 * 256;
    return (size_t)s * (args ? 3 : 2) * (size_t)N * (size_t)M * sizeof(float) + tickets;
}

// ---- the entry point that allocates nothing: split-K partials in a file-scope device array ----
// Each GPU the library runs on holds its own copy of the array until the process ends.  Its name is a
// host-side stand-in, not a device address: the device's set-up asks the runtime for the address once,
// and only that pointer is handed to kernels.
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;
static __device__ __attribute__((used)) __align__(256) unsigned char scratch[kStaticScratchBytes];
static void *g_scratch[kMaxDevices];

static int setup_device(int dev)
{
    void *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
        (void)hipGetLastError();
        g_scratch[dev] = nullptr;   // mam_fc_forward_static reports it; the other entry points do not need it
        return MAM_OK;
    }
    g_scratch[dev] = ptr;
    return MAM_OK;
}
static DeviceHookRegistration g_registration(setup_device);
static size_t static_scratch_bytes() { return kStaticScratchBytes; }
static void *static_scratch_of(int dev) { return g_scratch[dev]; }

// What a call will do: the kernel parameters, which tiling serves it, and the bytes of split-K partials.
struct Plan {
    Params p;
    bool use_sx;
    size_t need;          // workspace bytes: the partials, then the tickets of the fused merge
    size_t tickets_at;    // offset of the tickets
};

static int make_plan(Plan &plan, bool args, const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                     const float *bias, float *c, int32_t *argmax, int32_t *argmin, float *w_sel, float *x_sel,
                     int64_t N, int64_t K, int64_t M, int64_t range_len = 0)
{
    if (N < 0 || K < 0 || M < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (w_layout != MAM_W_KM && w_layout != MAM_W_MK)
        return fail(MAM_ERR_INVALID_ARGUMENT, "w_layout must be MAM_W_KM or MAM_W_MK");
    if (N == 0 || M == 0) return MAM_OK;
    if (K == 0) return fail(MAM_ERR_INVALID_ARGUMENT, "K == 0: max/min over an empty set");
    if (ldx < K || ldw < (w_layout == MAM_W_MK ? K : M))
        return fail(MAM_ERR_INVALID_ARGUMENT, "leading dimension smaller than the row length");
    if (N > INT32_MAX / 2 || K > INT32_MAX / 2 || M > INT32_MAX / 2)
        return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");

    Params &p = plan.p;
    p.x = x; p.ldx = ldx; p.w = w; p.ldw = ldw; p.bias = bias;
    p.c = c; p.argmax = argmax; p.argmin = argmin; p.wsel = w_sel; p.xsel = x_sel;
    p.N = (int)N; p.K = (int)K; p.M = (int)M;
    p.vec_x = (ldx % 4 == 0) && ((uintptr_t)x % 16 == 0);
    p.vec_w = (ldw % 4 == 0) && ((uintptr_t)w % 16 == 0);
    // The wave-uniform-rows tiling takes (M,K) weights with aligned rows and K a multiple of 16; option
    // MAM_OPT_FORWARD_TILING = MAM_FORWARD_TILING_WIDE keeps every shape on the first tiling (for
    // comparisons and tests).
    // (range_len > 0: the caller fixes the K ranges -- the module's `splits` -- instead of the launch
    // heuristics; the wave-uniform-rows tiling then also needs whole 64-k tiles per range)
    const bool use_sx = (w_layout == MAM_W_MK) && p.vec_x && p.vec_w && (K % G == 0) &&
                        (range_len % sx::KT == 0) && (ldw * sx::BM_MAX < (1ll << 30)) &&
                        option(MAM_OPT_FORWARD_TILING) != MAM_FORWARD_TILING_WIDE;
    plan.use_sx = use_sx;
    const int bn = use_sx ? sx::BN : BN, bm = use_sx ? sx::BM_MAX : BM;
    p.tiles_n = (int)ceil_div(N, bn);
    p.tiles_m = (int)ceil_div(M, bm);
    // Tile order: GROUP_N row tiles are swept under one W panel, panel after panel.  An XCD has 64 tiles in
    // flight; with fewer than 8 panels a group of 8 row tiles is shorter than that and the window straddles
    // groups, every panel of W in flight at once.  Groups of 64 row tiles keep one panel at a time there
    // (12608 x 3072 -> 768, 6 panels: 1.585 -> 1.517 ms; with 8 or more panels groups of 16 to 128 row tiles
    // change nothing or lose: 16384 x 4096 -> 1024 3.13 -> 3.29 ms at 64).
    p.group_n = p.tiles_m < 8 ? 8 * GROUP_N : GROUP_N;
    if (range_len > 0) {
        p.k_per_split = (int)(range_len < K ? range_len : K);
    } else {
        p.splits = choose_splits(N, K, M, bn, bm);
        const int kt = use_sx ? sx::KT : KT;
        p.k_per_split = (int)(ceil_div(ceil_div(K, p.splits), kt) * kt);
    }
    p.splits = (int)ceil_div(K, p.k_per_split);
    p.part = nullptr;
    plan.need = p.splits > 1 ? (size_t)p.splits * (args ? 3 : 2) * (size_t)N * (size_t)M * sizeof(float) : 0;
    // the fused merge keeps one ticket per tile behind the partials
    plan.tickets_at = plan.need;
    if (p.splits > 1 && option(MAM_OPT_FORWARD_TILING) == MAM_FORWARD_TILING_FUSED_MERGE)
        plan.need += ((size_t)p.tiles_n * p.tiles_m * sizeof(int) + 255) / 256 * 256;
    // the fast staging path addresses a tile with 32-bit element offsets from the tile base
    const int64_t w_rows = (w_layout == MAM_W_MK) ? fwd::BM : fwd::KT;
    // (and the first k of every K range has to be 16-byte aligned)
    p.fast = p.vec_x && p.vec_w && (ldx * fwd::BN < (1ll << 30)) && (ldw * w_rows < (1ll << 30)) &&
             (p.k_per_split % 4 == 0);
    // (64 rows of w within 4 GiB: the merge kernel addresses a patch's operands by 32-bit offsets)
    p.coop = (w_layout == MAM_W_MK) && p.vec_x && p.vec_w && (K % G == 0) && (ldw < (1ll << 24));
    // two groups per recorded span where the resolve is cheap next to the k loop (see mam_fwd_sx_kernel)
    p.gt = (args && use_sx && range_len == 0 && K >= 2048 && K % sx::KT == 0 && p.k_per_split % sx::KT == 0 &&
            option(MAM_OPT_FORWARD_TILING) != MAM_FORWARD_TILING_GROUPS16) ? 2 * G : G;
    // group ids are kept as 16-bit offsets from the first group of a workgroup's k range
    if ((int64_t)p.k_per_split / G > 65536)
        return fail(MAM_ERR_UNSUPPORTED, "K = %lld exceeds %d per K range", (long long)K, 65536 * G);
    return MAM_OK;
}

// Whether to transpose a (K, M) operand once and run the (M, K) tilings on the copy: two more passes
// over the weight against a kernel that is 1.7 times as fast per triple.  Measured, (K, M) operand as it
// is / transposed first / the same weight given as (M, K): 0.371 / 0.240 / 0.221 ms at 256 x 4096 x 4096,
// 0.160 / 0.086 / 0.070 ms at batch 64, 5.58 / 3.22 / 3.22 ms at 16384 x 4096 x 1024.
static bool transposed_operand_pays(int64_t N, int64_t K, int64_t M)
{
    (void)K;
    (void)M;
    return N >= 16 && option(MAM_OPT_FORWARD_TILING) != MAM_FORWARD_TILING_WIDE;
}

template <bool ARGS>
static int launch(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                  const float *bias, float *c, int32_t *argmax, int32_t *argmin, float *w_sel, float *x_sel,
                  int64_t N, int64_t K, int64_t M, void *workspace, size_t workspace_size, void *stream,
                  bool static_scratch = false, int64_t range_len = 0)
{
    Plan plan;
    int rc = make_plan(plan, ARGS, x, ldx, w, ldw, w_layout, bias, c, argmax, argmin, w_sel, x_sel, N, K, M,
                       range_len);
    if (rc != MAM_OK || N == 0 || M == 0) return rc;
    if (!x || !w || !c || (ARGS && (!argmax || !argmin)))
        return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    const size_t avail = static_scratch ? static_scratch_bytes() : (workspace ? workspace_size : (size_t)0);
    // The operand b of the reference operators is (K, M).  The general tiling takes it as it is and
    // transposes every tile through registers (0.37 ms at the 256 x 4096 x 4096 shape).  When the
    // workspace has room, b is transposed ONCE into it and the wave-uniform-rows tiling runs on the copy
    // (0.22 ms + the transpose): every output is the same, bit for bit.
    size_t wt_bytes = 0;
    if (w_layout == MAM_W_KM && transposed_operand_pays(N, K, M)) {
        Plan tplan;
        float *const aligned = reinterpret_cast<float *>((uintptr_t)256);   // stands in for the workspace
        const int trc = make_plan(tplan, ARGS, x, ldx, aligned, K, MAM_W_MK, bias, c, argmax, argmin, w_sel, x_sel,
                                  N, K, M, range_len);
        const size_t bytes = ((size_t)M * (size_t)K * sizeof(float) + 255) / 256 * 256;
        if (trc == MAM_OK && tplan.use_sx && bytes + tplan.need <= avail &&
            (static_scratch || (uintptr_t)workspace % 16 == 0)) {
            plan = tplan;
            wt_bytes = bytes;
            w_layout = MAM_W_MK;
        }
    }
    Params &p = plan.p;
    const bool use_sx = plan.use_sx;
    const size_t need = plan.need;
    if (static_scratch) {
        if (wt_bytes + need > static_scratch_bytes())
            return fail(MAM_ERR_UNSUPPORTED,
                        "this shape needs %zu bytes of split-K partials, the built-in scratch array holds %zu; "
                        "use mam_fc_forward with a workspace", need, static_scratch_bytes());
    } else if (wt_bytes + need > 0) {
        if (!workspace || workspace_size < wt_bytes + need)
            return fail(MAM_ERR_WORKSPACE, "forward needs %zu workspace bytes, got %zu", need,
                        workspace ? workspace_size : (size_t)0);
    }

    const int64_t nblk = (int64_t)p.tiles_n * p.tiles_m * p.splits;
    if (nblk > INT32_MAX) return fail(MAM_ERR_UNSUPPORTED, "too many tiles");
    const int dev = ensure_device(static_cast<hipStream_t>(stream));
    if (dev < 0) return dev;
    char *scratch_base = static_cast<char *>(workspace);
    if (static_scratch && wt_bytes + need > 0) {
        scratch_base = static_cast<char *>(static_scratch_of(dev));
        if (!scratch_base) return fail(MAM_ERR_LAUNCH, "the built-in scratch array has no device address");
    }
    if (need > 0) p.part = reinterpret_cast<float *>(scratch_base + wt_bytes);
    hipStream_t st = static_cast<hipStream_t>(stream);
    // the merge inside the forward launch (option MAM_FORWARD_TILING_FUSED_MERGE): whole 64-k tiles, spans of 32
    const bool tail_k = K % sx::KT != 0;
    const bool fuse = ARGS && use_sx && p.splits > 1 && !tail_k && p.gt == 2 * G && p.coop && range_len == 0 &&
                      option(MAM_OPT_FORWARD_TILING) == MAM_FORWARD_TILING_FUSED_MERGE;
    if (fuse) {
        p.tickets = reinterpret_cast<int *>(scratch_base + wt_bytes + plan.tickets_at);
        rc = fill_zero(p.tickets, (int64_t)p.tiles_n * p.tiles_m, st);
        if (rc != MAM_OK) return rc;
    }
    if (wt_bytes > 0) {
        float *wt = reinterpret_cast<float *>(scratch_base);
        rc = transpose(w, ldw, wt, K, M, st);
        if (rc != MAM_OK) return rc;
        p.w = wt;
    }
    const bool tail = K % sx::KT != 0;
    if (fuse)
        hipLaunchKernelGGL((mam_fwd_sx_kernel<2, ARGS, true, false, ARGS ? 2 * G : G, ARGS>), dim3((unsigned)nblk), dim3(sx::NT), 0, st, p);
    else if (use_sx && p.splits > 1 && tail)
        hipLaunchKernelGGL((mam_fwd_sx_kernel<2, ARGS, true, true>), dim3((unsigned)nblk), dim3(sx::NT), 0, st, p);
    else if (use_sx && p.splits > 1 && ARGS && p.gt == 2 * G)
        hipLaunchKernelGGL((mam_fwd_sx_kernel<2, ARGS, true, false, ARGS ? 2 * G : G>), dim3((unsigned)nblk), dim3(sx::NT), 0, st, p);
    else if (use_sx && p.splits > 1)
        hipLaunchKernelGGL((mam_fwd_sx_kernel<2, ARGS, true, false>), dim3((unsigned)nblk), dim3(sx::NT), 0, st, p);
    else if (use_sx && tail)
        hipLaunchKernelGGL((mam_fwd_sx_kernel<2, ARGS, false, true>), dim3((unsigned)nblk), dim3(sx::NT), 0, st, p);
    else if (use_sx && ARGS && p.gt == 2 * G)
        hipLaunchKernelGGL((mam_fwd_sx_kernel<2, ARGS, false, false, ARGS ? 2 * G : G>), dim3((unsigned)nblk), dim3(sx::NT), 0, st, p);
    else if (use_sx)
        hipLaunchKernelGGL((mam_fwd_sx_kernel<2, ARGS, false, false>), dim3((unsigned)nblk), dim3(sx::NT), 0, st, p);
    else if (w_layout == MAM_W_MK)
        hipLaunchKernelGGL((mam_fwd_kernel<MAM_W_MK, ARGS>), dim3((unsigned)nblk), dim3(NT), 0, st, p);
    else
        hipLaunchKernelGGL((mam_fwd_kernel<MAM_W_KM, ARGS>), dim3((unsigned)nblk), dim3(NT), 0, st, p);
    rc = check_launch("mam_fwd_kernel");
    if (rc != MAM_OK) return rc;
    if (p.splits > 1 && range_len > 0) {
        // the caller's ranges are neurons of their own: resolve each and add them up
        const unsigned mb = (unsigned)(ceil_div(N, 16) * ceil_div(M, 16));
        if (w_layout == MAM_W_MK)
            hipLaunchKernelGGL((mam_fwd_range_sum_kernel<MAM_W_MK, ARGS>), dim3(mb), dim3(256), 0, st, p);
        else
            hipLaunchKernelGGL((mam_fwd_range_sum_kernel<MAM_W_KM, ARGS>), dim3(mb), dim3(256), 0, st, p);
        rc = check_launch("mam_fwd_range_sum_kernel");
    } else if (p.splits > 1 && !fuse) {
        // 16 x 16 patches; 4 x 64 with the cooperative resolve
        const unsigned mb = (ARGS && p.coop) ? (unsigned)(ceil_div(N, 4) * ceil_div(M, 64))
                                             : (unsigned)(ceil_div(N, 16) * ceil_div(M, 16));
        if (ARGS && p.coop && p.gt == 2 * G)
            hipLaunchKernelGGL((mam_fwd_merge_kernel<MAM_W_MK, ARGS, ARGS, ARGS ? 2 * G : G>), dim3(mb), dim3(256), 0, st, p);
        else if (ARGS && p.coop)
            hipLaunchKernelGGL((mam_fwd_merge_kernel<MAM_W_MK, ARGS, ARGS>), dim3(mb), dim3(256), 0, st, p);
        else if (w_layout == MAM_W_MK)
            hipLaunchKernelGGL((mam_fwd_merge_kernel<MAM_W_MK, ARGS, false>), dim3(mb), dim3(256), 0, st, p);
        else
            hipLaunchKernelGGL((mam_fwd_merge_kernel<MAM_W_KM, ARGS, false>), dim3(mb), dim3(256), 0, st, p);
        rc = check_launch("mam_fwd_merge_kernel");
    }
    return rc;
}

// Every word of the partials that the merge reads is written by the same call's first kernel: nothing in
// the array has to be cleared between calls.
static int launch_static(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout, const float *bias,
                         float *c, int32_t *argmax, int32_t *argmin, float *w_sel, float *x_sel, int64_t N,
                         int64_t K, int64_t M, void *stream)
{
    return launch<true>(x, ldx, w, ldw, w_layout, bias, c, argmax, argmin, w_sel, x_sel, N, K, M, nullptr, 0, stream,
                        true);
}

}  // namespace fwd
}  // namespace mam

extern "C" size_t mam_fc_forward_workspace_for(int64_t N, int64_t K, int64_t M, int w_layout, int with_indices)
{
    if (N <= 0 || K <= 0 || M <= 0) return 0;
    size_t bytes = mam::fwd::workspace_bytes(N, K, M, with_indices != 0);
    // room for the transposed copy of a (K, M) operand (see launch); without it the call still works
    if (w_layout == MAM_W_KM && K % mam::fwd::G == 0 && mam::fwd::transposed_operand_pays(N, K, M))
        bytes += ((size_t)M * (size_t)K * sizeof(float) + 255) / 256 * 256;
    return bytes;
}

extern "C" size_t mam_fc_forward_ranges_workspace(int64_t N, int64_t K, int64_t M, int64_t range_len, int with_indices)
{
    if (N <= 0 || K <= 0 || M <= 0 || range_len <= 0 || range_len >= K) return 0;
    const size_t ranges = (size_t)((K + range_len - 1) / range_len);
    return ranges * (with_indices ? 3 : 2) * (size_t)N * (size_t)M * sizeof(float);
}

extern "C" int mam_fc_forward_ranges(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                                     const float *bias, float *c, int32_t *argmax, int32_t *argmin, int64_t N,
                                     int64_t K, int64_t M, int64_t range_len, void *workspace, size_t workspace_bytes,
                                     void *stream)
{
    using namespace mam;
    if (range_len <= 0) return fail(MAM_ERR_INVALID_ARGUMENT, "range_len must be positive");
    if ((argmax == nullptr) != (argmin == nullptr))
        return fail(MAM_ERR_INVALID_ARGUMENT, "argmax and argmin go together");
    if (K > 0 && (K + range_len - 1) / range_len > 65535) return fail(MAM_ERR_UNSUPPORTED, "more than 65535 ranges");
    if (argmax)
        return fwd::launch<true>(x, ldx, w, ldw, w_layout, bias, c, argmax, argmin, nullptr, nullptr, N, K, M, workspace,
                                 workspace_bytes, stream, false, range_len);
    return fwd::launch<false>(x, ldx, w, ldw, w_layout, bias, c, nullptr, nullptr, nullptr, nullptr, N, K, M, workspace,
                              workspace_bytes, stream, false, range_len);
}

static void describe_plan(const mam::fwd::Plan &plan, int w_layout, int64_t K, bool with_indices, char *text,
                          size_t text_bytes)
{
    using namespace mam;
    const fwd::Params &p = plan.p;
    const char *what = with_indices ? "args" : "values";
    if (plan.use_sx)
        snprintf(text, text_bytes, "mam_fwd_sx_kernel<%s%s%s%s> %d x %d tiles of 32 x 128", what, p.splits > 1 ? ", split" : "",
                 K % fwd::sx::KT != 0 ? ", partial last k tile" : "", p.gt > fwd::G ? ", indices per 32 k" : "", p.tiles_n,
                 p.tiles_m);
    else
        snprintf(text, text_bytes, "mam_fwd_kernel<%s, %s> %d x %d tiles of 64 x 128", w_layout == MAM_W_MK ? "(M,K)" : "(K,M)",
                 what, p.tiles_n, p.tiles_m);
    if (p.splits > 1) {
        const size_t used = strlen(text);
        snprintf(text + used, text_bytes - used, " x %d ranges of %d k + mam_fwd_merge_kernel<%s> (%zu bytes of partials)",
                 p.splits, p.k_per_split, (with_indices && p.coop) ? "cooperative resolve" : "per-thread resolve",
                 plan.need);
    }
}

extern "C" int mam_fc_forward_describe(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                                       int64_t N, int64_t K, int64_t M, int with_indices, char *text, size_t text_bytes)
{
    using namespace mam;
    fwd::Plan plan;
    const int rc = fwd::make_plan(plan, with_indices != 0, x, ldx, w, ldw, w_layout, nullptr, nullptr, nullptr,
                                  nullptr, nullptr, nullptr, N, K, M);
    if (rc != MAM_OK) return rc;
    if (!text || text_bytes == 0) return fail(MAM_ERR_INVALID_ARGUMENT, "no text buffer");
    if (N == 0 || M == 0) {
        snprintf(text, text_bytes, "nothing to launch");
        return MAM_OK;
    }
    // A (K, M) operand is transposed once into the workspace when that has room (what
    // mam_fc_forward_workspace_for() asks for) and the wave-uniform-rows tiling then runs on the copy: both
    // routes are named, the one a call takes depends on the workspace it brings.
    if (w_layout == MAM_W_KM && fwd::transposed_operand_pays(N, K, M)) {
        fwd::Plan tplan;
        float *const aligned = reinterpret_cast<float *>((uintptr_t)256);
        const int trc = fwd::make_plan(tplan, with_indices != 0, x, ldx, aligned, K, MAM_W_MK, nullptr, nullptr,
                                       nullptr, nullptr, nullptr, nullptr, N, K, M);
        if (trc == MAM_OK && tplan.use_sx) {
            const size_t copy = ((size_t)M * (size_t)K * sizeof(float) + 255) / 256 * 256;
            int used = snprintf(text, text_bytes, "with %zu workspace bytes: transpose_kernel + ", copy + tplan.need);
            if (used < 0 || (size_t)used >= text_bytes) return MAM_OK;
            describe_plan(tplan, MAM_W_MK, K, with_indices != 0, text + used, text_bytes - used);
            used = (int)strlen(text);
            const int more = snprintf(text + used, text_bytes - used, "; with less: ");
            if (more < 0 || (size_t)(used + more) >= text_bytes) return MAM_OK;
            describe_plan(plan, w_layout, K, with_indices != 0, text + used + more, text_bytes - used - more);
            return MAM_OK;
        }
    }
    describe_plan(plan, w_layout, K, with_indices != 0, text, text_bytes);
    return MAM_OK;
}

extern "C" size_t mam_fc_forward_static_limit(void) { return mam::fwd::kStaticScratchBytes; }

extern "C" int mam_fc_forward_static(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                                     const float *bias, float *c, int32_t *argmax, int32_t *argmin,
                                     float *w_sel, float *x_sel, int64_t N, int64_t K, int64_t M, void *stream)
{
    return mam::fwd::launch_static(x, ldx, w, ldw, w_layout, bias, c, argmax, argmin, w_sel, x_sel, N, K, M, stream);
}

extern "C" size_t mam_fc_forward_workspace(int64_t N, int64_t K, int64_t M)
{
    if (N <= 0 || K <= 0 || M <= 0) return 0;
    return mam::fwd::workspace_bytes(N, K, M, true);
}

extern "C" size_t mam_fc_forward_values_workspace(int64_t N, int64_t K, int64_t M)
{
    if (N <= 0 || K <= 0 || M <= 0) return 0;
    return mam::fwd::workspace_bytes(N, K, M, false);
}

extern "C" int mam_fc_forward(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                              const float *bias, float *c, int32_t *argmax, int32_t *argmin,
                              float *w_sel, float *x_sel, int64_t N, int64_t K, int64_t M,
                              void *workspace, size_t workspace_bytes, void *stream)
{
    return mam::fwd::launch<true>(x, ldx, w, ldw, w_layout, bias, c, argmax, argmin, w_sel, x_sel, N, K, M,
                                  workspace, workspace_bytes, stream);
}

extern "C" int mam_fc_forward_values(const float *x, int64_t ldx, const float *w, int64_t ldw,
                                     int w_layout, const float *bias, float *c, int64_t N, int64_t K,
                                     int64_t M, void *workspace, size_t workspace_bytes, void *stream)
{
    return mam::fwd::launch<false>(x, ldx, w, ldw, w_layout, bias, c, nullptr, nullptr, nullptr, nullptr, N, K, M,
                                   workspace, workspace_bytes, stream);
}
