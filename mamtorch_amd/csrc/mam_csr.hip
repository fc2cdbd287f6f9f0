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
// Forward: lanes are batch rows.  x is first transposed into the workspace, xT (K, ldt), so that the
// x column of a stored entry is contiguous over the batch.  A wave owns one CSR row (output
// neuron) for a tile of 64*TI batch rows: column indices and values of the row are wave-uniform
// (scalar loads), each entry costs one coalesced vector load of xT[col] and TI multiplies; two
// entries fold into the running extremes with one v_max3 / v_min3 each, and per PAIR of entries and
// extreme one strict compare with two selects records the pair and its first product, from which
// the entry is settled after the loop (first product equals the extreme: first entry, else second).
// Measured, 4096 x 4096 weight at 10 % / 3 % / 1 % density, batch 256: 89 / 40 / 26 us against
// 109 / 45 / 27 us with a compare and two selects per product; batch tiles of 64 rows per wave
// instead of 256 were slower at all three (131 / 50 / 28 us); 4 or 16 entries in flight per buffer
// instead of 8 changed nothing or spilled.  Timing-only builds at 10 %: the loads alone (arithmetic
// removed) 95 us, the arithmetic alone (every load hitting one L1-resident row) 78 us, together
// 90 us: the kernel sits on the vector memory path (1.7 GB of x values per call, half of them L1
// hits, at about half of the path's 64 bytes per clock and CU) with the arithmetic hidden under it.
// The lowest column missing from the row is found once per row; the
// implicit-zero candidate x[n, missing] * 0 is compared last under the dense rule (greater wins,
// equal -> lower index wins).  The 16 waves of a workgroup own 16 consecutive neurons and hand
// their results over through LDS so that every batch row stores 64 contiguous bytes per array.
//
// Backward: when the forward handed over the selected values and their entry positions, x_grad is the
// dense x_grad kernel fed with those values (an implicit zero contributes 0), and val_grad is
// accumulated by workgroups that own 8 consecutive CSR rows: an LDS histogram over the rows'
// entries, streamed out once, no atomics in global memory and no zero fill.  Without the hand-over:
// one workgroup per batch row; selected columns are located in the CSR row by binary search,
// x_grad is accumulated in an LDS histogram and stored once, val_grad takes global atomic adds (at
// most N contenders per entry).
#include "mam_common.h"
#include "mam_fixed.h"

namespace mam {
namespace csr {

constexpr int NT = 256;
constexpr int NT_B = 512;  // backward workgroup
constexpr int EG = 8;      // entries whose loads are issued together
constexpr int NT_F = 1024;      // forward workgroup
constexpr int ROWS = NT_F / 64;  // CSR rows per forward workgroup (one per wave)

typedef const __attribute__((address_space(4))) int64_t const_i64;
typedef const __attribute__((address_space(4))) float const_f32;

// xT[k][n] = x[n][k] for n < N, 0 for N <= n < ldt.  32 x 32 tiles through LDS.
__global__ __launch_bounds__(256) void transpose_kernel(const float *__restrict__ x, int64_t ldx,
                                                        float *__restrict__ xT, int ldt, int N, int K)
{
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    const int k0 = blockIdx.x * 32, n0 = blockIdx.y * 32;
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const int n = n0 + r, k = k0 + tx;
        tile[r][tx] = (n < N && k < K) ? x[(int64_t)n * ldx + k] : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const int k = k0 + r, n = n0 + tx;
        if (k < K && n < ldt) xT[(int64_t)k * ldt + n] = tile[tx][r];
    }
}

template <int TI> struct XVec;
template <> struct XVec<1> { typedef float type; };
template <> struct XVec<4> { typedef float4 type; };
__device__ __forceinline__ float lane_elem(const float &v, int) { return v; }
__device__ __forceinline__ float lane_elem(const float4 &v, int t)
{
    return t == 0 ? v.x : t == 1 ? v.y : t == 2 ? v.z : v.w;
}

// LM (lane-held entry data): the row's column offsets and values are read 64 entries at a time by the
// lanes of the wave (one coalesced load each, a block ahead of their use) and handed out with
// v_readlane, instead of coming through the scalar cache group by group: the scalar loads sat on every
// group's critical path, and their 64-bit address arithmetic took a third of the loop's instructions.
// Needs the byte offset of every xT row to fit 32 bits.
template <int TI, bool LM>
__global__ __launch_bounds__(NT_F) void csr_fwd_kernel(
    const float *__restrict__ xT, int ldt, const int64_t *__restrict__ crow,
    const int64_t *__restrict__ col, const float *__restrict__ val, const float *__restrict__ bias,
    float *__restrict__ c, int32_t *__restrict__ argmax, int32_t *__restrict__ argmin,
    float *__restrict__ w_sel, int32_t *__restrict__ pos_sel, float *__restrict__ x_sel, int N, int K, int M,
    int vec_out)
{
    typedef typename XVec<TI>::type xvec;
    constexpr int TILE_N = 64 * TI;
    // results of the workgroup's 16 neurons, [array][neuron][batch row]: 7 x 16 KiB for TI = 4
    extern __shared__ float out_lds[];
    float (*out_c)[TILE_N] = reinterpret_cast<float (*)[TILE_N]>(out_lds);
    int (*out_hi)[TILE_N] = reinterpret_cast<int (*)[TILE_N]>(out_lds + 1 * ROWS * TILE_N);
    int (*out_lo)[TILE_N] = reinterpret_cast<int (*)[TILE_N]>(out_lds + 2 * ROWS * TILE_N);
    float (*out_wh)[TILE_N] = reinterpret_cast<float (*)[TILE_N]>(out_lds + 3 * ROWS * TILE_N);
    float (*out_wl)[TILE_N] = reinterpret_cast<float (*)[TILE_N]>(out_lds + 4 * ROWS * TILE_N);
    int (*out_ph)[TILE_N] = reinterpret_cast<int (*)[TILE_N]>(out_lds + 5 * ROWS * TILE_N);
    int (*out_pl)[TILE_N] = reinterpret_cast<int (*)[TILE_N]>(out_lds + 6 * ROWS * TILE_N);
    float (*out_xh)[TILE_N] = reinterpret_cast<float (*)[TILE_N]>(out_lds + 7 * ROWS * TILE_N);
    float (*out_xl)[TILE_N] = reinterpret_cast<float (*)[TILE_N]>(out_lds + 8 * ROWS * TILE_N);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = blockIdx.x * ROWS + wave;
    const int n0 = blockIdx.y * TILE_N;
    int nl = n0 + lane * TI;
    if (nl > ldt - TI) nl = ldt - TI;  // lanes past the batch repeat the last rows; never stored

    if (m < M) {
        const_i64 *ccol = (const_i64 *)col;
        const_f32 *cval = (const_f32 *)val;
        const int64_t beg = ((const_i64 *)crow)[m], end = ((const_i64 *)crow)[m + 1];
        const int nnz = (int)(end - beg);
        const float *xl = xT + nl;

        // Running extremes, and the PAIR of consecutive entries (positions 2p, 2p+1 within the row) in which
        // each was last strictly improved: two products fold into the running extreme with one
        // v_max3 / v_min3, and one compare + select per extreme and pair records the pair.  Strict
        // compares in ascending entry order make the recorded pair the one that holds the FIRST
        // occurrence of the final extreme; which of its two entries it is, is settled once per output
        // after the loop from the pair's FIRST product, which is kept beside the pair id: if it equals
        // the extreme the first entry is the one, else the second.  (Tracking every product by itself
        // takes a compare and two selects per product and extreme; this takes one compare and two selects
        // per PAIR and extreme.)
        float vmax[TI], vmin[TI];
        float amax[TI], amin[TI];     // first product of the recorded pair
        int pmax[TI], pmin[TI];
#pragma unroll
        for (int t = 0; t < TI; ++t) {
            vmax[t] = -__builtin_inff();
            vmin[t] = __builtin_inff();
            pmax[t] = -1;
            pmin[t] = -1;
            amax[t] = 0.0f;
            amin[t] = 0.0f;
        }

        xvec xa[EG], xb[EG];
        float wa[EG], wb[EG];
        auto fold = [&](int pair, const xvec &x0, float w0, const xvec &x1, float w1) {
#pragma unroll
            for (int t = 0; t < TI; ++t) {
                const float a = lane_elem(x0, t) * w0, b = lane_elem(x1, t) * w1;
                const float hi = __builtin_fmaxf(__builtin_fmaxf(vmax[t], a), b);
                const float lo = __builtin_fminf(__builtin_fminf(vmin[t], a), b);
                const bool up = hi > vmax[t], down = lo < vmin[t];
                pmax[t] = up ? pair : pmax[t];
                amax[t] = up ? a : amax[t];
                pmin[t] = down ? pair : pmin[t];
                amin[t] = down ? a : amin[t];
                vmax[t] = hi;
                vmin[t] = lo;
            }
        };
        auto consume = [&](int g, const xvec (&xv)[EG], const float (&wv)[EG]) {
#pragma unroll
            for (int u = 0; u < EG; u += 2) fold(g * (EG / 2) + u / 2, xv[u], wv[u], xv[u + 1], wv[u + 1]);
        };
        // lowest column missing from the row: stored columns ascend, so it is the first position p
        // with col[p] != p, or nnz when the row is a full prefix
        int missing = nnz;
        if (LM) {
            static_assert(EG == 8, "the block loop below hands out 8 entries per group");
            // entries past the end of the row repeat the last one: a repeated product never wins a strict
            // compare, so every group is a whole group
            const char *xbytes = reinterpret_cast<const char *>(xl);
            const uint32_t row_bytes = (uint32_t)ldt * 4u;
            uint32_t off_cur = 0, off_nxt = 0;     // lane e: byte offset of the xT row of entry 64 blk + e
            float val_cur = 0.0f, val_nxt = 0.0f;
            bool hole_found = false;
            auto load_meta = [&](int blk, uint32_t &off, float &v) {
                const int e = blk * 64 + lane;
                const int ec = e < nnz ? e : nnz - 1;
                const int64_t cc = col[beg + ec];
                off = (uint32_t)cc * row_bytes;
                v = val[beg + ec];
                if (!hole_found) {
                    const uint64_t mask = __ballot(e < nnz && cc != (int64_t)e);
                    if (mask) { missing = blk * 64 + __builtin_ctzll(mask); hole_found = true; }
                }
            };
            const int nblk = (nnz + 63) >> 6;
            if (nblk > 0) load_meta(0, off_cur, val_cur);
            // one group = 8 lanes' worth of (offset, value), read out of the block's registers
#define MAM_CSR_ISSUE(G8, OFF, VAL, XV, WV)                                                                  \
    _Pragma("unroll") for (int u = 0; u < EG; ++u) {                                                         \
        const uint32_t so = __builtin_amdgcn_readlane(OFF, (G8) * EG + u);                                   \
        WV[u] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, VAL), (G8) * EG + u)); \
        XV[u] = *reinterpret_cast<const xvec *>(xbytes + so);                                                \
    }
            if (nblk > 0) { MAM_CSR_ISSUE(0, off_cur, val_cur, xa, wa) }
            for (int blk = 0; blk < nblk; ++blk) {
                const bool more = blk + 1 < nblk;
                if (more) load_meta(blk + 1, off_nxt, val_nxt);
                const int left = nnz - blk * 64;
                const int ngb = left >= 64 ? 8 : (left + EG - 1) / EG;     // groups of this block
                const int g0 = blk * 8;
                // groups 0, 2, 4, 6 sit in buffer a, the odd ones in b; the loads of the next group are in
                // flight while a group is consumed, across the block boundary too
#define MAM_CSR_STEP(G8, XCUR, WCUR, XNXT, WNXT)                                                             \
    if ((G8) < ngb) {                                                                                        \
        if ((G8) + 1 < ngb) { MAM_CSR_ISSUE((G8) + 1, off_cur, val_cur, XNXT, WNXT) }                        \
        __builtin_amdgcn_sched_barrier(0);                                                                   \
        consume(g0 + (G8), XCUR, WCUR);                                                                      \
        __builtin_amdgcn_sched_barrier(0);                                                                   \
    }
                MAM_CSR_STEP(0, xa, wa, xb, wb)
                MAM_CSR_STEP(1, xb, wb, xa, wa)
                MAM_CSR_STEP(2, xa, wa, xb, wb)
                MAM_CSR_STEP(3, xb, wb, xa, wa)
                MAM_CSR_STEP(4, xa, wa, xb, wb)
                MAM_CSR_STEP(5, xb, wb, xa, wa)
                MAM_CSR_STEP(6, xa, wa, xb, wb)
                // the last group of a whole block: the first group of the next block goes out before it
                if (7 < ngb) {
                    if (more) { MAM_CSR_ISSUE(0, off_nxt, val_nxt, xa, wa) }
                    __builtin_amdgcn_sched_barrier(0);
                    consume(g0 + 7, xb, wb);
                    __builtin_amdgcn_sched_barrier(0);
                }
                off_cur = off_nxt;
                val_cur = val_nxt;
            }
#undef MAM_CSR_STEP
#undef MAM_CSR_ISSUE
        } else {
        // full groups of EG entries, software-pipelined: the loads of group g+1 are in flight while
        // group g is consumed, so a row costs about one memory round trip per group
        const int ng = nnz / EG;
        auto issue = [&](int g, xvec (&xv)[EG], float (&wv)[EG]) {
#pragma unroll
            for (int u = 0; u < EG; ++u) {
                xv[u] = *reinterpret_cast<const xvec *>(xl + ccol[beg + g * EG + u] * (int64_t)ldt);
                wv[u] = cval[beg + g * EG + u];
            }
        };
        // two register buffers, the loop unrolled by two groups, so that no copy (which would
        // have to wait for the data) sits between issuing and consuming
        if (ng > 0) issue(0, xa, wa);
        for (int g = 0; g < ng; g += 2) {
            if (g + 1 < ng) issue(g + 1, xb, wb);
            __builtin_amdgcn_sched_barrier(0);
            consume(g, xa, wa);
            __builtin_amdgcn_sched_barrier(0);
            if (g + 1 >= ng) break;
            if (g + 2 < ng) issue(g + 2, xa, wa);
            __builtin_amdgcn_sched_barrier(0);
            consume(g + 1, xb, wb);
            __builtin_amdgcn_sched_barrier(0);
        }
        // the last, partial group pair by pair; an odd last entry is paired with itself (a repeated
        // product never wins a strict compare)
        for (int i = ng * EG; i < nnz; i += 2) {
            const int j = i + 1 < nnz ? i + 1 : i;
            const xvec x0 = *reinterpret_cast<const xvec *>(xl + ccol[beg + i] * (int64_t)ldt);
            const xvec x1 = *reinterpret_cast<const xvec *>(xl + ccol[beg + j] * (int64_t)ldt);
            fold(i / 2, x0, cval[beg + i], x1, cval[beg + j]);
        }
        for (int base = 0; base < nnz; base += 64) {
            const int p = base + lane;
            const bool hole = p < nnz && col[beg + p] != (int64_t)p;
            const uint64_t mask = __ballot(hole);
            if (mask) { missing = base + __builtin_ctzll(mask); break; }
        }
        }
        const bool has_zero = nnz < K;
        xvec zx;
        if (has_zero) zx = *reinterpret_cast<const xvec *>(xl + (int64_t)missing * ldt);
        const float bm = bias ? bias[m] : 0.0f;

        // Which entry of the recorded pair: the first one if the pair's first product equals the extreme,
        // else the second.  Column and value of the selected entry are two small divergent loads per
        // extreme.  The value is that of the selected entry's own product: the kept first product, or the
        // extreme itself, which equals the second product -- except that a zero extreme may carry the
        // other zero's sign, so a second entry selected for a zero extreme is recomputed (rare: a branch
        // that whole waves skip).
        // All 2 TI outputs of the lane are settled together: their column / value loads leave in one
        // batch and the selected inputs in a second one, so the epilogue is two trips to memory and not
        // one chain of dependent loads per output.
        int ri[2][TI];
        float rw[2][TI], rx[2][TI];
        if (nnz > 0) {
            int es[2][TI];
            bool ok[2][TI], first[2][TI];
#pragma unroll
            for (int t = 0; t < TI; ++t) {
#pragma unroll
                for (int ext = 0; ext < 2; ++ext) {
                    const int pair = ext ? pmin[t] : pmax[t];
                    const float kept = ext ? amin[t] : amax[t], target = ext ? vmin[t] : vmax[t];
                    ok[ext][t] = pair >= 0;
                    first[ext][t] = kept == target;
                    const int e0 = 2 * (pair < 0 ? 0 : pair);
                    es[ext][t] = first[ext][t] ? e0 : ((e0 + 1 < nnz) ? e0 + 1 : e0);
                }
            }
            int64_t cc[2][TI];
#pragma unroll
            for (int t = 0; t < TI; ++t) {
#pragma unroll
                for (int ext = 0; ext < 2; ++ext) {
                    cc[ext][t] = col[beg + es[ext][t]];
                    rw[ext][t] = val[beg + es[ext][t]];
                }
            }
            bool need_x = x_sel != nullptr;
            if (!need_x) {
                // a second entry selected for a zero extreme is recomputed (rare: whole waves skip the loads)
                bool rare = false;
#pragma unroll
                for (int t = 0; t < TI; ++t) {
                    rare = rare || (ok[0][t] && !first[0][t] && vmax[t] == 0.0f);
                    rare = rare || (ok[1][t] && !first[1][t] && vmin[t] == 0.0f);
                }
                need_x = __ballot(rare) != 0ull;
            }
#pragma unroll
            for (int t = 0; t < TI; ++t) {
#pragma unroll
                for (int ext = 0; ext < 2; ++ext) rx[ext][t] = need_x ? xT[cc[ext][t] * (int64_t)ldt + nl + t] : 0.0f;
            }
#pragma unroll
            for (int t = 0; t < TI; ++t) {
#pragma unroll
                for (int ext = 0; ext < 2; ++ext) {
                    float &target = ext ? vmin[t] : vmax[t];
                    int &pos = ext ? pmin[t] : pmax[t];
                    if (ok[ext][t]) {
                        if (first[ext][t]) target = ext ? amin[t] : amax[t];
                        else if (target == 0.0f) target = rx[ext][t] * rw[ext][t];
                        pos = es[ext][t];
                        ri[ext][t] = (int)cc[ext][t];
                        if (!x_sel) rx[ext][t] = 0.0f;
                    } else {
                        pos = -1;
                        ri[ext][t] = -1;
                        rw[ext][t] = 0.0f;
                        rx[ext][t] = 0.0f;
                    }
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < TI; ++t) {
#pragma unroll
                for (int ext = 0; ext < 2; ++ext) {
                    (ext ? pmin[t] : pmax[t]) = -1;
                    ri[ext][t] = -1;
                    rw[ext][t] = 0.0f;
                    rx[ext][t] = 0.0f;
                }
            }
        }

#pragma unroll
        for (int t = 0; t < TI; ++t) {
            float hi = vmax[t], lo = vmin[t], wh = rw[0][t], wl = rw[1][t], xh = rx[0][t], xl_ = rx[1][t];
            int ih = ri[0][t], il = ri[1][t], ph = pmax[t], pl = pmin[t];
            if (has_zero) {
                const float z = lane_elem(zx, t) * 0.0f;
                if (ih < 0 || z > hi || (z == hi && missing < ih)) { hi = z; ih = missing; wh = 0.0f; xh = 0.0f; ph = -1; }
                if (il < 0 || z < lo || (z == lo && missing < il)) { lo = z; il = missing; wl = 0.0f; xl_ = 0.0f; pl = -1; }
            }
            float s = hi + lo;
            if (bias) s = s + bm;
            const int o = lane * TI + t;
            out_c[wave][o] = s;
            out_hi[wave][o] = ih;
            out_lo[wave][o] = il;
            out_wh[wave][o] = wh;
            out_wl[wave][o] = wl;
            out_xh[wave][o] = xh;
            out_xl[wave][o] = xl_;
            out_ph[wave][o] = ph < 0 ? -1 : (int)(beg + ph);
            out_pl[wave][o] = pl < 0 ? -1 : (int)(beg + pl);
        }
    }
    __syncthreads();

    // a thread stores 4 consecutive neurons of one batch row: 16 bytes per output array, and the 4
    // threads of a batch row together one 64-byte run
    const int m0 = blockIdx.x * ROWS;
    const int64_t nm = (int64_t)N * M;
    for (int it = tid; it < TILE_N * (ROWS / 4); it += NT_F) {
        const int o = it / (ROWS / 4), q = it % (ROWS / 4);
        const int n = n0 + o;
        if (n >= N) continue;
        const int r0 = 4 * q;
        if (m0 + r0 >= M) continue;
        const int64_t base = (int64_t)n * M + m0 + r0;
        if (vec_out && m0 + r0 + 4 <= M) {
            *reinterpret_cast<float4 *>(c + base) = make_float4(out_c[r0][o], out_c[r0 + 1][o], out_c[r0 + 2][o], out_c[r0 + 3][o]);
            *reinterpret_cast<int4 *>(argmax + base) = make_int4(out_hi[r0][o], out_hi[r0 + 1][o], out_hi[r0 + 2][o], out_hi[r0 + 3][o]);
            *reinterpret_cast<int4 *>(argmin + base) = make_int4(out_lo[r0][o], out_lo[r0 + 1][o], out_lo[r0 + 2][o], out_lo[r0 + 3][o]);
            if (w_sel) {
                *reinterpret_cast<float4 *>(w_sel + base) = make_float4(out_wh[r0][o], out_wh[r0 + 1][o], out_wh[r0 + 2][o], out_wh[r0 + 3][o]);
                *reinterpret_cast<float4 *>(w_sel + nm + base) = make_float4(out_wl[r0][o], out_wl[r0 + 1][o], out_wl[r0 + 2][o], out_wl[r0 + 3][o]);
            }
            if (pos_sel) {
                *reinterpret_cast<int4 *>(pos_sel + base) = make_int4(out_ph[r0][o], out_ph[r0 + 1][o], out_ph[r0 + 2][o], out_ph[r0 + 3][o]);
                *reinterpret_cast<int4 *>(pos_sel + nm + base) = make_int4(out_pl[r0][o], out_pl[r0 + 1][o], out_pl[r0 + 2][o], out_pl[r0 + 3][o]);
            }
            if (x_sel) {
                *reinterpret_cast<float4 *>(x_sel + base) = make_float4(out_xh[r0][o], out_xh[r0 + 1][o], out_xh[r0 + 2][o], out_xh[r0 + 3][o]);
                *reinterpret_cast<float4 *>(x_sel + nm + base) = make_float4(out_xl[r0][o], out_xl[r0 + 1][o], out_xl[r0 + 2][o], out_xl[r0 + 3][o]);
            }
        } else {
            for (int r = r0; r < r0 + 4 && m0 + r < M; ++r) {
                const int64_t dst = (int64_t)n * M + m0 + r;
                c[dst] = out_c[r][o];
                argmax[dst] = out_hi[r][o];
                argmin[dst] = out_lo[r][o];
                if (w_sel) { w_sel[dst] = out_wh[r][o]; w_sel[nm + dst] = out_wl[r][o]; }
                if (pos_sel) { pos_sel[dst] = out_ph[r][o]; pos_sel[nm + dst] = out_pl[r][o]; }
                if (x_sel) { x_sel[dst] = out_xh[r][o]; x_sel[nm + dst] = out_xl[r][o]; }
            }
        }
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

// A float LDS atomic costs ~3 cycles per active lane on this chip, an integer one ~5 cycles per
// 64-lane instruction: one compare-and-swap round settles every lane that met no contender, and
// only the losers take the float atomic.  Entries of a row are rarely selected twice by the lanes
// of one instruction.
__device__ __forceinline__ void lds_add_sparse(float *addr, float v)
{
    int *word = reinterpret_cast<int *>(addr);
    const int seen = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    int expected = seen;
    const bool done = __hip_atomic_compare_exchange_strong(word, &expected, __float_as_int(__int_as_float(seen) + v),
                                                           __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                           __HIP_MEMORY_SCOPE_WORKGROUP);
    if (!done) __hip_atomic_fetch_add(addr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

#ifndef MAM_CSR_RB
#define MAM_CSR_RB 16
#endif
constexpr int RB = MAM_CSR_RB;   // CSR rows per val_grad workgroup
constexpr int VAL_CAP = 16384;   // histogram floats per pass (64 KiB)

// val_grad of the entries of RB consecutive CSR rows, from the entry positions recorded by the
// forward (pos_sel, (2, N, M), -1 where an implicit zero was selected).
__global__ __launch_bounds__(NT) void csr_bwd_val_kernel(
    const float *__restrict__ x, int64_t ldx, const int64_t *__restrict__ crow,
    const float *__restrict__ grad, const int32_t *__restrict__ argmax,
    const int32_t *__restrict__ argmin, const int32_t *__restrict__ pos_sel,
    const float *__restrict__ x_sel, int64_t nm, float *__restrict__ val_grad, int N, int M, int vec_in)
{
    __shared__ float hist[VAL_CAP];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.x * RB;
    const int rows = (M - m0) < RB ? (M - m0) : RB;
    const int64_t e_beg = crow[m0], e_end = crow[m0 + rows];
    for (int64_t c0 = e_beg; c0 < e_end; c0 += VAL_CAP) {
        const int len = (int)((e_end - c0) < VAL_CAP ? (e_end - c0) : VAL_CAP);
        for (int i = tid; i < len; i += NT) hist[i] = 0.0f;
        __syncthreads();
        for (int n = tid; n < N; n += NT) {
            const int64_t o = (int64_t)n * M + m0;
            const float *xr = x + (int64_t)n * ldx;
            float g[RB];
            int p1[RB], p2[RB], a1[RB], a2[RB];
            if (vec_in && rows == RB) {
#pragma unroll
                for (int q = 0; q < RB / 4; ++q) {
                    const float4 gv = *reinterpret_cast<const float4 *>(grad + o + 4 * q);
                    const int4 u1 = *reinterpret_cast<const int4 *>(pos_sel + o + 4 * q);
                    const int4 u2 = *reinterpret_cast<const int4 *>(pos_sel + nm + o + 4 * q);
                    const int4 k1 = *reinterpret_cast<const int4 *>(argmax + o + 4 * q);
                    const int4 k2 = *reinterpret_cast<const int4 *>(argmin + o + 4 * q);
                    g[4 * q + 0] = gv.x; g[4 * q + 1] = gv.y; g[4 * q + 2] = gv.z; g[4 * q + 3] = gv.w;
                    p1[4 * q + 0] = u1.x; p1[4 * q + 1] = u1.y; p1[4 * q + 2] = u1.z; p1[4 * q + 3] = u1.w;
                    p2[4 * q + 0] = u2.x; p2[4 * q + 1] = u2.y; p2[4 * q + 2] = u2.z; p2[4 * q + 3] = u2.w;
                    a1[4 * q + 0] = k1.x; a1[4 * q + 1] = k1.y; a1[4 * q + 2] = k1.z; a1[4 * q + 3] = k1.w;
                    a2[4 * q + 0] = k2.x; a2[4 * q + 1] = k2.y; a2[4 * q + 2] = k2.z; a2[4 * q + 3] = k2.w;
                }
            } else {
#pragma unroll
                for (int r = 0; r < RB; ++r) {
                    const bool ok = r < rows;
                    g[r] = ok ? grad[o + r] : 0.0f;
                    p1[r] = ok ? pos_sel[o + r] : -1;
                    p2[r] = ok ? pos_sel[nm + o + r] : -1;
                    a1[r] = ok ? argmax[o + r] : 0;
                    a2[r] = ok ? argmin[o + r] : 0;
                }
            }
            float x1[RB], x2[RB];
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                const int64_t q1 = (int64_t)p1[r] - c0, q2 = (int64_t)p2[r] - c0;
                p1[r] = (p1[r] >= 0 && q1 >= 0 && q1 < len) ? (int)q1 : -1;
                p2[r] = (p2[r] >= 0 && q2 >= 0 && q2 < len) ? (int)q2 : -1;
                // (the forward can hand the selected inputs over; else gather them)
                x1[r] = p1[r] >= 0 ? (x_sel ? x_sel[o + r] : xr[a1[r]]) : 0.0f;
                x2[r] = p2[r] >= 0 ? (x_sel ? x_sel[nm + o + r] : xr[a2[r]]) : 0.0f;
            }
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                if (p1[r] >= 0) lds_add_sparse(&hist[p1[r]], x1[r] * g[r]);
                if (p2[r] >= 0) lds_add_sparse(&hist[p2[r]], x2[r] * g[r]);
            }
        }
        __syncthreads();
        for (int i = tid; i < len; i += NT) val_grad[c0 + i] = hist[i];
        __syncthreads();
    }
}

// The same for 16-byte aligned inputs with M a multiple of 4 (what the operators produce): 1024 threads,
// a thread's item is one batch row x 4 consecutive CSR rows -- five 16-byte loads (the selected inputs as
// handed over by the forward; without them up to eight single-word gathers from x, which then take two
// thirds of the kernel's time)
// -- so that the four threads of a batch row cover whole 64-byte sectors and sixteen waves hide each
// other's latencies.  The entries' cells are 64-bit fixed point (mam_fixed.h): 256 batch rows pick among
// the few entries of a pruned row, so most lanes of an LDS atomic meet a contender, which costs an fp32
// atomic ~190 cycles per instruction and the integer one ~8 plus 2 per lane that shares an address; the sums
// are exact and val_grad does not depend on the order of arrival.  Terms outside the window go through a
// queue and are added in fp64 before the one rounding, a window that fits almost nothing to the fp32 LDS atomics.
constexpr int NT_V = 1024;
constexpr int VAL_CELLS = 7168;    // entries per pass (56 KiB of 8-byte cells: with the queue under 64 KiB)

__global__ __launch_bounds__(NT_V) void csr_bwd_val_vec_kernel(
    const float *__restrict__ x, int64_t ldx, const int64_t *__restrict__ crow,
    const float *__restrict__ grad, const int32_t *__restrict__ argmax,
    const int32_t *__restrict__ argmin, const int32_t *__restrict__ pos_sel,
    const float *__restrict__ x_sel, int64_t nm, float *__restrict__ val_grad, int N, int M, int span)
{
    using namespace fixedpoint;
    __shared__ unsigned long long cells[VAL_CELLS];
    __shared__ FixedQueue q;
    __shared__ uint32_t s_max;
    float *hist = reinterpret_cast<float *>(cells);
    const int tid = threadIdx.x;
    const int m0 = blockIdx.x * RB;
    const int rows = (M - m0) < RB ? (M - m0) : RB;
    const int64_t e_beg = crow[m0], e_end = crow[m0 + rows];
    constexpr int QPR = RB / 4;                      // items per batch row
    const int items = N * QPR;

    // one item: batch row n, CSR rows m0 + r0 .. r0 + 3; positions relative to the pass, -1 = nothing to add
    float4 g, s1, s2;
    int4 u1, u2, k1, k2;
    float x1[4], x2[4];
    int p1[4], p2[4];
#define MAM_VAL_LOAD(it, c0, len)                                                                    \
    do {                                                                                             \
        const int n_ = (it) / QPR, r0_ = ((it) % QPR) * 4;                                           \
        const bool ok_ = (it) < items && r0_ < rows;                                                 \
        u1 = u2 = make_int4(-1, -1, -1, -1);                                                         \
        k1 = k2 = make_int4(0, 0, 0, 0);                                                             \
        g = s1 = s2 = make_float4(0.f, 0.f, 0.f, 0.f);                                               \
        if (ok_) {                                                                                   \
            const int64_t o_ = (int64_t)n_ * M + m0 + r0_;                                           \
            g = *reinterpret_cast<const float4 *>(grad + o_);                                        \
            u1 = *reinterpret_cast<const int4 *>(pos_sel + o_);                                      \
            u2 = *reinterpret_cast<const int4 *>(pos_sel + nm + o_);                                 \
            if (x_sel) {                                                                             \
                s1 = *reinterpret_cast<const float4 *>(x_sel + o_);                                  \
                s2 = *reinterpret_cast<const float4 *>(x_sel + nm + o_);                             \
            } else {                                                                                 \
                k1 = *reinterpret_cast<const int4 *>(argmax + o_);                                   \
                k2 = *reinterpret_cast<const int4 *>(argmin + o_);                                   \
            }                                                                                        \
        }                                                                                            \
        const float sa_[4] = {s1.x, s1.y, s1.z, s1.w}, sb_[4] = {s2.x, s2.y, s2.z, s2.w};            \
        const int pa_[4] = {u1.x, u1.y, u1.z, u1.w}, pb_[4] = {u2.x, u2.y, u2.z, u2.w};              \
        const int ka_[4] = {k1.x, k1.y, k1.z, k1.w}, kb_[4] = {k2.x, k2.y, k2.z, k2.w};              \
        const float *xr_ = x + (int64_t)n_ * ldx;                                                    \
        _Pragma("unroll") for (int u_ = 0; u_ < 4; ++u_) {                                           \
            const int64_t qa_ = (int64_t)pa_[u_] - (c0), qb_ = (int64_t)pb_[u_] - (c0);              \
            p1[u_] = (pa_[u_] >= 0 && qa_ >= 0 && qa_ < (len)) ? (int)qa_ : -1;                      \
            p2[u_] = (pb_[u_] >= 0 && qb_ >= 0 && qb_ < (len)) ? (int)qb_ : -1;                      \
            x1[u_] = p1[u_] >= 0 ? (x_sel ? sa_[u_] : xr_[ka_[u_]]) : 0.0f;                          \
            x2[u_] = p2[u_] >= 0 ? (x_sel ? sb_[u_] : xr_[kb_[u_]]) : 0.0f;                          \
        }                                                                                            \
    } while (0)

    if (tid == 0) {
        s_max = 0u;
        q.count = 0;
    }
    __syncthreads();
    bool fixed = span >= 8;
    bool loaded = false;
    int e_lo = 1;
    {
        const int len0 = (int)((e_end - e_beg) < VAL_CELLS ? (e_end - e_beg) : VAL_CELLS);
        if (fixed) {
            MAM_VAL_LOAD(tid, e_beg, len0);
            loaded = true;
            const float gv[4] = {g.x, g.y, g.z, g.w};
            uint32_t mx = 0u;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t b1 = magnitude_bits(x1[u] * gv[u]), b2 = magnitude_bits(x2[u] * gv[u]);
                mx = mx > b1 ? mx : b1;
                mx = mx > b2 ? mx : b2;
            }
            const bool everything = items <= NT_V && e_end - e_beg <= VAL_CELLS;
            fixed = make_window(workgroup_max(mx, &s_max), everything ? 0 : 4, span, e_lo);
        }
    }
    for (int64_t c0 = e_beg; c0 < e_end; c0 += VAL_CELLS) {
        const int len = (int)((e_end - c0) < VAL_CELLS ? (e_end - c0) : VAL_CELLS);
        for (int attempt = fixed ? 0 : 1; attempt < 2; ++attempt) {
            const bool fx = attempt == 0;
            if (fx) for (int i = tid; i < len; i += NT_V) cells[i] = 0ull;
            else for (int i = tid; i < len; i += NT_V) hist[i] = 0.0f;
            __syncthreads();
            for (int it = tid; it < items; it += NT_V) {
                if (!loaded) MAM_VAL_LOAD(it, c0, len);
                loaded = false;
                const float gv[4] = {g.x, g.y, g.z, g.w};
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (p1[u] >= 0) {
                        const float t = x1[u] * gv[u];
                        if (!fx) lds_add_sparse(&hist[p1[u]], t);
                        else if (fixed_add(&cells[p1[u]], t, e_lo, span)) queue_push(q, p1[u], t);
                    }
                    if (p2[u] >= 0) {
                        const float t = x2[u] * gv[u];
                        if (!fx) lds_add_sparse(&hist[p2[u]], t);
                        else if (fixed_add(&cells[p2[u]], t, e_lo, span)) queue_push(q, p2[u], t);
                    }
                }
            }
            __syncthreads();
            const int queued = fx ? q.count : 0;
            __syncthreads();
            if (queued > QCAP) {
                if (tid == 0) q.count = 0;
                fixed = false;
                continue;
            }
            float *dst = val_grad + c0;
            if (queued > 0) {
                settle_queue<NT_V>(cells, len, q, queued, e_lo, 0);
                const double *d = reinterpret_cast<const double *>(cells);
                for (int i = tid; i < len; i += NT_V) dst[i] = (float)d[i];
                if (tid == 0) q.count = 0;
            } else if (fx) {
                for (int i = tid; i < len; i += NT_V) dst[i] = cell_value(cells[i], e_lo);
            } else {
                for (int i = tid; i < len; i += NT_V) dst[i] = hist[i];
            }
            __syncthreads();
            break;
        }
    }
#undef MAM_VAL_LOAD
}

// Checks the CSR invariants the sparse kernels rely on; ORs the violations found into *status.
//   1: crow[0] != 0 or crow[M] != nnz   2: crow not non-decreasing   4: a column index outside [0, K)
//   8: columns not strictly ascending within a row
__global__ __launch_bounds__(256) void csr_validate_kernel(const int64_t *__restrict__ crow,
                                                           const int64_t *__restrict__ col, int M, int K,
                                                           int64_t nnz, int *__restrict__ status)
{
    int bad = 0;
    const int64_t stride = (int64_t)gridDim.x * 256;
    const int64_t first = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (first == 0 && (crow[0] != 0 || crow[M] != nnz)) bad |= 1;
    for (int64_t m = first; m < M; m += stride) {
        const int64_t b = crow[m], e = crow[m + 1];
        if (e < b || b < 0 || e > nnz) {
            bad |= 2;
            continue;
        }
        for (int64_t i = b; i < e; ++i) {
            const int64_t cc = col[i];
            if (cc < 0 || cc >= K) bad |= 4;
            if (i > b && col[i - 1] >= cc) bad |= 8;
        }
    }
    if (bad) atomicOr(status, bad);
}

// Once per device: the forward kernels park 7 planes of results per workgroup in dynamic LDS (more than
// the 64 KiB a launch gets by default), and the fallback backward keeps up to 128 KiB of histogram.
static int g_bwd_lds_floats[kMaxDevices];

static int setup_device(int dev)
{
    bool ok = true;
    const void *small[] = {(const void *)csr_fwd_kernel<1, false>, (const void *)csr_fwd_kernel<1, true>};
    const void *large[] = {(const void *)csr_fwd_kernel<4, false>, (const void *)csr_fwd_kernel<4, true>};
    for (const void *k : small)
        ok = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 9 * ROWS * 64 * 4) == hipSuccess && ok;
    for (const void *k : large)
        ok = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 9 * ROWS * 256 * 4) == hipSuccess && ok;
    if (!ok) {
        (void)hipGetLastError();
        return fail(MAM_ERR_LAUNCH, "could not raise the LDS limit of the CSR forward kernels");
    }
    constexpr int kWant = 128 * 1024;
    if (hipFuncSetAttribute((const void *)csr_bwd_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kWant) ==
        hipSuccess) {
        g_bwd_lds_floats[dev] = kWant / 4;
    } else {
        (void)hipGetLastError();
        g_bwd_lds_floats[dev] = 64 * 1024 / 4;
    }
    return MAM_OK;
}
static DeviceHookRegistration g_registration(setup_device);

}  // namespace csr
}  // namespace mam

static int64_t transposed_ld(int64_t N) { return (N + 3) / 4 * 4; }

extern "C" int mam_csr_validate(const int64_t *crow, const int64_t *col, int64_t M, int64_t K, int64_t nnz,
                                int *status, void *stream)
{
    using namespace mam;
    if (M < 0 || K < 0 || nnz < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (!crow || !status || (nnz > 0 && !col)) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (M > INT32_MAX / 2 || K > INT32_MAX / 2) return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    hipStream_t st = static_cast<hipStream_t>(stream);
    int rc = fill_zero(status, 1, st);
    if (rc != MAM_OK) return rc;
    int64_t blocks = ceil_div(M > 0 ? M : 1, 256);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(csr::csr_validate_kernel, dim3((unsigned)blocks), dim3(256), 0, st, crow, col, (int)M, (int)K,
                       nnz, status);
    return check_launch("csr_validate_kernel");
}

extern "C" size_t mam_csr_fc_forward_workspace(int64_t N, int64_t K, int64_t M)
{
    if (N <= 0 || K <= 0 || M <= 0) return 0;
    return (size_t)K * (size_t)transposed_ld(N) * sizeof(float);
}

extern "C" int mam_csr_fc_forward(const float *x, int64_t ldx, const int64_t *crow, const int64_t *col,
                                  const float *val, const float *bias, float *c, int32_t *argmax,
                                  int32_t *argmin, float *w_sel, int32_t *pos_sel, float *x_sel, int64_t N,
                                  int64_t K, int64_t M, int64_t nnz, void *workspace, size_t workspace_bytes,
                                  void *stream)
{
    using namespace mam;
    if (N < 0 || K < 0 || M < 0 || nnz < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (N == 0 || M == 0) return MAM_OK;
    if (K == 0) return fail(MAM_ERR_INVALID_ARGUMENT, "K == 0: max/min over an empty set");
    if (!x || !crow || !c || !argmax || !argmin || (nnz > 0 && (!col || !val)))
        return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (ldx < K) return fail(MAM_ERR_INVALID_ARGUMENT, "ldx smaller than K");
    if (N > INT32_MAX / 2 || K > INT32_MAX / 2 || M > INT32_MAX / 2 || nnz > INT32_MAX)
        return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30 or nnz exceeds 2^31");
    const int64_t ldt = transposed_ld(N);
    const size_t need = (size_t)K * (size_t)ldt * sizeof(float);
    if (!workspace || workspace_bytes < need || (uintptr_t)workspace % 16 != 0)
        return fail(MAM_ERR_WORKSPACE, "CSR forward needs %zu workspace bytes, 16-byte aligned, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    const int dev = ensure_device(static_cast<hipStream_t>(stream));
    if (dev < 0) return dev;
    hipStream_t st = static_cast<hipStream_t>(stream);
    float *xT = static_cast<float *>(workspace);
    const int64_t gk = ceil_div(K, 32), gn = ceil_div(ldt, 32);
    if (gn > 65535) return fail(MAM_ERR_UNSUPPORTED, "N too large for the transpose grid");
    hipLaunchKernelGGL(csr::transpose_kernel, dim3((unsigned)gk, (unsigned)gn), dim3(256), 0, st, x, ldx, xT,
                       (int)ldt, (int)N, (int)K);
    int rc = check_launch("transpose_kernel");
    if (rc != MAM_OK) return rc;
    const int vec_out = (M % 4 == 0) && ((uintptr_t)c % 16 == 0) && ((uintptr_t)argmax % 16 == 0) &&
                        ((uintptr_t)argmin % 16 == 0) && ((uintptr_t)w_sel % 16 == 0) &&
                        ((uintptr_t)pos_sel % 16 == 0) && ((uintptr_t)x_sel % 16 == 0);
    // the lane-held entry data needs every xT row's byte offset in 32 bits
    const bool lm = (int64_t)K * ldt * 4 < ((int64_t)1 << 32);
    const dim3 grid1((unsigned)ceil_div(M, csr::ROWS), 1u);
    const int64_t gy = ceil_div(N, 256);
    if (gy > 65535) return fail(MAM_ERR_UNSUPPORTED, "N too large for the CSR forward grid");
    const dim3 grid4((unsigned)ceil_div(M, csr::ROWS), (unsigned)gy);
    const size_t lds1 = (size_t)9 * csr::ROWS * 64 * sizeof(float), lds4 = (size_t)9 * csr::ROWS * 256 * sizeof(float);
#define MAM_CSR_LAUNCH(TI, LM, GRID, LDS)                                                                           \
    hipLaunchKernelGGL((csr::csr_fwd_kernel<TI, LM>), GRID, dim3(csr::NT_F), LDS, st, xT, (int)ldt, crow, col, val, \
                       bias, c, argmax, argmin, w_sel, pos_sel, x_sel, (int)N, (int)K, (int)M, vec_out)
    if (N <= 64 && lm) MAM_CSR_LAUNCH(1, true, grid1, lds1);
    else if (N <= 64) MAM_CSR_LAUNCH(1, false, grid1, lds1);
    else if (lm) MAM_CSR_LAUNCH(4, true, grid4, lds4);
    else MAM_CSR_LAUNCH(4, false, grid4, lds4);
#undef MAM_CSR_LAUNCH
    return check_launch("csr_fwd_kernel");
}

extern "C" int mam_csr_fc_backward(const float *x, int64_t ldx, const int64_t *crow, const int64_t *col,
                                   const float *val, const float *grad, const int32_t *argmax,
                                   const int32_t *argmin, const float *w_sel, const int32_t *pos_sel,
                                   const float *x_sel, float *x_grad, float *val_grad, int64_t N, int64_t K,
                                   int64_t M, int64_t nnz, void *stream)
{
    using namespace mam;
    if (N < 0 || K < 0 || M < 0 || nnz < 0) return fail(MAM_ERR_INVALID_ARGUMENT, "negative size");
    if (N > INT32_MAX / 2 || K > INT32_MAX / 2 || M > INT32_MAX / 2)
        return fail(MAM_ERR_UNSUPPORTED, "a dimension exceeds 2^30");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool handed = w_sel && pos_sel;
    int rc = MAM_OK;
    if (val_grad && (!handed || N == 0 || M == 0)) rc = fill_zero(val_grad, nnz, st);
    if (rc != MAM_OK) return rc;
    if (N == 0 || K == 0) return MAM_OK;
    if (M == 0) return x_grad ? fill_zero(x_grad, N * K, st) : MAM_OK;
    if (!x || !crow || !grad || !argmax || !argmin) return fail(MAM_ERR_INVALID_ARGUMENT, "null pointer");
    if (ldx < K) return fail(MAM_ERR_INVALID_ARGUMENT, "ldx smaller than K");
    if (handed) {
        // the two kernels are independent: side by side where that pays (see ForkedStream)
        ForkedStream fork(st, (x_grad && val_grad) ? N * M : 0);
        if (x_grad) {
            rc = bwd::x_grad_from_selected(grad, argmax, argmin, w_sel, x_grad, N, K, M, fork.side());
            if (rc != MAM_OK) return rc;
            fork.join_later();
        }
        if (val_grad) {
            const int vec_in = (M % 4 == 0) && ((uintptr_t)grad % 16 == 0) && ((uintptr_t)argmax % 16 == 0) &&
                               ((uintptr_t)argmin % 16 == 0) && ((uintptr_t)pos_sel % 16 == 0) &&
                               ((uintptr_t)x_sel % 16 == 0) && ((N * M) % 4 == 0);
            if (vec_in)
                hipLaunchKernelGGL(csr::csr_bwd_val_vec_kernel, dim3((unsigned)ceil_div(M, csr::RB)), dim3(csr::NT_V),
                                   0, st, x, ldx, crow, grad, argmax, argmin, pos_sel, x_sel, N * M, val_grad, (int)N,
                                   (int)M, fixedpoint::window_span(2 * N));
            else
                hipLaunchKernelGGL(csr::csr_bwd_val_kernel, dim3((unsigned)ceil_div(M, csr::RB)), dim3(csr::NT), 0,
                                   st, x, ldx, crow, grad, argmax, argmin, pos_sel, x_sel, N * M, val_grad, (int)N,
                                   (int)M, 0);
            rc = check_launch("csr_bwd_val_kernel");
        }
        const int rc_join = fork.join();
        return rc != MAM_OK ? rc : rc_join;
    }
    const int dev = ensure_device(st);
    if (dev < 0) return dev;
    const int budget = csr::g_bwd_lds_floats[dev];
    const int kc = (int)(K < budget ? K : budget);
    hipLaunchKernelGGL(csr::csr_bwd_kernel, dim3((unsigned)N), dim3(csr::NT_B), (size_t)kc * sizeof(float),
                       st, x, ldx, crow, col, val, grad, argmax, argmin, x_grad, val_grad, (int)K, (int)M,
                       kc);
    return check_launch("csr_bwd_kernel");
}
