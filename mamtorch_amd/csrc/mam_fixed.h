// Exact accumulation of scattered fp32 terms in 64-bit fixed-point LDS cells (gfx950).
// Shared by the kernels that own a slab of a gradient and sum the terms that land in it.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mam {
namespace fixedpoint {

// An fp32 term is m * 2^(e - 150) with a 24-bit integer m.  Relative to a window [e_lo, e_lo + span) of
// biased exponents it is the integer m << (e - e_lo), and integer adds are exact and commute: the cell ends
// up with the exact sum of its terms whatever order the lanes arrive in, rounded to fp32 once when the slab
// is stored -- and the integer LDS atomic costs ~8 cycles per 64-lane instruction where ds_add_f32 costs
// ~190.  span leaves room for every term a cell can receive (2 * M * planes), so the sum cannot overflow.
// The window is placed by the largest term of the workgroup's first trip (plus 4 binades where that is
// not the whole row).  The rare term outside it (tiny, huge, denormal, inf, nan) is parked in a small LDS
// queue and added, in fp64, before the slab is rounded and stored; if the queue overflows -- a first trip
// that says nothing about the rest -- the workgroup starts over with the fp32 LDS atomics.
constexpr int QCAP = 512;
struct FixedQueue {
    int count;
    int cell[QCAP];
    float val[QCAP];
};

__device__ __forceinline__ bool make_window(uint32_t maxbits, int margin, int span, int &e_lo)
{
    const int e = (int)(maxbits >> 23);               // biased exponent of the largest |term|
    if (e == 0 || e + margin >= 255) return false;    // only zeros and denormals, or inf / nan among them
    e_lo = e + margin - span + 1;
    if (e_lo < 1) e_lo = 1;
    return true;
}

// Adds t to the cell if it lies in the window; returns true when the caller has to queue it.
__device__ __forceinline__ bool fixed_add(unsigned long long *cell, float t, int e_lo, int span)
{
    const uint32_t b = __float_as_uint(t);
    const uint32_t sh = ((b >> 23) & 0xffu) - (uint32_t)e_lo;
    if (sh < (uint32_t)span) {
        const unsigned long long mag = (unsigned long long)((b & 0x7fffffu) | 0x800000u) << sh;
        __hip_atomic_fetch_add(cell, (b >> 31) ? 0ull - mag : mag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        return false;
    }
    return (b << 1) != 0u;
}

__device__ __forceinline__ void queue_push(FixedQueue &q, int cell, float t)
{
    const int slot = __hip_atomic_fetch_add(&q.count, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (slot < QCAP) {
        q.cell[slot] = cell;
        q.val[slot] = t;
    }
}

// The cell as fp64 and as fp32: through fp64, whose conversions and scaling are single instructions (an
// int64 -> fp32 conversion is a ~20-instruction sequence, and a slab has one cell per output element).  The
// fp64 value is exact below 2^53 in magnitude and rounded once to fp32; a larger sum (dozens of terms of the
// window's top binades in one cell) is first rounded to 53 bits, which can move the fp32 result by one unit in
// the last place only when that rounding lands exactly on an fp32 tie.
__device__ __forceinline__ double cell_double(unsigned long long c, int e_lo)
{
    const double hi = (double)(int)(c >> 32) * 4294967296.0;
    const double lo = (double)(unsigned int)c;
    return ldexp(hi + lo, e_lo - 150);
}
__device__ __forceinline__ float cell_value(unsigned long long c, int e_lo) { return (float)cell_double(c, e_lo); }

// A slab with queued terms: every cell is replaced by its fp64 value, in place, and the queued terms (each
// fp32, outside the window) are added in fp64, so that the one rounding to fp32 happens after them as well;
// the caller then stores (float) of the doubles.  Queue entries name cells as `cell_base` + index.
template <int NT>
__device__ __forceinline__ void settle_queue(unsigned long long *cells, int ncells, const FixedQueue &q, int queued,
                                             int e_lo, int cell_base)
{
    double *d = reinterpret_cast<double *>(cells);
    for (int i = threadIdx.x; i < ncells; i += NT) d[i] = cell_double(cells[i], e_lo);
    __syncthreads();
    for (int i = threadIdx.x; i < queued; i += NT) {
        const int idx = q.cell[i] - cell_base;
        if ((unsigned)idx < (unsigned)ncells)
            __hip_atomic_fetch_add(&d[idx], (double)q.val[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __syncthreads();
}

__device__ __forceinline__ uint32_t magnitude_bits(float t) { return __float_as_uint(t) & 0x7fffffffu; }

// Largest value over the workgroup; *slot is zero on entry (and a barrier has passed since).
__device__ __forceinline__ uint32_t workgroup_max(uint32_t v, uint32_t *slot)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const uint32_t other = (uint32_t)__shfl_xor((int)v, o);
        v = v > other ? v : other;
    }
    if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_max(slot, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __syncthreads();
    return *slot;
}


// Bits of room a cell needs for `terms` additions: span = 63 - 24 - count_bits(terms) binades fit a window.
inline int window_span(int64_t terms)
{
    int count_bits = 1;
    while (count_bits < 62 && ((int64_t)1 << count_bits) <= terms) ++count_bits;
    return 63 - 24 - count_bits;
}

}  // namespace fixedpoint
}  // namespace mam
