// Streaming a slab of packed selection counts from LDS into the (M, K) int32 counters (gfx950).
// Shared by the selection-count kernel and by the backward kernel that counts while it owns the slab.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mam_hip.h"

namespace mam {
namespace selcount {

// cnt: [rows][kc] words of two 16-bit fields (low: argmax picks, high: argmin picks) of the neurons
// m0 .. m0 + rn - 1 and the columns k0 .. k0 + kn - 1 (kn a multiple of 4, counters 16-byte aligned).  Every
// 16-byte chunk of counters that received a pick is read, added to and written back; chunks nobody touched
// are skipped.  FU chunks per thread are in flight between their loads and their stores.
template <int MODE, int NT, int FU>
__device__ __forceinline__ void stream_counts(const uint32_t *cnt, int32_t *__restrict__ max_count,
                                              int32_t *__restrict__ min_count, int tid, int m0, int k0, int rn,
                                              int kn, int kc, int K)
{
    const int q = kn >> 2;
    const int total = rn * q;
    for (int eb = tid; eb < total; eb += FU * NT) {
        uint4 v[FU];
        int4 amx[FU], amn[FU];
        int64_t cell[FU];
#pragma unroll
        for (int u = 0; u < FU; ++u) {
            const int e = eb + u * NT;
            v[u] = make_uint4(0u, 0u, 0u, 0u);
            cell[u] = 0;
            if (e < total) {
                const int r = e / q, c4 = e - r * q;
                v[u] = *reinterpret_cast<const uint4 *>(&cnt[r * kc + c4 * 4]);
                cell[u] = (int64_t)(m0 + r) * K + k0 + c4 * 4;
            }
        }
        if (MODE == MAM_COUNT_REFERENCE) {
            // both flags land in max_count: fold them into the low field
#pragma unroll
            for (int u = 0; u < FU; ++u) {
                v[u].x = (v[u].x & 1u) + (v[u].x >> 16);
                v[u].y = (v[u].y & 1u) + (v[u].y >> 16);
                v[u].z = (v[u].z & 1u) + (v[u].z >> 16);
                v[u].w = (v[u].w & 1u) + (v[u].w >> 16);
            }
        }
#pragma unroll
        for (int u = 0; u < FU; ++u) {
            const uint32_t any = v[u].x | v[u].y | v[u].z | v[u].w;
            if (any & 0xffffu) amx[u] = *reinterpret_cast<const int4 *>(max_count + cell[u]);
            if (any >> 16) amn[u] = *reinterpret_cast<const int4 *>(min_count + cell[u]);
        }
#pragma unroll
        for (int u = 0; u < FU; ++u) {
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
}

}  // namespace selcount
}  // namespace mam
