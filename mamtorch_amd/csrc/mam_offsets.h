// 32-bit byte offsets of weight rows as the index-resolving code of the forward forms them.  Plain
// C++ without HIP headers, so that a host-only test can compile and check the arithmetic at sizes
// (weight matrices beyond 4 GiB) that no GPU test allocates.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define MAM_HOST_DEVICE __host__ __device__
#else
#define MAM_HOST_DEVICE
#endif

namespace mam {

// Byte offset, from the first weight row of a set of `rows_in_set` consecutive neurons starting at neuron
// `first` (already < M), of row `r` of the set; rows past the last neuron M-1 repeat the last one.
// `ld_bytes` is the row stride in bytes.  The clamp is applied to the ROW NUMBER, before the multiply:
// (M - 1 - first) * ld_bytes may exceed 32 bits for a large matrix, (rows_in_set - 1) * ld_bytes does not
// (the host checks that a set of rows spans less than 4 GiB).
MAM_HOST_DEVICE inline uint32_t last_row_offset(int M, int first, int rows_in_set, uint32_t ld_bytes)
{
    const int last = (M - 1 - first) < (rows_in_set - 1) ? (M - 1 - first) : (rows_in_set - 1);
    return (uint32_t)last * ld_bytes;
}

MAM_HOST_DEVICE inline uint32_t clamped_row_offset(uint32_t row_offset, uint32_t last_offset)
{
    return row_offset < last_offset ? row_offset : last_offset;
}

}  // namespace mam
