// Shared host/device helpers of libmam_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/mam_hip.h"

namespace mam {

// Records the detail of a failure for mam_last_error() and returns `code`.
int fail(int code, const char *fmt, ...);

// Checks the launch that was just issued on the calling thread.
int check_launch(const char *what);

// Asynchronously sets `count` 32-bit words to zero with a small kernel (graph-capture safe).
int fill_zero(void *ptr, int64_t count, hipStream_t stream);

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

constexpr int kNumXCD = 8;   // MI355X: 8 accelerator complex dies, each with its own L2
constexpr int kNumCU = 256;  // 32 active CUs per XCD

// Workgroups are handed to the XCDs round-robin by linear id.  This maps the hardware id
// to a logical id such that logical ids [i*per, (i+1)*per) all run on XCD i, so that
// neighbouring logical tiles share one L2.
__device__ __forceinline__ int xcd_remap(int bid, int nblk)
{
    const int xcd = bid % kNumXCD, slot = bid / kNumXCD;
    const int q = nblk / kNumXCD, r = nblk % kNumXCD;
    return slot + xcd * q + (xcd < r ? xcd : r);
}

template <int LAYOUT>
__device__ __forceinline__ float load_w(const float *__restrict__ w, int64_t ldw, int64_t k, int64_t m)
{
    return LAYOUT == MAM_W_MK ? w[m * ldw + k] : w[k * ldw + m];
}

namespace bwd {
// x_grad (N,K) from the selected weights (2,N,M) written by a forward (mam_backward.hip).
int x_grad_from_selected(const float *grad, const int32_t *argmax, const int32_t *argmin, const float *w_sel,
                         float *x_grad, int64_t N, int64_t K, int64_t M, hipStream_t st);
}  // namespace bwd

}  // namespace mam
