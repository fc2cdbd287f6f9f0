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

// ---- per-device set-up ------------------------------------------------------------------------
// Everything that has to happen once per device before kernels are launched there (raising the LDS
// limit of the kernels that use more than 64 KiB, creating the library's second stream and its events,
// taking the address of the file-scope scratch array) is collected in hooks, one per source file, and run
// by ensure_device() under a per-device lock the first time an entry point sees that device -- or by
// mam_init(), which a caller that records HIP graphs calls before capturing.
constexpr int kMaxDevices = 16;
typedef int (*DeviceHook)(int dev);
struct DeviceHookRegistration { explicit DeviceHookRegistration(DeviceHook fn); };
// Returns the current device's index (0..kMaxDevices-1) after its hooks have run, or a negative MAM_ERR_*.
// `st` is the stream the entry point launches on: while it is being captured the hooks still run (they
// create nothing), and the second stream and its events are left for the first call outside a capture.
int ensure_device(hipStream_t st = nullptr);

// Run-time switches (mam_set_option; initial values come from the environment, read once at load).
int option(int which);

// Compute units of the current device (read from the device at its set-up).
int num_cus();

// dst (cols, rows) contiguous = transpose of src (rows, cols), row stride ld.
int transpose(const float *src, int64_t ld, float *dst, int64_t rows, int64_t cols, hipStream_t stream);

// Two independent kernels of one call side by side: the first runs on a second stream of the library
// (default priority, one per device) between a fork and a join event on the caller's stream.
//   ForkedStream fork(st, units);      // decides; fork.side() is `st` itself when not forked
//   launch A on fork.side(); fork.join_later(); launch B on st; rc = fork.join();
// Between eager launches the two events cost ~15 us, inside a captured graph next to nothing: the fork
// is taken from 2^22 `units` (outputs of the call) on where the caller says that it pays between eager
// launches (`eager_pays`), and from 2^16 on while `st` is being captured.
// Option MAM_OPT_BACKWARD_FORK forces it off / on.  The enqueue sequences of concurrent callers on one
// device are serialised (the events are reused), so an object of this class holds that device's lock
// while forked.  The second stream is created by the device's set-up, never inside a capture.
class ForkedStream {
public:
    ForkedStream(hipStream_t st, int64_t units, bool eager_pays = true);
    ~ForkedStream();
    hipStream_t side() const { return side_; }
    bool forked() const { return forked_; }
    void join_later();   // after the last launch on side(): records the join event
    int join();          // after the launches on the caller's stream: it waits for the side stream
private:
    hipStream_t st_, side_;
    int dev_;
    bool forked_, recorded_;
};

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

constexpr int kNumXCD = 8;   // MI355X: 8 accelerator complex dies, each with its own L2
constexpr int kNumCU = 256;  // 32 active CUs per XCD (fallback when the device cannot be asked)

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
