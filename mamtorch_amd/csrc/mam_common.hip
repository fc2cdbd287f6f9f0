// Error reporting and version of libmam_hip.so.
#include "mam_common.h"

#include <stdarg.h>
#include <stdlib.h>

#include <mutex>

namespace mam {

static thread_local char g_last_error[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char *what)
{
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MAM_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return MAM_OK;
}

__global__ __launch_bounds__(256) void fill_zero_kernel(uint32_t *__restrict__ p, int64_t count)
{
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += stride) p[i] = 0u;
}

int fill_zero(void *ptr, int64_t count, hipStream_t stream)
{
    if (count <= 0) return MAM_OK;
    int64_t blocks = ceil_div(count, 256);
    if (blocks > 16 * kNumCU) blocks = 16 * kNumCU;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                       static_cast<uint32_t *>(ptr), count);
    return check_launch("fill_zero_kernel");
}

namespace {
struct SideStream {
    hipStream_t stream = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    bool ok = false, tried = false;
};
std::mutex side_mutex;
SideStream side_streams[16];

SideStream *side_stream_of_current_device()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) {
        (void)hipGetLastError();
        return nullptr;
    }
    SideStream &s = side_streams[dev];
    if (!s.tried) {
        s.tried = true;
        s.ok = hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking) == hipSuccess &&
               hipEventCreateWithFlags(&s.fork, hipEventDisableTiming) == hipSuccess &&
               hipEventCreateWithFlags(&s.join, hipEventDisableTiming) == hipSuccess;
        if (!s.ok) (void)hipGetLastError();
    }
    return s.ok ? &s : nullptr;
}
}  // namespace

ForkedStream::ForkedStream(hipStream_t st, int64_t units) : st_(st), side_(st), forked_(false), recorded_(false)
{
    if (units <= 0) return;
    const char *env = getenv("MAM_BACKWARD_FORK");
    bool want;
    if (env && (env[0] == '0' || env[0] == '1')) {
        want = env[0] == '1';
    } else {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (st && hipStreamIsCapturing(st, &capturing) != hipSuccess) (void)hipGetLastError();
        want = units >= (1 << 22) || (capturing == hipStreamCaptureStatusActive && units >= (1 << 16));
    }
    if (!want) return;
    side_mutex.lock();
    SideStream *s = side_stream_of_current_device();
    if (s && hipEventRecord(s->fork, st) == hipSuccess && hipStreamWaitEvent(s->stream, s->fork, 0) == hipSuccess) {
        side_ = s->stream;
        forked_ = true;
        return;
    }
    (void)hipGetLastError();
    side_mutex.unlock();
}

void ForkedStream::join_later()
{
    if (!forked_ || recorded_) return;
    SideStream *s = side_stream_of_current_device();
    recorded_ = s && hipEventRecord(s->join, side_) == hipSuccess;
}

int ForkedStream::join()
{
    if (!forked_) return MAM_OK;
    join_later();
    SideStream *s = side_stream_of_current_device();
    const bool ok = recorded_ && s && hipStreamWaitEvent(st_, s->join, 0) == hipSuccess;
    forked_ = false;
    side_mutex.unlock();
    return ok ? MAM_OK : fail(MAM_ERR_LAUNCH, "could not join the library's second stream");
}

ForkedStream::~ForkedStream()
{
    if (forked_) (void)join();
}

}  // namespace mam

extern "C" int mam_version(void) { return 100; }

extern "C" const char *mam_last_error(void) { return mam::g_last_error; }

extern "C" const char *mam_error_string(int code)
{
    switch (code) {
        case MAM_OK: return "ok";
        case MAM_ERR_INVALID_ARGUMENT: return "invalid argument";
        case MAM_ERR_UNSUPPORTED: return "unsupported size";
        case MAM_ERR_WORKSPACE: return "workspace missing or too small";
        case MAM_ERR_LAUNCH: return "HIP launch error";
        default: return "unknown error code";
    }
}
