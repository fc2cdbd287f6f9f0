// Error reporting and version of libmam_hip.so.
#include "mam_common.h"

#include <stdarg.h>
#include <stdlib.h>

#include <string.h>

#include <atomic>
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

// dst (cols, rows) contiguous = transpose of src (rows, cols) with row stride ld: 64 x 64 tiles through LDS,
// 16-byte accesses on both sides when the shapes allow it.
__global__ __launch_bounds__(256) void transpose_kernel(const float *__restrict__ src, int64_t ld,
                                                        float *__restrict__ dst, int rows, int cols, int vec)
{
    __shared__ float tile[64][65];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = r0 + ty + 16 * i, c = c0 + tx * 4;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (r < rows) {
            const float *row = src + (int64_t)r * ld;
            if (vec && c + 3 < cols) {
                v = *reinterpret_cast<const float4 *>(row + c);
            } else {
                if (c < cols) v.x = row[c];
                if (c + 1 < cols) v.y = row[c + 1];
                if (c + 2 < cols) v.z = row[c + 2];
                if (c + 3 < cols) v.w = row[c + 3];
            }
        }
        float *t = &tile[ty + 16 * i][tx * 4];
        t[0] = v.x; t[1] = v.y; t[2] = v.z; t[3] = v.w;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = c0 + ty + 16 * i, r = r0 + tx * 4;       // dst row c, dst columns r .. r + 3
        if (c >= cols) continue;
        float *out = dst + (int64_t)c * rows;
        const float4 v = make_float4(tile[tx * 4][ty + 16 * i], tile[tx * 4 + 1][ty + 16 * i],
                                     tile[tx * 4 + 2][ty + 16 * i], tile[tx * 4 + 3][ty + 16 * i]);
        if (vec && r + 3 < rows && (rows & 3) == 0) {
            *reinterpret_cast<float4 *>(out + r) = v;
        } else {
            if (r < rows) out[r] = v.x;
            if (r + 1 < rows) out[r + 1] = v.y;
            if (r + 2 < rows) out[r + 2] = v.z;
            if (r + 3 < rows) out[r + 3] = v.w;
        }
    }
}

int transpose(const float *src, int64_t ld, float *dst, int64_t rows, int64_t cols, hipStream_t stream)
{
    if (rows <= 0 || cols <= 0) return MAM_OK;
    const int64_t gx = ceil_div(cols, 64), gy = ceil_div(rows, 64);
    if (gy > 65535 || gx > INT32_MAX) return fail(MAM_ERR_UNSUPPORTED, "matrix too large for the transpose grid");
    const int vec = (ld % 4 == 0) && ((uintptr_t)src % 16 == 0) && ((uintptr_t)dst % 16 == 0);
    hipLaunchKernelGGL(transpose_kernel, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, stream, src, ld, dst,
                       (int)rows, (int)cols, vec);
    return check_launch("transpose_kernel");
}

namespace {
struct DeviceState {
    std::mutex lock;             // set-up of this device, and its fork/join sequences
    std::atomic<int> ready{0};   // 1 once every hook has run, 2 once the second stream exists as well
    int rc = MAM_OK;
    std::atomic<int> cus{0};     // compute units, 0 = not asked yet
    hipStream_t stream = nullptr;   // the library's second stream (default priority)
    hipEvent_t fork = nullptr, join = nullptr;
    bool side_ok = false, side_tried = false;
};
DeviceState g_devices[kMaxDevices];

constexpr int kMaxHooks = 16;
DeviceHook g_hooks[kMaxHooks];
int g_num_hooks = 0;

// The values each option accepts.
struct OptionRange { const char *env; int lo, hi, fallback; bool wide_word; };
constexpr OptionRange kOptionRanges[MAM_OPT_COUNT_] = {
    {"MAM_FORWARD_TILING", MAM_FORWARD_TILING_AUTO, MAM_FORWARD_TILING_FUSED_MERGE, MAM_FORWARD_TILING_AUTO, true},
    {"MAM_BACKWARD_FORK", MAM_BACKWARD_FORK_AUTO, MAM_BACKWARD_FORK_ON, MAM_BACKWARD_FORK_AUTO, false},
    {"MAM_BACKWARD_ONE_LAUNCH", MAM_BACKWARD_ONE_LAUNCH_OFF, MAM_BACKWARD_ONE_LAUNCH_ON, MAM_BACKWARD_ONE_LAUNCH_AUTO,
     false},
    {"MAM_BACKWARD_EXACT", MAM_BACKWARD_EXACT_OFF, MAM_BACKWARD_EXACT_ON, MAM_BACKWARD_EXACT_OFF, false},
};

// An option's initial value: its environment variable when that holds "auto", a number inside the option's
// range or (forward tiling only) "wide"; the default otherwise.
int env_choice(int which)
{
    const OptionRange &r = kOptionRanges[which];
    const char *v = getenv(r.env);
    if (!v || !v[0] || strcmp(v, "auto") == 0) return r.fallback;
    if (r.wide_word && strcmp(v, "wide") == 0) return MAM_FORWARD_TILING_WIDE;
    char *end = nullptr;
    const long n = strtol(v, &end, 10);
    if (end == v || *end != '\0' || n < r.lo || n > r.hi) return r.fallback;
    return (int)n;
}
// initial values from the environment, read once when the library is loaded
std::atomic<int> g_options[MAM_OPT_COUNT_] = {
    {env_choice(0)}, {env_choice(1)}, {env_choice(2)}, {env_choice(3)},
};
}  // namespace

DeviceHookRegistration::DeviceHookRegistration(DeviceHook fn)
{
    if (g_num_hooks < kMaxHooks) g_hooks[g_num_hooks++] = fn;
}

int option(int which) { return g_options[which].load(std::memory_order_relaxed); }

// Whether `st`, the stream an entry point launches on, is being captured into a graph.
static bool stream_is_capturing(hipStream_t st)
{
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &status) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return status == hipStreamCaptureStatusActive;
}

static void create_side_stream(DeviceState &d)
{
    d.side_ok = hipStreamCreateWithFlags(&d.stream, hipStreamNonBlocking) == hipSuccess &&
                hipEventCreateWithFlags(&d.fork, hipEventDisableTiming) == hipSuccess &&
                hipEventCreateWithFlags(&d.join, hipEventDisableTiming) == hipSuccess;
    if (!d.side_ok) (void)hipGetLastError();
    d.side_tried = true;
}

int ensure_device(hipStream_t st)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return fail(MAM_ERR_LAUNCH, "no current HIP device");
    }
    if (dev < 0 || dev >= kMaxDevices) return fail(MAM_ERR_UNSUPPORTED, "device index %d beyond %d", dev, kMaxDevices - 1);
    DeviceState &d = g_devices[dev];
    if (d.ready.load(std::memory_order_acquire) == 2) return d.rc == MAM_OK ? dev : d.rc;
    // The kernel attributes and the scratch array's address may be taken at any time; the second stream and
    // its events must not be created while the caller's stream is being captured: that part waits for the
    // first call outside a capture (until then nothing forks).
    const bool capturing = stream_is_capturing(st);
    std::lock_guard<std::mutex> hold(d.lock);
    int state = d.ready.load(std::memory_order_relaxed);
    if (state == 0) {
        for (int i = 0; i < g_num_hooks && d.rc == MAM_OK; ++i) d.rc = g_hooks[i](dev);
        state = 1;
    }
    if (state == 1 && !capturing) {
        create_side_stream(d);
        state = 2;
    }
    d.ready.store(state, std::memory_order_release);
    return d.rc == MAM_OK ? dev : d.rc;
}

int num_cus()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return kNumCU;
    }
    int cus = g_devices[dev].cus.load(std::memory_order_relaxed);
    if (cus == 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
            (void)hipGetLastError();
            cus = kNumCU;
        }
        g_devices[dev].cus.store(cus, std::memory_order_relaxed);
    }
    return cus;
}

ForkedStream::ForkedStream(hipStream_t st, int64_t units, bool eager_pays)
    : st_(st), side_(st), dev_(-1), forked_(false), recorded_(false)
{
    if (units <= 0) return;
    const int choice = option(MAM_OPT_BACKWARD_FORK);
    bool want;
    if (choice == MAM_BACKWARD_FORK_OFF || choice == MAM_BACKWARD_FORK_ON) {
        want = choice == MAM_BACKWARD_FORK_ON;
    } else {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (st && hipStreamIsCapturing(st, &capturing) != hipSuccess) (void)hipGetLastError();
        want = (eager_pays && units >= (1 << 22)) || (capturing == hipStreamCaptureStatusActive && units >= (1 << 16));
    }
    if (!want) return;
    const int dev = ensure_device(st);
    if (dev < 0 || !g_devices[dev].side_ok) return;
    DeviceState &d = g_devices[dev];
    d.lock.lock();
    if (hipEventRecord(d.fork, st) == hipSuccess && hipStreamWaitEvent(d.stream, d.fork, 0) == hipSuccess) {
        side_ = d.stream;
        dev_ = dev;
        forked_ = true;
        return;
    }
    (void)hipGetLastError();
    d.lock.unlock();
}

void ForkedStream::join_later()
{
    if (!forked_ || recorded_) return;
    recorded_ = hipEventRecord(g_devices[dev_].join, side_) == hipSuccess;
}

int ForkedStream::join()
{
    if (!forked_) return MAM_OK;
    join_later();
    DeviceState &d = g_devices[dev_];
    const bool ok = recorded_ && hipStreamWaitEvent(st_, d.join, 0) == hipSuccess;
    forked_ = false;
    d.lock.unlock();
    return ok ? MAM_OK : fail(MAM_ERR_LAUNCH, "could not join the library's second stream");
}

ForkedStream::~ForkedStream()
{
    if (forked_) (void)join();
}

}  // namespace mam

extern "C" int mam_version(void) { return 200; }

extern "C" int mam_init(void)
{
    const int dev = mam::ensure_device();
    return dev < 0 ? dev : MAM_OK;
}

extern "C" int mam_device_info(int *compute_units, int *max_clock_khz)
{
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return mam::fail(MAM_ERR_LAUNCH, "no current HIP device");
    }
    if (compute_units) *compute_units = mam::num_cus();
    if (max_clock_khz) {
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeClockRate, dev) != hipSuccess) {
            (void)hipGetLastError();
            v = 0;
        }
        *max_clock_khz = v;
    }
    return MAM_OK;
}

extern "C" int mam_set_option(int option, int value)
{
    if (option < 0 || option >= MAM_OPT_COUNT_) return mam::fail(MAM_ERR_INVALID_ARGUMENT, "unknown option %d", option);
    const mam::OptionRange &r = mam::kOptionRanges[option];
    if (value < r.lo || value > r.hi)
        return mam::fail(MAM_ERR_INVALID_ARGUMENT, "option %d takes values %d..%d, got %d", option, r.lo, r.hi, value);
    mam::g_options[option].store(value, std::memory_order_relaxed);
    return MAM_OK;
}

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
