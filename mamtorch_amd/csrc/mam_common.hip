// Error reporting and version of libmam_hip.so.
#include "mam_common.h"

#include <stdarg.h>

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
