// A host without PyTorch: plain C++ against the C ABI of libmam_hip.so, device memory from the HIP
// runtime, results checked against the C oracle (oracle/mam_oracle.c).  This is what the reference's
// C++ operator layer (mamtorch/kernel/v4/csrc/cuda/fullyconnected.cu:41-149 and
// fullyconnected_backward.cu:80-135) would call.  Built by tests/Makefile, run by
// tests/test_gpu_cabi_host.py.
//
//   cabi_host N K M seed     ->  prints one line per check and "PASS" / "FAIL"; exit status 0 / 1
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "mam_hip.h"

extern "C" {
void mam_oracle_forward(const float *x, int64_t ldx, const float *w, int64_t ldw, int layout, const float *bias,
                        float *c, int32_t *argmax, int32_t *argmin, int64_t N, int64_t K, int64_t M);
void mam_oracle_backward(const float *x, int64_t ldx, const float *w, int64_t ldw, int layout, const float *g,
                         const int32_t *argmax, const int32_t *argmin, float *x_grad, float *w_grad, int64_t N,
                         int64_t K, int64_t M);
void mam_oracle_selection_count(const int32_t *argmax, const int32_t *argmin, int32_t *max_count,
                                int32_t *min_count, int64_t N, int64_t M, int64_t K, int mode);
}

#define HIP_OK(call)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) {                                                               \
            std::printf("%s: %s\n", #call, hipGetErrorString(e_));                            \
            return 2;                                                                         \
        }                                                                                     \
    } while (0)
#define MAM_CALL(call)                                                                        \
    do {                                                                                      \
        int rc_ = (call);                                                                     \
        if (rc_ != MAM_OK) {                                                                  \
            std::printf("%s: %s (%s)\n", #call, mam_error_string(rc_), mam_last_error());     \
            return 2;                                                                         \
        }                                                                                     \
    } while (0)

static uint32_t lcg_state;
static float uniform_pm1()
{
    lcg_state = lcg_state * 1664525u + 1013904223u;
    return (float)((lcg_state >> 8) & 0xffff) / 32768.0f - 1.0f;   // multiples of 2^-15 in [-1, 1): ties happen
}

template <class T>
struct DeviceBuffer {
    T *p = nullptr;
    ~DeviceBuffer() { if (p) (void)hipFree(p); }
    hipError_t alloc(size_t n) { return hipMalloc(reinterpret_cast<void **>(&p), (n ? n : 1) * sizeof(T)); }
};

static bool same_bits(const std::vector<float> &a, const std::vector<float> &b, const char *what)
{
    for (size_t i = 0; i < a.size(); ++i)
        if (std::memcmp(&a[i], &b[i], 4) != 0) {
            std::printf("%s: first mismatch at %zu: got %.9g want %.9g\n", what, i, a[i], b[i]);
            return false;
        }
    std::printf("%s: %zu values bit-exact\n", what, a.size());
    return true;
}

static bool same_ints(const std::vector<int32_t> &a, const std::vector<int32_t> &b, const char *what)
{
    for (size_t i = 0; i < a.size(); ++i)
        if (a[i] != b[i]) {
            std::printf("%s: first mismatch at %zu: got %d want %d\n", what, i, a[i], b[i]);
            return false;
        }
    std::printf("%s: %zu values equal\n", what, a.size());
    return true;
}

// |got - want| <= 1e-5 |want| + 2^-22 * (sum of |terms| of the cell): the floor of any fp32 summation order
static bool close_enough(const std::vector<float> &got, const std::vector<float> &want,
                         const std::vector<float> &abs_sum, const char *what)
{
    for (size_t i = 0; i < got.size(); ++i) {
        const double tol = 1e-5 * std::fabs((double)want[i]) + std::ldexp((double)abs_sum[i], -22) + 1e-30;
        if (std::fabs((double)got[i] - (double)want[i]) > tol) {
            std::printf("%s: cell %zu out of tolerance: got %.9g want %.9g\n", what, i, got[i], want[i]);
            return false;
        }
    }
    std::printf("%s: %zu values within rtol 1e-5 + summation floor\n", what, got.size());
    return true;
}

int main(int argc, char **argv)
{
    const int64_t N = argc > 1 ? std::atoll(argv[1]) : 64, K = argc > 2 ? std::atoll(argv[2]) : 784,
                  M = argc > 3 ? std::atoll(argv[3]) : 256;
    lcg_state = argc > 4 ? (uint32_t)std::atoll(argv[4]) : 1u;
    std::printf("cabi_host: N %lld K %lld M %lld, library version %d\n", (long long)N, (long long)K, (long long)M,
                mam_version());
    const size_t nk = (size_t)(N * K), mk = (size_t)(M * K), nm = (size_t)(N * M);
    std::vector<float> x(nk), w(mk), g(nm), bias((size_t)M);
    for (auto &v : x) v = uniform_pm1();
    for (auto &v : w) v = uniform_pm1() * 0.125f;
    for (auto &v : g) v = uniform_pm1();
    for (auto &v : bias) v = uniform_pm1();

    // ---- oracle on the host ----
    std::vector<float> c_ref(nm), xg_ref(nk), wg_ref(mk), xg_abs(nk), wg_abs(mk);
    std::vector<int32_t> amax_ref(nm), amin_ref(nm), maxc_ref(mk, 3), minc_ref(mk, 5);
    mam_oracle_forward(x.data(), K, w.data(), K, MAM_W_MK, bias.data(), c_ref.data(), amax_ref.data(),
                       amin_ref.data(), N, K, M);
    mam_oracle_backward(x.data(), K, w.data(), K, MAM_W_MK, g.data(), amax_ref.data(), amin_ref.data(),
                        xg_ref.data(), wg_ref.data(), N, K, M);
    {
        std::vector<float> xa(x), wa(w), ga(g);
        for (auto &v : xa) v = std::fabs(v);
        for (auto &v : wa) v = std::fabs(v);
        for (auto &v : ga) v = std::fabs(v);
        mam_oracle_backward(xa.data(), K, wa.data(), K, MAM_W_MK, ga.data(), amax_ref.data(), amin_ref.data(),
                            xg_abs.data(), wg_abs.data(), N, K, M);
    }
    mam_oracle_selection_count(amax_ref.data(), amin_ref.data(), maxc_ref.data(), minc_ref.data(), N, M, K,
                               MAM_COUNT_HITS);

    // ---- the library on the GPU, everything on one stream of the caller ----
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    DeviceBuffer<float> dx, dw, dg, dbias, dc, dcv, dwsel, dxsel, dxg, dwg;
    DeviceBuffer<int32_t> damax, damin, dmaxc, dminc;
    DeviceBuffer<char> dws;
    HIP_OK(dx.alloc(nk)); HIP_OK(dw.alloc(mk)); HIP_OK(dg.alloc(nm)); HIP_OK(dbias.alloc((size_t)M));
    HIP_OK(dc.alloc(nm)); HIP_OK(dcv.alloc(nm)); HIP_OK(dwsel.alloc(2 * nm)); HIP_OK(dxsel.alloc(2 * nm));
    HIP_OK(dxg.alloc(nk)); HIP_OK(dwg.alloc(mk)); HIP_OK(damax.alloc(nm)); HIP_OK(damin.alloc(nm));
    HIP_OK(dmaxc.alloc(mk)); HIP_OK(dminc.alloc(mk));
    const size_t ws_args = mam_fc_forward_workspace(N, K, M), ws_vals = mam_fc_forward_values_workspace(N, K, M);
    const size_t ws_bytes = ws_args > ws_vals ? ws_args : ws_vals;
    HIP_OK(dws.alloc(ws_bytes));
    HIP_OK(hipMemcpyAsync(dx.p, x.data(), nk * 4, hipMemcpyHostToDevice, stream));
    HIP_OK(hipMemcpyAsync(dw.p, w.data(), mk * 4, hipMemcpyHostToDevice, stream));
    HIP_OK(hipMemcpyAsync(dg.p, g.data(), nm * 4, hipMemcpyHostToDevice, stream));
    HIP_OK(hipMemcpyAsync(dbias.p, bias.data(), (size_t)M * 4, hipMemcpyHostToDevice, stream));
    std::vector<int32_t> three(mk, 3), five(mk, 5);
    HIP_OK(hipMemcpyAsync(dmaxc.p, three.data(), mk * 4, hipMemcpyHostToDevice, stream));
    HIP_OK(hipMemcpyAsync(dminc.p, five.data(), mk * 4, hipMemcpyHostToDevice, stream));

    MAM_CALL(mam_fc_forward(dx.p, K, dw.p, K, MAM_W_MK, dbias.p, dc.p, damax.p, damin.p, dwsel.p, dxsel.p, N, K, M,
                            dws.p, ws_bytes, stream));
    MAM_CALL(mam_fc_forward_values(dx.p, K, dw.p, K, MAM_W_MK, dbias.p, dcv.p, N, K, M, dws.p, ws_bytes, stream));
    MAM_CALL(mam_fc_backward(dx.p, K, dw.p, K, MAM_W_MK, dg.p, damax.p, damin.p, dwsel.p, dxsel.p, dxg.p, dwg.p, N,
                             K, M, stream));
    MAM_CALL(mam_selection_count(damax.p, damin.p, dmaxc.p, dminc.p, N, M, K, MAM_COUNT_HITS, stream));

    std::vector<float> c(nm), cv(nm), xg(nk), wg(mk);
    std::vector<int32_t> amax(nm), amin(nm), maxc(mk), minc(mk);
    HIP_OK(hipMemcpyAsync(c.data(), dc.p, nm * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(cv.data(), dcv.p, nm * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(amax.data(), damax.p, nm * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(amin.data(), damin.p, nm * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(xg.data(), dxg.p, nk * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(wg.data(), dwg.p, mk * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(maxc.data(), dmaxc.p, mk * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(minc.data(), dminc.p, mk * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipStreamDestroy(stream));

    bool ok = true;
    ok &= same_bits(c, c_ref, "forward c");
    ok &= same_bits(cv, c_ref, "values-only c");
    ok &= same_ints(amax, amax_ref, "argmax");
    ok &= same_ints(amin, amin_ref, "argmin");
    ok &= close_enough(xg, xg_ref, xg_abs, "x_grad");
    ok &= close_enough(wg, wg_ref, wg_abs, "w_grad");
    ok &= same_ints(maxc, maxc_ref, "max_count");
    ok &= same_ints(minc, minc_ref, "min_count");
    // an error path: the code and the message come back through the ABI, nothing is launched
    const int rc = mam_fc_forward(dx.p, K, dw.p, K, 7, nullptr, dc.p, damax.p, damin.p, nullptr, nullptr, N, K, M,
                                  dws.p, ws_bytes, nullptr);
    std::printf("bad layout -> %d (%s)\n", rc, mam_last_error());
    ok &= rc == MAM_ERR_INVALID_ARGUMENT;
    std::printf(ok ? "PASS\n" : "FAIL\n");
    return ok ? 0 : 1;
}
