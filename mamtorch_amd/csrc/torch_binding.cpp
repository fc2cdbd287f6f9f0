// PyTorch-ROCm operator registration for the MAM hot path.  This file is plumbing only: it
// checks tensors, allocates outputs / workspace through torch's caching allocator, picks up the
// current HIP stream and calls the C ABI of libmam_hip.so (include/mam_hip.h).  No kernels here.
//
// Operator names and schemas are those of SSIGPRO/mamtorch 1.5.2
// (mamtorch/kernel/v1/csrc/register_functions.cpp:21-24,
//  mamtorch/kernel/v4/csrc/register_functions.cpp:10-14,
//  mamtorch/sparse/kernel/v1/csrc/cuda/register_functions.cu:18-28), so the reference's Python
// wrappers, fake kernels and autograd formulas bind to them unchanged.  Operators without an
// upstream name (weight-layout variants, selection_count, sparse MAM) are additions.
//
// Unlike the reference (whose TORCH_CHECKs are commented out,
// mamtorch/kernel/v1/csrc/cuda/fullyconnected.cu:181-189) every entry validates dtype, shape,
// device and contiguity and raises RuntimeError; launches go to the current stream under a
// device guard instead of the legacy default stream.
#include <ATen/ATen.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <vector>

#include "../../include/mam_hip.h"

namespace {

void *current_stream(const at::Tensor &t)
{
    return static_cast<void *>(c10::hip::getCurrentHIPStream(t.get_device()).stream());
}

void check_rc(int rc, const char *what)
{
    TORCH_CHECK(rc == MAM_OK, what, " failed: ", mam_error_string(rc), " (", mam_last_error(), ")");
}

void check_f32_2d(const at::Tensor &t, const char *name)
{
    TORCH_CHECK(t.is_cuda(), name, " must be on the GPU");
    TORCH_CHECK(t.scalar_type() == at::kFloat, name, " must be float32");
    TORCH_CHECK(t.dim() == 2, name, " must be 2-dimensional");
}

// Rows may be strided (a narrow() along the last dimension), elements within a row may not.
int64_t row_stride(const at::Tensor &t, const char *name)
{
    TORCH_CHECK(t.size(1) <= 1 || t.stride(1) == 1, name, " must have unit stride in its last dimension");
    if (t.size(0) <= 1) return std::max<int64_t>(t.size(1), 1);
    TORCH_CHECK(t.stride(0) >= t.size(1), name, " has overlapping rows");
    return t.stride(0);
}

void check_same_device(const at::Tensor &a, const at::Tensor &b, const char *name)
{
    TORCH_CHECK(a.device() == b.device(), name, " is on a different device");
}

void check_index(const at::Tensor &t, const at::Tensor &like, const char *name)
{
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt, name, " must be an int32 GPU tensor");
    TORCH_CHECK(t.sizes() == like.sizes(), name, " has the wrong shape");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    check_same_device(t, like, name);
}

at::Tensor workspace_for(size_t bytes, const at::Tensor &like)
{
    if (bytes == 0) return at::Tensor();
    return at::empty({static_cast<int64_t>(bytes)}, like.options().dtype(at::kByte));
}

struct FwdShape { int64_t N, K, M; };

FwdShape check_forward(const at::Tensor &a, const at::Tensor &w, int layout,
                       const c10::optional<at::Tensor> &bias)
{
    check_f32_2d(a, "a");
    check_f32_2d(w, layout == MAM_W_MK ? "weight" : "b");
    check_same_device(a, w, "the weight operand");
    FwdShape s{a.size(0), a.size(1), layout == MAM_W_MK ? w.size(0) : w.size(1)};
    TORCH_CHECK((layout == MAM_W_MK ? w.size(1) : w.size(0)) == s.K,
                "inner dimensions do not match: a is (", a.size(0), ",", a.size(1), "), the weight operand is (",
                w.size(0), ",", w.size(1), ")");
    TORCH_CHECK(s.K > 0 || s.N == 0 || s.M == 0, "in_features must be positive");
    if (bias.has_value() && bias->defined()) {
        TORCH_CHECK(bias->is_cuda() && bias->scalar_type() == at::kFloat && bias->dim() == 1 &&
                        bias->size(0) == s.M && bias->is_contiguous(),
                    "bias must be a contiguous float32 GPU vector of out_features elements");
        check_same_device(a, *bias, "bias");
    }
    return s;
}

const float *bias_ptr(const c10::optional<at::Tensor> &bias)
{
    return (bias.has_value() && bias->defined()) ? bias->data_ptr<float>() : nullptr;
}

std::vector<at::Tensor> forward_impl(const at::Tensor &a, const at::Tensor &w, int layout,
                                     const c10::optional<at::Tensor> &bias, bool with_sel, bool hand_over)
{
    const FwdShape s = check_forward(a, w, layout, bias);
    const c10::DeviceGuard guard(a.device());
    auto c = at::empty({s.N, s.M}, a.options());
    auto argmax = at::empty({s.N, s.M}, a.options().dtype(at::kInt));
    auto argmin = at::empty({s.N, s.M}, a.options().dtype(at::kInt));
    // selected operands for the backward, only where the caller keeps them: planes 0, 1 hold
    // w[argmax], w[argmin], planes 2, 3 hold x[argmax], x[argmin]
    at::Tensor sel;
    if (with_sel) sel = at::empty({hand_over ? 4 : 0, s.N, s.M}, a.options());
    float *w_sel = (with_sel && hand_over) ? sel.data_ptr<float>() : nullptr;
    float *x_sel = w_sel ? w_sel + 2 * s.N * s.M : nullptr;
    if (s.N == 0 || s.M == 0) {
        if (with_sel) return {c, argmax, argmin, sel};
        return {c, argmax, argmin};
    }
    const size_t ws_bytes = mam_fc_forward_workspace_for(s.N, s.K, s.M, layout, 1);
    auto ws = workspace_for(ws_bytes, a);
    check_rc(mam_fc_forward(a.data_ptr<float>(), row_stride(a, "a"), w.data_ptr<float>(),
                            row_stride(w, "the weight operand"), layout, bias_ptr(bias),
                            c.data_ptr<float>(), argmax.data_ptr<int32_t>(), argmin.data_ptr<int32_t>(),
                            w_sel, x_sel, s.N, s.K, s.M,
                            ws.defined() ? ws.data_ptr() : nullptr, ws_bytes, current_stream(a)),
             "mam_fc_forward");
    if (with_sel) return {c, argmax, argmin, sel};
    return {c, argmax, argmin};
}

at::Tensor forward_values_impl(const at::Tensor &a, const at::Tensor &w, int layout,
                               const c10::optional<at::Tensor> &bias)
{
    const FwdShape s = check_forward(a, w, layout, bias);
    const c10::DeviceGuard guard(a.device());
    auto c = at::empty({s.N, s.M}, a.options());
    if (s.N == 0 || s.M == 0) return c;
    const size_t ws_bytes = mam_fc_forward_workspace_for(s.N, s.K, s.M, layout, 0);
    auto ws = workspace_for(ws_bytes, a);
    check_rc(mam_fc_forward_values(a.data_ptr<float>(), row_stride(a, "a"), w.data_ptr<float>(),
                                   row_stride(w, "the weight operand"), layout, bias_ptr(bias),
                                   c.data_ptr<float>(), s.N, s.K, s.M,
                                   ws.defined() ? ws.data_ptr() : nullptr, ws_bytes, current_stream(a)),
             "mam_fc_forward_values");
    return c;
}

std::vector<at::Tensor> backward_impl(const at::Tensor &a, const at::Tensor &w, int layout,
                                      const at::Tensor &grad, const at::Tensor &argmax,
                                      const at::Tensor &argmin, const c10::optional<at::Tensor> &sel)
{
    const FwdShape s = check_forward(a, w, layout, c10::nullopt);
    check_f32_2d(grad, "grad");
    TORCH_CHECK(grad.size(0) == s.N && grad.size(1) == s.M, "grad must be (batch, out_features)");
    check_same_device(a, grad, "grad");
    check_index(argmax, grad, "argmax");
    check_index(argmin, grad, "argmin");
    const float *w_sel_ptr = nullptr, *x_sel_ptr = nullptr;
    if (sel.has_value() && sel->defined() && sel->numel() > 0) {
        TORCH_CHECK(sel->is_cuda() && sel->scalar_type() == at::kFloat && sel->is_contiguous() &&
                        sel->dim() == 3 && sel->size(0) == 4 && sel->size(1) == s.N && sel->size(2) == s.M,
                    "sel must be a contiguous float32 GPU tensor of shape (4, batch, out_features)");
        check_same_device(a, *sel, "sel");
        w_sel_ptr = sel->data_ptr<float>();
        x_sel_ptr = w_sel_ptr + 2 * s.N * s.M;
    }
    const c10::DeviceGuard guard(a.device());
    const at::Tensor g = grad.contiguous();
    auto a_grad = at::empty({s.N, s.K}, a.options());
    auto w_grad = at::empty(w.sizes(), w.options());
    check_rc(mam_fc_backward(a.data_ptr<float>(), row_stride(a, "a"), w.data_ptr<float>(),
                             row_stride(w, "the weight operand"), layout, g.data_ptr<float>(),
                             argmax.data_ptr<int32_t>(), argmin.data_ptr<int32_t>(), w_sel_ptr, x_sel_ptr,
                             a_grad.data_ptr<float>(), w_grad.data_ptr<float>(), s.N, s.K, s.M,
                             current_stream(a)),
             "mam_fc_backward");
    return {a_grad, w_grad};
}

// ---- reference operator names: b is (in_features, out_features).  Rows of a and b may be
// strided views (the module's splits > 1 path narrows them); the reference reads such views as if
// they were contiguous. ----
std::vector<at::Tensor> fullyconnected(at::Tensor a, at::Tensor b)
{
    return forward_impl(a, b, MAM_W_KM, c10::nullopt, false, false);
}

at::Tensor fullyconnected_fast(at::Tensor a, at::Tensor b)
{
    return forward_values_impl(a, b, MAM_W_KM, c10::nullopt);
}

std::vector<at::Tensor> fullyconnected_backward(at::Tensor a, at::Tensor b, at::Tensor grad,
                                                at::Tensor argmax, at::Tensor argmin)
{
    return backward_impl(a, b, MAM_W_KM, grad, argmax, argmin, c10::nullopt);
}

// ---- additions: weight in the module's own (out_features, in_features) layout, fused bias ----
std::vector<at::Tensor> fullyconnected_wt(const at::Tensor &a, const at::Tensor &weight,
                                          const c10::optional<at::Tensor> &bias, bool hand_over)
{
    return forward_impl(a, weight, MAM_W_MK, bias, true, hand_over);
}

at::Tensor fullyconnected_fast_wt(const at::Tensor &a, const at::Tensor &weight,
                                  const c10::optional<at::Tensor> &bias)
{
    return forward_values_impl(a, weight, MAM_W_MK, bias);
}

std::vector<at::Tensor> fullyconnected_wt_backward(const at::Tensor &a, const at::Tensor &weight,
                                                   const at::Tensor &grad, const at::Tensor &argmax,
                                                   const at::Tensor &argmin,
                                                   const c10::optional<at::Tensor> &sel)
{
    return backward_impl(a, weight, MAM_W_MK, grad, argmax, argmin, sel);
}

// ---- the module's `splits`: consecutive K ranges, each a MAM neuron of its own, summed ----
std::vector<at::Tensor> fullyconnected_ranges(const at::Tensor &a, const at::Tensor &weight,
                                              const c10::optional<at::Tensor> &bias, int64_t range_len,
                                              bool with_indices)
{
    const FwdShape s = check_forward(a, weight, MAM_W_MK, bias);
    TORCH_CHECK(range_len > 0, "range_len must be positive");
    const c10::DeviceGuard guard(a.device());
    const int64_t ranges = std::max<int64_t>(1, (s.K + range_len - 1) / range_len);
    auto c = at::empty({s.N, s.M}, a.options());
    auto argmax = at::empty({with_indices ? ranges : 0, s.N, s.M}, a.options().dtype(at::kInt));
    auto argmin = at::empty({with_indices ? ranges : 0, s.N, s.M}, a.options().dtype(at::kInt));
    if (s.N == 0 || s.M == 0) return {c, argmax, argmin};
    const size_t ws_bytes = mam_fc_forward_ranges_workspace(s.N, s.K, s.M, range_len, with_indices ? 1 : 0);
    auto ws = workspace_for(ws_bytes, a);
    check_rc(mam_fc_forward_ranges(a.data_ptr<float>(), row_stride(a, "a"), weight.data_ptr<float>(),
                                   row_stride(weight, "weight"), MAM_W_MK, bias_ptr(bias), c.data_ptr<float>(),
                                   with_indices ? argmax.data_ptr<int32_t>() : nullptr,
                                   with_indices ? argmin.data_ptr<int32_t>() : nullptr, s.N, s.K, s.M, range_len,
                                   ws.defined() ? ws.data_ptr() : nullptr, ws_bytes, current_stream(a)),
             "mam_fc_forward_ranges");
    return {c, argmax, argmin};
}

std::vector<at::Tensor> fullyconnected_ranges_backward(const at::Tensor &a, const at::Tensor &weight,
                                                       const at::Tensor &grad, const at::Tensor &argmax,
                                                       const at::Tensor &argmin, int64_t range_len)
{
    const FwdShape s = check_forward(a, weight, MAM_W_MK, c10::nullopt);
    check_f32_2d(grad, "grad");
    TORCH_CHECK(grad.size(0) == s.N && grad.size(1) == s.M, "grad must be (batch, out_features)");
    TORCH_CHECK(range_len > 0, "range_len must be positive");
    const int64_t ranges = std::max<int64_t>(1, (s.K + range_len - 1) / range_len);
    for (const at::Tensor *t : {&argmax, &argmin})
        TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kInt && t->is_contiguous() && t->dim() == 3 &&
                        t->size(0) == ranges && t->size(1) == s.N && t->size(2) == s.M && t->device() == a.device(),
                    "argmax / argmin must be contiguous int32 (ranges, batch, out_features) tensors on a's device");
    const c10::DeviceGuard guard(a.device());
    const at::Tensor g = grad.contiguous();
    auto a_grad = at::empty({s.N, s.K}, a.options());
    auto w_grad = at::empty(weight.sizes(), weight.options());
    check_rc(mam_fc_backward_ranges(a.data_ptr<float>(), row_stride(a, "a"), weight.data_ptr<float>(),
                                    row_stride(weight, "weight"), MAM_W_MK, g.data_ptr<float>(),
                                    argmax.data_ptr<int32_t>(), argmin.data_ptr<int32_t>(), a_grad.data_ptr<float>(),
                                    w_grad.data_ptr<float>(), s.N, s.K, s.M, range_len, current_stream(a)),
             "mam_fc_backward_ranges");
    return {a_grad, w_grad};
}

void selection_count(const at::Tensor &argmax, const at::Tensor &argmin, at::Tensor max_count,
                     at::Tensor min_count, int64_t mode)
{
    TORCH_CHECK(argmax.dim() == 2, "argmax must be (batch, out_features)");
    check_index(argmax, argmax, "argmax");
    check_index(argmin, argmax, "argmin");
    TORCH_CHECK(max_count.dim() == 2 && max_count.size(0) == argmax.size(1),
                "max_count must be (out_features, in_features)");
    check_index(max_count, max_count, "max_count");
    check_index(min_count, max_count, "min_count");
    check_same_device(argmax, max_count, "max_count");
    const c10::DeviceGuard guard(argmax.device());
    check_rc(mam_selection_count(argmax.data_ptr<int32_t>(), argmin.data_ptr<int32_t>(),
                                 max_count.data_ptr<int32_t>(), min_count.data_ptr<int32_t>(),
                                 argmax.size(0), argmax.size(1), max_count.size(1), (int)mode,
                                 current_stream(argmax)),
             "mam_selection_count");
}

// ---- module helpers: the MAC blend, and the window gather / scatter behind the MAM convolutions ----
at::Tensor blend(const at::Tensor &mam, const at::Tensor &mac, const c10::optional<at::Tensor> &bias, double alpha,
                 double beta)
{
    check_f32_2d(mam, "mam");
    check_f32_2d(mac, "mac");
    TORCH_CHECK(mam.sizes() == mac.sizes(), "mam and mac must have the same shape");
    check_same_device(mam, mac, "mac");
    const int64_t N = mam.size(0), M = mam.size(1);
    if (bias.has_value() && bias->defined()) {
        TORCH_CHECK(bias->is_cuda() && bias->scalar_type() == at::kFloat && bias->dim() == 1 && bias->size(0) == M &&
                        bias->is_contiguous(),
                    "bias must be a contiguous float32 GPU vector of out_features elements");
        check_same_device(mam, *bias, "bias");
    }
    const c10::DeviceGuard guard(mam.device());
    const at::Tensor a = mam.contiguous(), b = mac.contiguous();
    auto out = at::empty({N, M}, mam.options());
    check_rc(mam_blend(a.data_ptr<float>(), b.data_ptr<float>(), bias_ptr(bias), (float)alpha, (float)beta,
                       out.data_ptr<float>(), N, M, current_stream(mam)),
             "mam_blend");
    return out;
}

// column sums of the output gradient: the bias gradient of the layer
at::Tensor bias_grad(const at::Tensor &grad)
{
    check_f32_2d(grad, "grad");
    const int64_t N = grad.size(0), M = grad.size(1);
    const c10::DeviceGuard guard(grad.device());
    const at::Tensor g = grad.stride(1) == 1 ? grad : grad.contiguous();
    auto out = at::empty({M}, grad.options());
    const size_t ws_bytes = mam_bias_grad_workspace(N, M);
    auto ws = workspace_for(ws_bytes, grad);
    check_rc(mam_bias_grad(g.data_ptr<float>(), g.stride(0), out.data_ptr<float>(), N, M,
                           ws.defined() ? ws.data_ptr() : nullptr, ws_bytes, current_stream(grad)),
             "mam_bias_grad");
    return out;
}

// weight (out, in) times a {0, 1} mask kept as bool / uint8: the module's weight dropout and its gradient
at::Tensor apply_keep(const at::Tensor &w, const at::Tensor &keep)
{
    check_f32_2d(w, "weight");
    TORCH_CHECK(keep.is_cuda() && (keep.scalar_type() == at::kBool || keep.scalar_type() == at::kByte) &&
                    keep.sizes() == w.sizes() && keep.is_contiguous(),
                "keep must be a contiguous bool or uint8 GPU tensor of the weight's shape");
    check_same_device(w, keep, "keep");
    const c10::DeviceGuard guard(w.device());
    const at::Tensor wc = (w.stride(1) == 1 && w.stride(0) >= w.size(1)) || w.numel() == 0 ? w : w.contiguous();
    auto out = at::empty({w.size(0), w.size(1)}, w.options());
    if (out.numel() > 0)
        check_rc(mam_apply_keep(wc.data_ptr<float>(), wc.stride(0), static_cast<const unsigned char *>(keep.data_ptr()),
                                out.data_ptr<float>(), w.size(0), w.size(1), current_stream(w)),
                 "mam_apply_keep");
    return out;
}

at::Tensor im2col(const at::Tensor &x, int64_t k1, int64_t k2, int64_t s1, int64_t s2)
{
    TORCH_CHECK(x.is_cuda() && x.scalar_type() == at::kFloat && x.dim() == 4, "x must be a float32 GPU tensor (B, C, H, W)");
    TORCH_CHECK(k1 >= 1 && k2 >= 1 && s1 >= 1 && s2 >= 1, "window and stride must be positive");
    TORCH_CHECK(x.size(2) >= k1 && x.size(3) >= k2, "the window is larger than the input");
    const c10::DeviceGuard guard(x.device());
    const at::Tensor xc = x.contiguous();
    const int64_t B = x.size(0), C = x.size(1), H = x.size(2), W = x.size(3);
    const int64_t L1 = (H - k1) / s1 + 1, L2 = (W - k2) / s2 + 1;
    auto cols = at::empty({B * L1 * L2, k2 * k1 * C}, x.options());
    if (cols.numel() > 0)
        check_rc(mam_im2col(xc.data_ptr<float>(), cols.data_ptr<float>(), B, C, H, W, k1, k2, s1, s2, current_stream(x)),
                 "mam_im2col");
    return cols;
}

at::Tensor col2im(const at::Tensor &cols, int64_t B, int64_t C, int64_t H, int64_t W, int64_t k1, int64_t k2,
                  int64_t s1, int64_t s2)
{
    check_f32_2d(cols, "cols");
    TORCH_CHECK(k1 >= 1 && k2 >= 1 && s1 >= 1 && s2 >= 1 && H >= k1 && W >= k2, "bad window geometry");
    const int64_t L1 = (H - k1) / s1 + 1, L2 = (W - k2) / s2 + 1;
    TORCH_CHECK(cols.size(0) == B * L1 * L2 && cols.size(1) == k2 * k1 * C, "cols does not match the geometry");
    const c10::DeviceGuard guard(cols.device());
    const at::Tensor cc = cols.contiguous();
    auto xg = at::empty({B, C, H, W}, cols.options());
    if (xg.numel() > 0)
        check_rc(mam_col2im(cc.data_ptr<float>(), xg.data_ptr<float>(), B, C, H, W, k1, k2, s1, s2, current_stream(cols)),
                 "mam_col2im");
    return xg;
}

// ---- CSR-sparse MAM: w_csr is the pruned weight (out_features, in_features) ----
struct CsrParts { at::Tensor crow, col, val; };

CsrParts csr_parts(const at::Tensor &w_csr, const at::Tensor &a)
{
    TORCH_CHECK(w_csr.layout() == at::kSparseCsr, "w_csr must be a torch.sparse_csr tensor");
    TORCH_CHECK(w_csr.dim() == 2 && w_csr.size(1) == a.size(1), "w_csr must be (out_features, in_features)");
    CsrParts p{w_csr.crow_indices().to(at::kLong).contiguous(), w_csr.col_indices().to(at::kLong).contiguous(),
               w_csr.values().contiguous()};
    TORCH_CHECK(p.val.scalar_type() == at::kFloat, "w_csr values must be float32");
    TORCH_CHECK(p.val.is_cuda() && p.val.device() == a.device(), "w_csr is on a different device");
    return p;
}

std::vector<at::Tensor> sparse_forward_impl(const at::Tensor &a, const at::Tensor &w_csr, bool hand_over)
{
    check_f32_2d(a, "a");
    const CsrParts p = csr_parts(w_csr, a);
    const int64_t N = a.size(0), K = a.size(1), M = w_csr.size(0);
    TORCH_CHECK(K > 0 || N == 0 || M == 0, "in_features must be positive");
    const c10::DeviceGuard guard(a.device());
    auto c = at::empty({N, M}, a.options());
    auto argmax = at::empty({N, M}, a.options().dtype(at::kInt));
    auto argmin = at::empty({N, M}, a.options().dtype(at::kInt));
    at::Tensor w_sel, pos_sel;
    if (hand_over) {
        // planes 0, 1: the selected stored values; planes 2, 3: the selected inputs
        w_sel = at::empty({4, N, M}, a.options());
        pos_sel = at::empty({2, N, M}, a.options().dtype(at::kInt));
    }
    if (N > 0 && M > 0) {
        const size_t need = mam_csr_fc_forward_workspace(N, K, M);
        auto ws = at::empty({(int64_t)(need ? need : 1)}, a.options().dtype(at::kByte));
        check_rc(mam_csr_fc_forward(a.data_ptr<float>(), row_stride(a, "a"), p.crow.data_ptr<int64_t>(),
                                    p.col.data_ptr<int64_t>(), p.val.data_ptr<float>(), nullptr,
                                    c.data_ptr<float>(), argmax.data_ptr<int32_t>(), argmin.data_ptr<int32_t>(),
                                    hand_over ? w_sel.data_ptr<float>() : nullptr,
                                    hand_over ? pos_sel.data_ptr<int32_t>() : nullptr,
                                    hand_over ? w_sel.data_ptr<float>() + 2 * N * M : nullptr, N, K, M,
                                    p.val.numel(), ws.data_ptr(), need, current_stream(a)),
                 "mam_csr_fc_forward");
    }
    if (hand_over) return {c, argmax, argmin, w_sel, pos_sel};
    return {c, argmax, argmin};
}

std::vector<at::Tensor> sparse_fullyconnected(const at::Tensor &a, const at::Tensor &w_csr)
{
    return sparse_forward_impl(a, w_csr, false);
}

std::vector<at::Tensor> sparse_fullyconnected_sel(const at::Tensor &a, const at::Tensor &w_csr)
{
    return sparse_forward_impl(a, w_csr, true);
}

std::vector<at::Tensor> sparse_fullyconnected_sel_backward(const at::Tensor &a, const at::Tensor &w_csr,
                                                           const at::Tensor &grad, const at::Tensor &argmax,
                                                           const at::Tensor &argmin,
                                                           const c10::optional<at::Tensor> &w_sel,
                                                           const c10::optional<at::Tensor> &pos_sel)
{
    check_f32_2d(a, "a");
    check_f32_2d(grad, "grad");
    const CsrParts p = csr_parts(w_csr, a);
    const int64_t N = a.size(0), K = a.size(1), M = w_csr.size(0);
    TORCH_CHECK(grad.size(0) == N && grad.size(1) == M, "grad must be (batch, out_features)");
    check_index(argmax, grad, "argmax");
    check_index(argmin, grad, "argmin");
    const bool handed = w_sel.has_value() && w_sel->defined() && pos_sel.has_value() && pos_sel->defined();
    if (handed) {
        TORCH_CHECK(w_sel->scalar_type() == at::kFloat && w_sel->is_contiguous() && w_sel->dim() == 3 &&
                        (w_sel->size(0) == 2 || w_sel->size(0) == 4) && w_sel->size(1) == N && w_sel->size(2) == M &&
                        w_sel->device() == a.device(),
                    "w_sel must be a contiguous float32 (2 or 4, batch, out_features) tensor on a's device");
        TORCH_CHECK(pos_sel->scalar_type() == at::kInt && pos_sel->is_contiguous() && pos_sel->dim() == 3 &&
                        pos_sel->size(0) == 2 && pos_sel->size(1) == N && pos_sel->size(2) == M &&
                        pos_sel->device() == a.device(),
                    "pos_sel must be a contiguous int32 (2, batch, out_features) tensor on a's device");
    }
    const c10::DeviceGuard guard(a.device());
    const at::Tensor g = grad.contiguous();
    auto a_grad = at::empty({N, K}, a.options());
    auto val_grad = at::empty_like(p.val);
    check_rc(mam_csr_fc_backward(a.data_ptr<float>(), row_stride(a, "a"), p.crow.data_ptr<int64_t>(),
                                 p.col.data_ptr<int64_t>(), p.val.data_ptr<float>(), g.data_ptr<float>(),
                                 argmax.data_ptr<int32_t>(), argmin.data_ptr<int32_t>(),
                                 handed ? w_sel->data_ptr<float>() : nullptr,
                                 handed ? pos_sel->data_ptr<int32_t>() : nullptr,
                                 handed && w_sel->size(0) == 4 ? w_sel->data_ptr<float>() + 2 * N * M : nullptr,
                                 a_grad.data_ptr<float>(), val_grad.data_ptr<float>(), N, K, M, p.val.numel(),
                                 current_stream(a)),
             "mam_csr_fc_backward");
    return {a_grad, val_grad};
}

std::vector<at::Tensor> sparse_fullyconnected_backward(const at::Tensor &a, const at::Tensor &w_csr,
                                                       const at::Tensor &grad, const at::Tensor &argmax,
                                                       const at::Tensor &argmin)
{
    return sparse_fullyconnected_sel_backward(a, w_csr, grad, argmax, argmin, c10::nullopt, c10::nullopt);
}

// ---- sum-of-products SpMM: a sparse (R, K), b dense (K, C) -> dense (R, C) ----
// Schema and keys of mamtorch/sparse/kernel/v1/csrc/cuda/register_functions.cu:18-28.
void check_spmm_operands(const at::Tensor &a, const at::Tensor &b)
{
    check_f32_2d(b, "b");
    TORCH_CHECK(a.dim() == 2 && a.size(1) == b.size(0), "a must be (rows, k) with k = b.size(0)");
    TORCH_CHECK(a.scalar_type() == at::kFloat, "a must be float32");
    TORCH_CHECK(a.device() == b.device(), "a and b are on different devices");
}

// From about one stored entry in eight on, walking the entries (each costs a row of b) takes longer than a
// dense fp32 GEMM over the zero-filled operand: the operand is written out dense (one pass) and the
// product is the platform's library GEMM.  4096 x 4096 x 4096: 3.06 -> ~1.05 ms at 30 % density; the two
// routes cross at ~10 %.
// `one_in`: the density from which the route is taken, one stored entry in `one_in`: 8 for CSR; 16 for COO,
// whose kernel (any order, duplicates, atomics) takes about twice the CSR kernel's time per entry (4096^3 at
// 10 % density: 1.89 against 1.05 ms, the GEMM 0.99 ms).
bool dense_route_pays(int64_t nnz, int64_t R, int64_t K, int64_t C, int64_t one_in)
{
    return R > 0 && K > 0 && C >= 64 && nnz >= (R * K + one_in - 1) / one_in && R * K <= (int64_t(1) << 29);
}

at::Tensor cusparsemm_csr(const at::Tensor &a, const at::Tensor &b)
{
    TORCH_CHECK(a.layout() == at::kSparseCsr, "a must be a torch.sparse_csr tensor");
    check_spmm_operands(a, b);
    const int64_t R = a.size(0), K = a.size(1), C = b.size(1);
    const c10::DeviceGuard guard(b.device());
    const at::Tensor crow = a.crow_indices().to(at::kLong).contiguous();
    const at::Tensor col = a.col_indices().to(at::kLong).contiguous();
    const at::Tensor val = a.values().contiguous();
    if (dense_route_pays(val.numel(), R, K, C, 8)) {
        auto dense = at::empty({R, K}, b.options());
        check_rc(mam_csr_to_dense(crow.data_ptr<int64_t>(), col.data_ptr<int64_t>(), val.data_ptr<float>(),
                                  dense.data_ptr<float>(), K, R, K, current_stream(b)),
                 "mam_csr_to_dense");
        return at::mm(dense, b);
    }
    auto c = at::empty({R, C}, b.options());
    if (R == 0 || C == 0) return c;
    check_rc(mam_csr_spmm(crow.data_ptr<int64_t>(), col.data_ptr<int64_t>(), val.data_ptr<float>(),
                          b.data_ptr<float>(), row_stride(b, "b"), c.data_ptr<float>(), R, K, C,
                          current_stream(b)),
             "mam_csr_spmm");
    return c;
}

at::Tensor cusparsemm_coo(const at::Tensor &a, const at::Tensor &b)
{
    TORCH_CHECK(a.layout() == at::kSparse, "a must be a torch.sparse_coo tensor");
    check_spmm_operands(a, b);
    TORCH_CHECK(a.sparse_dim() == 2 && a.dense_dim() == 0, "a must have two sparse dimensions");
    const int64_t R = a.size(0), K = a.size(1), C = b.size(1);
    const c10::DeviceGuard guard(b.device());
    const at::Tensor idx = a._indices().to(at::kLong).contiguous();   // (2, nnz); need not be coalesced
    const at::Tensor val = a._values().contiguous();
    const int64_t nnz = val.numel();
    if (dense_route_pays(nnz, R, K, C, 16)) {
        auto dense = at::empty({R, K}, b.options());
        check_rc(mam_coo_to_dense(idx.data_ptr<int64_t>(), idx.data_ptr<int64_t>() + nnz, val.data_ptr<float>(), nnz,
                                  dense.data_ptr<float>(), K, R, K, current_stream(b)),
                 "mam_coo_to_dense");
        return at::mm(dense, b);
    }
    auto c = at::empty({R, C}, b.options());
    if (R == 0 || C == 0) return c;
    check_rc(mam_coo_spmm(idx.data_ptr<int64_t>(), idx.data_ptr<int64_t>() + nnz, val.data_ptr<float>(), nnz,
                          b.data_ptr<float>(), row_stride(b, "b"), c.data_ptr<float>(), R, K, C,
                          current_stream(b)),
             "mam_coo_spmm");
    return c;
}

}  // namespace

TORCH_LIBRARY(mamtorch_kernel_v1, m)
{
    m.def("fullyconnected(Tensor a, Tensor b) -> Tensor[]");
    m.def("fullyconnected_backward(Tensor a, Tensor b, Tensor grad, Tensor argmax, Tensor argmin) -> Tensor[]");
}

TORCH_LIBRARY(mamtorch_kernel_v4, m)
{
    m.def("fullyconnected(Tensor a, Tensor b) -> Tensor[]");
    m.def("fullyconnected_fast(Tensor a, Tensor b) -> Tensor");
    m.def("fullyconnected_backward(Tensor a, Tensor b, Tensor grad, Tensor argmax, Tensor argmin) -> Tensor[]");
    m.def("fullyconnected_wt(Tensor a, Tensor weight, Tensor? bias, bool hand_over) -> Tensor[]");
    m.def("fullyconnected_fast_wt(Tensor a, Tensor weight, Tensor? bias) -> Tensor");
    m.def("fullyconnected_wt_backward(Tensor a, Tensor weight, Tensor grad, Tensor argmax, Tensor argmin, Tensor? sel) -> Tensor[]");
    m.def("selection_count(Tensor argmax, Tensor argmin, Tensor(a!) max_count, Tensor(b!) min_count, int mode) -> ()");
    m.def("fullyconnected_ranges(Tensor a, Tensor weight, Tensor? bias, int range_len, bool with_indices) -> Tensor[]");
    m.def("fullyconnected_ranges_backward(Tensor a, Tensor weight, Tensor grad, Tensor argmax, Tensor argmin, int range_len) -> Tensor[]");
    m.def("blend(Tensor mam, Tensor mac, Tensor? bias, float alpha, float beta) -> Tensor");
    m.def("bias_grad(Tensor grad) -> Tensor");
    m.def("apply_keep(Tensor weight, Tensor keep) -> Tensor");
    m.def("im2col(Tensor x, int k1, int k2, int s1, int s2) -> Tensor");
    m.def("col2im(Tensor cols, int B, int C, int H, int W, int k1, int k2, int s1, int s2) -> Tensor");
}

TORCH_LIBRARY(mamtorch_kernel_sparsev1, m)
{
    m.def("fullyconnected(Tensor a, Tensor w_csr) -> Tensor[]");
    m.def("fullyconnected_backward(Tensor a, Tensor w_csr, Tensor grad, Tensor argmax, Tensor argmin) -> Tensor[]");
    m.def("cusparsemm(Tensor a, Tensor b) -> Tensor");
    m.def("fullyconnected_sel(Tensor a, Tensor w_csr) -> Tensor[]");
    m.def("fullyconnected_sel_backward(Tensor a, Tensor w_csr, Tensor grad, Tensor argmax, Tensor argmin, Tensor? w_sel, Tensor? pos_sel) -> Tensor[]");
}

// On PyTorch-ROCm the HIP device is served by the CUDA dispatch key.
TORCH_LIBRARY_IMPL(mamtorch_kernel_v1, CUDA, m)
{
    m.impl("fullyconnected", &fullyconnected);
    m.impl("fullyconnected_backward", &fullyconnected_backward);
}

TORCH_LIBRARY_IMPL(mamtorch_kernel_v4, CUDA, m)
{
    m.impl("fullyconnected", &fullyconnected);
    m.impl("fullyconnected_fast", &fullyconnected_fast);
    m.impl("fullyconnected_backward", &fullyconnected_backward);
    m.impl("fullyconnected_wt", &fullyconnected_wt);
    m.impl("fullyconnected_fast_wt", &fullyconnected_fast_wt);
    m.impl("fullyconnected_wt_backward", &fullyconnected_wt_backward);
    m.impl("selection_count", &selection_count);
    m.impl("fullyconnected_ranges", &fullyconnected_ranges);
    m.impl("fullyconnected_ranges_backward", &fullyconnected_ranges_backward);
    m.impl("blend", &blend);
    m.impl("bias_grad", &bias_grad);
    m.impl("apply_keep", &apply_keep);
    m.impl("im2col", &im2col);
    m.impl("col2im", &col2im);
}

// The dense operand decides the key for mixed dense / sparse-CSR arguments only when the sparse
// key is absent, so the sparse operators are registered on the sparse-CSR key, as the reference
// does for cusparsemm (mamtorch/sparse/kernel/v1/csrc/cuda/register_functions.cu:26-28).
TORCH_LIBRARY_IMPL(mamtorch_kernel_sparsev1, SparseCsrCUDA, m)
{
    m.impl("fullyconnected", &sparse_fullyconnected);
    m.impl("fullyconnected_backward", &sparse_fullyconnected_backward);
    m.impl("fullyconnected_sel", &sparse_fullyconnected_sel);
    m.impl("fullyconnected_sel_backward", &sparse_fullyconnected_sel_backward);
    m.impl("cusparsemm", &cusparsemm_csr);
}

TORCH_LIBRARY_IMPL(mamtorch_kernel_sparsev1, SparseCUDA, m)
{
    m.impl("cusparsemm", &cusparsemm_coo);
}
