// repdl_amd.backend._hip_ext -- the compiled counterpart of RepDL's repdl.backend.cuda
// (backend/cuda/bind.cpp:6-19): a PyTorch C++ extension module that exports the same ten
// functions with the same positional signatures (matrix_multiplication.cu:234-235, 267;
// convolution.cu:153-155, 259-262, 359-362, 385-387; summation.cu:149-155;
// softmax.cpp:15, 28; cross_entropy.cpp:15, 31), plus exp / log / sqrt / div / div_scalar and
// mm_bias / conv2d_bias (the layer's bias added in the kernel's epilogue) and the fused elementwise
// passes of batch normalisation (bn_apply, bn_gvar_term, bn_gweight_term).
// It is the only file of this library that knows about PyTorch: every function checks its
// tensors, allocates the output on the input's device, and hands raw pointers and the current
// stream to the C ABI of include/repdl_hip.h.  Host C++ only; built with the host compiler
// against the PyTorch headers (repdl_amd/build.py, build_ext).
#include <torch/extension.h>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include "../../include/repdl_hip.h"

namespace repdl
{
namespace hip
{
namespace
{
// PyTorch-ROCm presents HIP devices and streams under the CUDA names.
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;

void *current_stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

torch::Tensor checked(const torch::Tensor &t, const char *name, int64_t dim, c10::ScalarType dtype = torch::kFloat)
{
    TORCH_CHECK(t.is_cuda(), name, " must be on the GPU (this backend has no CPU path)");
    TORCH_CHECK(t.scalar_type() == dtype, name, " must be ", dtype, ", got ", t.scalar_type());
    TORCH_CHECK(dim < 0 || t.dim() == dim, name, " must have ", dim, " dimensions, got ", t.dim());
    return t.contiguous();
}

void same_device(const torch::Tensor &a, const torch::Tensor &b)
{
    TORCH_CHECK(a.device() == b.device(), "tensors are on different devices: ", a.device(), " and ", b.device());
}

void ok(int rc, const char *what) { TORCH_CHECK(rc == 0, what, " failed with code ", rc, ": ", repdl_hip_error_string(rc)); }

// Scratch memory of a call from PyTorch's allocator (the *_ws entry points): the library then allocates,
// frees and keeps nothing of its own, and the call can be captured into a graph like any PyTorch operator.
// The tensor dies when the binding returns; PyTorch hands its memory to later work on the same stream only.
struct Scratch
{
    torch::Tensor hold;
    size_t bytes;
    Scratch(size_t nbytes, const torch::Tensor &like) : bytes(nbytes)
    {
        if (nbytes > 0)
            hold = torch::empty({(int64_t)nbytes}, like.options().dtype(torch::kUInt8));
    }
    void *ptr() const { return bytes > 0 ? hold.data_ptr() : nullptr; }
};
} // namespace

namespace
{
// the bias of a layer: [channels] on the same device, or none
const float *bias_pointer(const c10::optional<torch::Tensor> &bias, torch::Tensor &hold, const torch::Tensor &like,
                          int64_t channels)
{
    if (!bias.has_value())
        return nullptr;
    hold = checked(*bias, "bias", 1);
    same_device(hold, like);
    TORCH_CHECK(hold.size(0) == channels, "bias has ", hold.size(0), " elements for ", channels, " output channels");
    return hold.data_ptr<float>();
}
} // namespace

// mm followed by `+= bias` (repdl/nn/linear.py:21-22) with the addition in the kernel's epilogue
torch::Tensor mm_bias(const torch::Tensor &input, const torch::Tensor &mat2, const c10::optional<torch::Tensor> &bias,
                      bool transA, bool transB)
{
    const auto a = checked(input, "input", 2), b = checked(mat2, "mat2", 2);
    same_device(a, b);
    const int64_t M = !transA ? a.size(0) : a.size(1), K = !transA ? a.size(1) : a.size(0);
    const int64_t N = !transB ? b.size(1) : b.size(0), Kb = !transB ? b.size(0) : b.size(1);
    TORCH_CHECK(K == Kb, "mm: inner dimensions differ (", K, " vs ", Kb, ")");
    const DeviceGuard guard(a.device());
    torch::Tensor hold;
    const float *bp = bias_pointer(bias, hold, a, N);
    auto out = torch::empty({M, N}, a.options());
    ok(repdl_hip_mm_bias(a.data_ptr<float>(), b.data_ptr<float>(), bp, out.data_ptr<float>(), M, N, K, transA, transB,
                         current_stream()),
       "repdl_hip_mm");
    return out;
}

torch::Tensor mm(const torch::Tensor &input, const torch::Tensor &mat2, bool transA, bool transB)
{
    return mm_bias(input, mat2, c10::nullopt, transA, transB);
}

// conv2d followed by `+= bias` per output channel (repdl/nn/conv.py:27-28), the addition in the epilogue
torch::Tensor conv2d_bias(const torch::Tensor &input, const torch::Tensor &kernel, const c10::optional<torch::Tensor> &bias,
                          int64_t sH, int64_t sW, int64_t pH, int64_t pW, int64_t groups)
{
    const auto x = checked(input, "input", 4), k = checked(kernel, "kernel", 4);
    same_device(x, k);
    const int64_t N = x.size(0), IC = x.size(1), H = x.size(2), W = x.size(3);
    const int64_t OC = k.size(0), ICg = k.size(1), KH = k.size(2), KW = k.size(3);
    TORCH_CHECK(groups > 0 && IC % groups == 0 && OC % groups == 0 && ICg == IC / groups, "conv2d: channels (", IC,
                " in, ", OC, " out, kernel ", ICg, ") do not match groups=", groups);
    TORCH_CHECK(sH > 0 && sW > 0 && pH >= 0 && pW >= 0, "conv2d: bad stride or padding");
    TORCH_CHECK(H + 2 * pH >= KH && W + 2 * pW >= KW, "conv2d: kernel larger than padded input");
    const int64_t OH = (H + 2 * pH - KH) / sH + 1, OW = (W + 2 * pW - KW) / sW + 1;
    const DeviceGuard guard(x.device());
    torch::Tensor hold;
    const float *bp = bias_pointer(bias, hold, x, OC);
    auto out = torch::empty({N, OC, OH, OW}, x.options());
    const Scratch work(repdl_hip_conv2d_workspace_bytes(x.data_ptr<float>(), k.data_ptr<float>(), N, IC, H, W, OC, KH, KW, sH, sW,
                                                        pH, pW, groups),
                       x);
    ok(repdl_hip_conv2d_ws(x.data_ptr<float>(), k.data_ptr<float>(), bp, out.data_ptr<float>(), N, IC, H, W, OC, KH, KW, sH,
                           sW, pH, pW, groups, work.ptr(), work.bytes, current_stream()),
       "repdl_hip_conv2d_ws");
    return out;
}

torch::Tensor conv2d(const torch::Tensor &input, const torch::Tensor &kernel, int64_t sH, int64_t sW, int64_t pH,
                     int64_t pW, int64_t groups)
{
    return conv2d_bias(input, kernel, c10::nullopt, sH, sW, pH, pW, groups);
}

torch::Tensor conv2d_grad_input(const torch::Tensor &grad_output, const torch::Tensor &kernel, int64_t H, int64_t W,
                                int64_t sH, int64_t sW, int64_t pH, int64_t pW)
{
    const auto go = checked(grad_output, "grad_output", 4), k = checked(kernel, "kernel", 4);
    same_device(go, k);
    const int64_t N = go.size(0), OC = go.size(1), OH = go.size(2), OW = go.size(3);
    const int64_t IC = k.size(1), KH = k.size(2), KW = k.size(3);
    TORCH_CHECK(k.size(0) == OC, "conv2d_grad_input: grad_output has ", OC, " channels, kernel has ", k.size(0));
    const DeviceGuard guard(go.device());
    auto out = torch::empty({N, IC, H, W}, go.options());
    const Scratch work(repdl_hip_conv2d_grad_input_workspace_bytes(go.data_ptr<float>(), k.data_ptr<float>(), N, OC, OH, OW, IC, KH,
                                                                   KW, H, W, sH, sW, pH, pW),
                       go);
    ok(repdl_hip_conv2d_grad_input_ws(go.data_ptr<float>(), k.data_ptr<float>(), out.data_ptr<float>(), N, OC, OH, OW, IC,
                                      KH, KW, H, W, sH, sW, pH, pW, work.ptr(), work.bytes, current_stream()),
       "repdl_hip_conv2d_grad_input_ws");
    return out;
}

torch::Tensor conv2d_grad_kernel(const torch::Tensor &grad_output, const torch::Tensor &input, int64_t KH, int64_t KW,
                                 int64_t sH, int64_t sW, int64_t pH, int64_t pW)
{
    const auto go = checked(grad_output, "grad_output", 4), x = checked(input, "input", 4);
    same_device(go, x);
    const int64_t N = x.size(0), IC = x.size(1), H = x.size(2), W = x.size(3);
    const int64_t OC = go.size(1), OH = go.size(2), OW = go.size(3);
    TORCH_CHECK(go.size(0) == N, "conv2d_grad_kernel: batch sizes differ (", N, " vs ", go.size(0), ")");
    const DeviceGuard guard(x.device());
    auto out = torch::empty({OC, IC, KH, KW}, x.options());
    const Scratch work(repdl_hip_conv2d_grad_kernel_workspace_bytes(go.data_ptr<float>(), x.data_ptr<float>(), N, IC, H, W, OC, OH,
                                                                    OW, KH, KW, sH, sW, pH, pW),
                       x);
    ok(repdl_hip_conv2d_grad_kernel_ws(go.data_ptr<float>(), x.data_ptr<float>(), out.data_ptr<float>(), N, IC, H, W, OC,
                                       OH, OW, KH, KW, sH, sW, pH, pW, work.ptr(), work.bytes, current_stream()),
       "repdl_hip_conv2d_grad_kernel_ws");
    return out;
}

torch::Tensor sum1d(const torch::Tensor &input, bool average)
{
    const auto x = checked(input, "input", 1);
    const int64_t n = x.size(0);
    const DeviceGuard guard(x.device());
    auto out = torch::empty({}, x.options());
    // scratch for the parallel evaluation of the sequential chain
    const Scratch work(repdl_hip_sum1d_workspace_bytes(n), x);
    ok(repdl_hip_sum1d_ws(x.data_ptr<float>(), out.data_ptr<float>(), n, average, work.ptr(), work.bytes, current_stream()),
       "repdl_hip_sum1d_ws");
    return out;
}

torch::Tensor sum2d_dim0(const torch::Tensor &input, bool keepdim, bool average)
{
    const auto x = checked(input, "input", 2);
    const DeviceGuard guard(x.device());
    auto out = torch::empty({1, x.size(1)}, x.options());
    ok(repdl_hip_sum2d_dim0(x.data_ptr<float>(), out.data_ptr<float>(), x.size(0), x.size(1), average, current_stream()),
       "repdl_hip_sum2d_dim0");
    return keepdim ? out : out.squeeze();
}

torch::Tensor sum2d_dim1(const torch::Tensor &input, bool keepdim, bool average)
{
    const auto x = checked(input, "input", 2);
    const DeviceGuard guard(x.device());
    auto out = torch::empty({x.size(0), 1}, x.options());
    const Scratch work(repdl_hip_sum2d_dim1_workspace_bytes(x.size(0), x.size(1)), x);
    ok(repdl_hip_sum2d_dim1_ws(x.data_ptr<float>(), out.data_ptr<float>(), x.size(0), x.size(1), average, work.ptr(), work.bytes,
                               current_stream()),
       "repdl_hip_sum2d_dim1_ws");
    return keepdim ? out : out.squeeze();
}

torch::Tensor sum4d_dim023(const torch::Tensor &input, bool keepdim, bool average)
{
    const auto x = checked(input, "input", 4);
    const DeviceGuard guard(x.device());
    auto out = torch::empty({1, x.size(1), 1, 1}, x.options());
    const Scratch work(repdl_hip_sum4d_dim023_workspace_bytes(x.size(0), x.size(1), x.size(2), x.size(3)), x);
    ok(repdl_hip_sum4d_dim023_ws(x.data_ptr<float>(), out.data_ptr<float>(), x.size(0), x.size(1), x.size(2), x.size(3),
                                 average, work.ptr(), work.bytes, current_stream()),
       "repdl_hip_sum4d_dim023_ws");
    return keepdim ? out : out.squeeze();
}

namespace
{
template <typename F>
torch::Tensor unary(const torch::Tensor &input, F fn, const char *what)
{
    const auto x = checked(input, "input", -1);
    const DeviceGuard guard(x.device());
    auto out = torch::empty_like(x);
    ok(fn(x.data_ptr<float>(), out.data_ptr<float>(), x.numel(), current_stream()), what);
    return out;
}
} // namespace

torch::Tensor exp(const torch::Tensor &input) { return unary(input, repdl_hip_exp, "repdl_hip_exp"); }
torch::Tensor log(const torch::Tensor &input) { return unary(input, repdl_hip_log, "repdl_hip_log"); }
torch::Tensor sqrt(const torch::Tensor &input) { return unary(input, repdl_hip_sqrt, "repdl_hip_sqrt"); }

torch::Tensor div_scalar(const torch::Tensor &input, double other)
{
    const auto x = checked(input, "input", -1);
    const DeviceGuard guard(x.device());
    auto out = torch::empty_like(x);
    ok(repdl_hip_div_scalar(x.data_ptr<float>(), (float)other, out.data_ptr<float>(), x.numel(), current_stream()),
       "repdl_hip_div_scalar");
    return out;
}

// input / other elementwise; `other` is broadcast to the common shape; a 0-dim `other` goes
// through the scalar entry point (repdl/ops.py:98-103 divides by Python numbers and tensors alike)
torch::Tensor div(const torch::Tensor &input, const torch::Tensor &other)
{
    if (other.dim() == 0)
        return div_scalar(input, other.item<double>());
    auto x = checked(input, "input", -1), y = checked(other, "other", -1);
    same_device(x, y);
    const auto shape = at::infer_size(x.sizes(), y.sizes());
    x = x.expand(shape).contiguous();
    y = y.expand(shape).contiguous();
    const DeviceGuard guard(x.device());
    auto out = torch::empty(shape, x.options());
    ok(repdl_hip_div(x.data_ptr<float>(), y.data_ptr<float>(), out.data_ptr<float>(), out.numel(), current_stream()),
       "repdl_hip_div");
    return out;
}

torch::Tensor softmax(const torch::Tensor &input)
{
    const auto x = checked(input, "input", 2);
    const DeviceGuard guard(x.device());
    auto out = torch::empty_like(x);
    ok(repdl_hip_softmax(x.data_ptr<float>(), out.data_ptr<float>(), x.size(0), x.size(1), current_stream()),
       "repdl_hip_softmax");
    return out;
}

torch::Tensor cross_entropy(const torch::Tensor &input, const torch::Tensor &target)
{
    const auto x = checked(input, "input", 2), t = checked(target, "target", 1, torch::kLong);
    same_device(x, t);
    TORCH_CHECK(t.size(0) == x.size(0), "cross_entropy: ", x.size(0), " rows but ", t.size(0), " targets");
    const DeviceGuard guard(x.device());
    auto out = torch::empty({}, x.options());
    // the row losses and the scratch of their mean
    const Scratch work(repdl_hip_cross_entropy_workspace_bytes(x.size(0), x.size(1)), x);
    ok(repdl_hip_cross_entropy_ws(x.data_ptr<float>(), t.data_ptr<int64_t>(), out.data_ptr<float>(), x.size(0), x.size(1),
                                  work.ptr(), work.bytes, current_stream()),
       "repdl_hip_cross_entropy_ws");
    return out;
}
namespace
{
// [N,C,H,W] or [B,F] with per-channel vectors -> outer, channels, inner
void bn_geometry(const torch::Tensor &x, std::initializer_list<torch::Tensor> vectors, int64_t &outer, int64_t &channels,
                 int64_t &inner)
{
    TORCH_CHECK(x.dim() == 4 || x.dim() == 2, "batch norm takes 2-D or 4-D tensors, got ", x.dim(), " dimensions");
    outer = x.size(0);
    channels = x.size(1);
    inner = x.dim() == 4 ? x.size(2) * x.size(3) : 1;
    for (const auto &v : vectors)
    {
        TORCH_CHECK(v.numel() == channels, "a per-channel vector has ", v.numel(), " elements for ", channels, " channels");
        same_device(v, x);
    }
}
} // namespace

// ((input - mean) / std) * weight + bias per channel, every operation rounded (repdl/nn/batchnorm.py:25-32)
torch::Tensor bn_apply(const torch::Tensor &input, const torch::Tensor &mean, const torch::Tensor &std,
                       const torch::Tensor &weight, const torch::Tensor &bias)
{
    const auto x = checked(input, "input", -1);
    const auto m = checked(mean, "mean", 1), s = checked(std, "std", 1), w = checked(weight, "weight", 1),
               b = checked(bias, "bias", 1);
    int64_t outer, channels, inner;
    bn_geometry(x, {m, s, w, b}, outer, channels, inner);
    const DeviceGuard guard(x.device());
    auto out = torch::empty_like(x);
    ok(repdl_hip_bn_apply(x.data_ptr<float>(), m.data_ptr<float>(), s.data_ptr<float>(), w.data_ptr<float>(),
                          b.data_ptr<float>(), out.data_ptr<float>(), outer, channels, inner, current_stream()),
       "repdl_hip_bn_apply");
    return out;
}

// (grad_output * (mean - input)) * coef per channel: what grad_var sums (repdl/nn/batchnorm.py:56-58)
torch::Tensor bn_gvar_term(const torch::Tensor &grad_output, const torch::Tensor &input, const torch::Tensor &mean,
                           const torch::Tensor &coef)
{
    const auto g = checked(grad_output, "grad_output", -1), x = checked(input, "input", -1);
    const auto m = checked(mean, "mean", 1), c = checked(coef, "coef", 1);
    TORCH_CHECK(g.sizes() == x.sizes(), "grad_output and input differ in shape");
    same_device(g, x);
    int64_t outer, channels, inner;
    bn_geometry(x, {m, c}, outer, channels, inner);
    const DeviceGuard guard(x.device());
    auto out = torch::empty_like(x);
    ok(repdl_hip_bn_gvar_term(g.data_ptr<float>(), x.data_ptr<float>(), m.data_ptr<float>(), c.data_ptr<float>(),
                              out.data_ptr<float>(), outer, channels, inner, current_stream()),
       "repdl_hip_bn_gvar_term");
    return out;
}

// ((input - mean) / std) * grad_output per channel: what grad_weight sums (repdl/nn/batchnorm.py:60-61)
torch::Tensor bn_gweight_term(const torch::Tensor &input, const torch::Tensor &mean, const torch::Tensor &std,
                              const torch::Tensor &grad_output)
{
    const auto x = checked(input, "input", -1), g = checked(grad_output, "grad_output", -1);
    const auto m = checked(mean, "mean", 1), s = checked(std, "std", 1);
    TORCH_CHECK(g.sizes() == x.sizes(), "grad_output and input differ in shape");
    same_device(g, x);
    int64_t outer, channels, inner;
    bn_geometry(x, {m, s}, outer, channels, inner);
    const DeviceGuard guard(x.device());
    auto out = torch::empty_like(x);
    ok(repdl_hip_bn_gweight_term(x.data_ptr<float>(), m.data_ptr<float>(), s.data_ptr<float>(), g.data_ptr<float>(),
                                 out.data_ptr<float>(), outer, channels, inner, current_stream()),
       "repdl_hip_bn_gweight_term");
    return out;
}

} // namespace hip
} // namespace repdl

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    namespace h = repdl::hip;
    // Importing the module touches no device.  The one-time check of the matrix instructions runs inside the
    // first GEMM-shaped call on a device, or when the program calls init() -- which a program that captures
    // graphs does before its first capture (a check cannot run under capture).
    m.def("init", []() {
        const int rc = repdl_hip_init();
        TORCH_CHECK(rc == 0, "repdl_hip_init failed with code ", rc, ": ", repdl_hip_error_string(rc));
    });
    m.def("conv2d", &h::conv2d);
    m.def("conv2d_grad_input", &h::conv2d_grad_input);
    m.def("conv2d_grad_kernel", &h::conv2d_grad_kernel);
    m.def("cross_entropy", &h::cross_entropy);
    m.def("mm", &h::mm);
    m.def("softmax", &h::softmax);
    m.def("sum1d", &h::sum1d, py::arg("input"), py::arg("average") = false);
    m.def("sum2d_dim0", &h::sum2d_dim0, py::arg("input"), py::arg("keepdim") = false, py::arg("average") = false);
    m.def("sum2d_dim1", &h::sum2d_dim1, py::arg("input"), py::arg("keepdim") = false, py::arg("average") = false);
    m.def("sum4d_dim023", &h::sum4d_dim023, py::arg("input"), py::arg("keepdim") = false, py::arg("average") = false);
    m.def("exp", &h::exp);
    m.def("log", &h::log);
    m.def("sqrt", &h::sqrt);
    m.def("div", &h::div);
    m.def("div_scalar", &h::div_scalar);
    m.def("mm_bias", &h::mm_bias);
    m.def("conv2d_bias", &h::conv2d_bias);
    m.def("bn_apply", &h::bn_apply);
    m.def("bn_gvar_term", &h::bn_gvar_term);
    m.def("bn_gweight_term", &h::bn_gweight_term);
}
