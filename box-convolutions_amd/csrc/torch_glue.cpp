// Host-side fast path of BoxConv2d's forward and backward: the autograd node in C++.
//
// What it replaces: the Python glue around the two native calls of a training step,
//   box_convolution/box_convolution_function.py (BoxConvolutionFunction.forward / .backward, the
//   counterpart of the reference's box_convolution/box_convolution_function.py:30-65) and the
//   tensor-level checks and allocations of box_convolution/_native.py,
// for the common case only: float32 or float64, or float16 / bfloat16 tensors with float32
// parameters, everything on one GPU; training mode (parameters clipped on the way in) and eval
// mode (parameters only read). On the layer shapes of the reference's model zoo the kernels of
// a step take under 100 us, and the Python versions of this glue cost more than that per step
// (argument checks, seven tensor allocations, two ctypes calls with 22 and 24 arguments, and the
// autograd engine calling back into Python from its own thread). Here the engine calls straight
// into C++.
//
// This file contains no arithmetic and links to nothing but libtorch: the kernels stay behind
// the C ABI of libboxconv_hip.so (include/boxconv.h), whose entry points are handed over as
// plain function addresses by box_convolution/_native.py at start-up (init). PyTorch is used for
// device memory, the autograd graph and error reporting only.

#include <torch/extension.h>

#include <cstdint>
#include <mutex>
#include <unordered_map>

namespace {

// ---- the C ABI entry points this file calls (signatures: include/boxconv.h) --------------------
template <class T>
using TrainingForwardFn = int (*)(const T*, T*, T*, T*, T*, T*, T*, T*, int, int, int, int, int, double, double,
                                  double, double, int, int, void*, size_t, void*);
template <class T>
using BackwardFn = int (*)(const T*, const T*, const T*, const T*, const T*, const T*, const T*, float, float,
                           int, int, T*, T*, T*, T*, T*, int, int, int, int, int, void*, size_t, void*);
template <class T>
using InferenceForwardFn = int (*)(const T*, const T*, const T*, const T*, const T*, T*, T*, T*, int, int, int, int,
                                   int, double, double, int, int, void*, size_t, void*);
using TrainingForwardHalfFn = int (*)(const void*, int, float*, float*, float*, float*, float*, float*, void*, int,
                                      int, int, int, int, double, double, double, double, int, int, int, void*,
                                      size_t, void*);
using BackwardHalfFn = int (*)(const float*, const float*, const float*, const float*, const float*, const void*,
                               int, float, float, int, int, void*, float*, float*, float*, float*, int, int, int,
                               int, int, void*, size_t, void*);
using IntegralWorkspaceFn = size_t (*)(int64_t, int, int);
using BackwardWorkspaceFn = size_t (*)(int, int, int, int, int, int, int, int);
using LastErrorFn = const char* (*)();

struct Abi {
    void* training_forward_f32 = nullptr;
    void* training_forward_f64 = nullptr;
    void* inference_forward_f32 = nullptr;
    void* inference_forward_f64 = nullptr;
    void* backward_f32 = nullptr;
    void* backward_f64 = nullptr;
    TrainingForwardHalfFn training_forward_half = nullptr;
    BackwardHalfFn backward_half = nullptr;
    IntegralWorkspaceFn integral_workspace_bytes = nullptr;
    BackwardWorkspaceFn backward_workspace_bytes = nullptr;
    LastErrorFn last_error = nullptr;
} g_abi;

template <class T> TrainingForwardFn<T> training_forward_fn();
template <> TrainingForwardFn<float> training_forward_fn<float>() {
    return reinterpret_cast<TrainingForwardFn<float>>(g_abi.training_forward_f32);
}
template <> TrainingForwardFn<double> training_forward_fn<double>() {
    return reinterpret_cast<TrainingForwardFn<double>>(g_abi.training_forward_f64);
}
template <class T> InferenceForwardFn<T> inference_forward_fn();
template <> InferenceForwardFn<float> inference_forward_fn<float>() {
    return reinterpret_cast<InferenceForwardFn<float>>(g_abi.inference_forward_f32);
}
template <> InferenceForwardFn<double> inference_forward_fn<double>() {
    return reinterpret_cast<InferenceForwardFn<double>>(g_abi.inference_forward_f64);
}
template <class T> BackwardFn<T> backward_fn();
template <> BackwardFn<float> backward_fn<float>() { return reinterpret_cast<BackwardFn<float>>(g_abi.backward_f32); }
template <> BackwardFn<double> backward_fn<double>() { return reinterpret_cast<BackwardFn<double>>(g_abi.backward_f64); }

void check_rc(int rc, const char* what) {
    TORCH_CHECK(rc == 0, "box_convolution: ", what, " failed (code ", rc, "): ",
                g_abi.last_error ? g_abi.last_error() : "");
}

// ---- scratch memory ------------------------------------------------------------------------------
// One buffer per (device, stream), grown on demand: every native call needs its scratch only until
// its own kernels have run, and calls on one stream run in order. A stream that is being captured
// into a graph gets a fresh allocation instead (from the capture's own pool): a cached buffer may
// be replaced, and so freed, by a later, larger call while the graph still points at it.
std::mutex g_ws_mutex;
std::unordered_map<uint64_t, at::Tensor> g_workspaces;

at::Tensor workspace(size_t nbytes, const at::Device& device, uint64_t stream, bool capturing) {
    if (nbytes == 0) return at::Tensor();
    const auto opts = at::TensorOptions().dtype(at::kByte).device(device);
    if (capturing) return at::empty({static_cast<int64_t>(nbytes)}, opts);
    const uint64_t key = (static_cast<uint64_t>(device.index()) << 56) ^ stream;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    at::Tensor& ws = g_workspaces[key];
    if (!ws.defined() || static_cast<size_t>(ws.numel()) < nbytes) {
        ws = at::Tensor();                          // released before the larger one is requested
        ws = at::empty({static_cast<int64_t>(nbytes)}, opts);
    }
    return ws;
}

void* ptr_or_null(const at::Tensor& t) { return t.defined() ? t.data_ptr() : nullptr; }

bool is_half(at::ScalarType t) { return t == at::kHalf || t == at::kBFloat16; }
int half_code(at::ScalarType t) { return t == at::kHalf ? 1 : 2; }     // BOXCONV_F16, BOXCONV_BF16

// ---- the autograd node -----------------------------------------------------------------------------
struct TrainingStep : public torch::autograd::Function<TrainingStep> {
    // Returns the output [B, C*F, h, w]. x_min .. y_max are the stored parameters, clipped in place
    // if `clip` (training mode), only read otherwise (eval mode).
    static at::Tensor forward(torch::autograd::AutogradContext* ctx, const at::Tensor& input,
                              const at::Tensor& x_min, const at::Tensor& x_max, const at::Tensor& y_min,
                              const at::Tensor& y_max, double reparam_h, double reparam_w, double max_h,
                              double max_w, bool normalize, bool exact, bool clip, int64_t stream,
                              bool capturing) {
        const at::Tensor in = input.contiguous();
        const int64_t B = in.size(0), C = in.size(1), h = in.size(2), w = in.size(3), F = x_min.size(1);
        const bool half = is_half(in.scalar_type());
        // (half tensors: float32 integral image and bounds; the kernels read and write the half type)
        const auto opts = half ? in.options().dtype(at::kFloat) : in.options();
        at::Tensor integrated = at::empty({B, C, h + 1, w + 1}, opts);
        at::Tensor output = at::empty({B, C * F, h, w}, in.options());
        at::Tensor real = at::empty({4, C, F}, opts);
        const size_t nbytes = g_abi.integral_workspace_bytes(B * C, static_cast<int>(h), static_cast<int>(w));
        at::Tensor ws = workspace(nbytes, in.device(), static_cast<uint64_t>(stream), capturing);
        if (half)
            check_rc(g_abi.training_forward_half(
                         in.data_ptr(), half_code(in.scalar_type()), x_min.data_ptr<float>(),
                         x_max.data_ptr<float>(), y_min.data_ptr<float>(), y_max.data_ptr<float>(),
                         real.data_ptr<float>(), integrated.data_ptr<float>(), output.data_ptr(),
                         static_cast<int>(B), static_cast<int>(C), static_cast<int>(F), static_cast<int>(h),
                         static_cast<int>(w), reparam_h, reparam_w, max_h, max_w, clip ? 1 : 0, normalize ? 1 : 0,
                         exact ? 1 : 0, ptr_or_null(ws), nbytes, reinterpret_cast<void*>(stream)),
                     "training_forward_half");
        else
        AT_DISPATCH_FLOATING_TYPES(in.scalar_type(), "boxconv_module_forward", [&] {
            if (clip)
                check_rc(training_forward_fn<scalar_t>()(
                             in.data_ptr<scalar_t>(), x_min.data_ptr<scalar_t>(), x_max.data_ptr<scalar_t>(),
                             y_min.data_ptr<scalar_t>(), y_max.data_ptr<scalar_t>(), real.data_ptr<scalar_t>(),
                             integrated.data_ptr<scalar_t>(), output.data_ptr<scalar_t>(), static_cast<int>(B),
                             static_cast<int>(C), static_cast<int>(F), static_cast<int>(h), static_cast<int>(w),
                             reparam_h, reparam_w, max_h, max_w, normalize ? 1 : 0, exact ? 1 : 0,
                             ptr_or_null(ws), nbytes, reinterpret_cast<void*>(stream)),
                         "training_forward");
            else
                check_rc(inference_forward_fn<scalar_t>()(
                             in.data_ptr<scalar_t>(), x_min.data_ptr<scalar_t>(), x_max.data_ptr<scalar_t>(),
                             y_min.data_ptr<scalar_t>(), y_max.data_ptr<scalar_t>(), real.data_ptr<scalar_t>(),
                             integrated.data_ptr<scalar_t>(), output.data_ptr<scalar_t>(), static_cast<int>(B),
                             static_cast<int>(C), static_cast<int>(F), static_cast<int>(h), static_cast<int>(w),
                             reparam_h, reparam_w, normalize ? 1 : 0, exact ? 1 : 0, ptr_or_null(ws), nbytes,
                             reinterpret_cast<void*>(stream)),
                         "inference_forward");
        });
        // (as the reference: the integral image and the bounds in pixel units; the saved forward
        // output is not needed, the backward kernels rebuild the one sum that would use it)
        ctx->save_for_backward({integrated, real});
        ctx->saved_data["reparam_h"] = reparam_h;
        ctx->saved_data["reparam_w"] = reparam_w;
        ctx->saved_data["normalize"] = normalize;
        ctx->saved_data["exact"] = exact;
        ctx->saved_data["stream"] = stream;
        ctx->saved_data["capturing"] = capturing;
        return output;
    }

    static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx,
                                                   torch::autograd::variable_list grad_outputs) {
        const auto saved = ctx->get_saved_variables();
        const at::Tensor& integrated = saved[0];
        const at::Tensor& real = saved[1];
        const at::Tensor grad_output = grad_outputs[0].contiguous();
        const int64_t B = integrated.size(0), C = integrated.size(1), h = integrated.size(2) - 1,
                      w = integrated.size(3) - 1, F = real.size(2);
        TORCH_CHECK(grad_output.dim() == 4, "grad_output for box_convolution must have 4 dimensions");
        TORCH_CHECK(grad_output.size(0) == B && grad_output.size(1) == C * F && grad_output.size(2) == h &&
                        grad_output.size(3) == w,
                    "box_convolution: sizes of grad_output and input_integrated don't match");
        const bool half = is_half(grad_output.scalar_type());
        TORCH_CHECK(grad_output.device() == integrated.device() &&
                        (grad_output.scalar_type() == integrated.scalar_type() ||
                         (half && integrated.scalar_type() == at::kFloat)),
                    "box_convolution: grad_output and input_integrated differ in device or dtype");
        const bool need_input = ctx->needs_input_grad(0);
        bool need[4];
        bool any_param = false;
        for (int k = 0; k < 4; ++k) { need[k] = ctx->needs_input_grad(1 + k); any_param = any_param || need[k]; }
        const auto opts = integrated.options();
        at::Tensor grad_input;
        const auto io_opts = grad_output.options();         // (the input's own type)
        if (need_input) grad_input = F > 0 ? at::empty({B, C, h, w}, io_opts) : at::zeros({B, C, h, w}, io_opts);
        at::Tensor grad_params;                               // one allocation for the four
        if (any_param) grad_params = at::empty({4, C, F}, opts);
        const bool want_input = need_input && grad_input.numel() > 0 && F > 0;
        const bool want_params = any_param && C * F > 0;
        const int64_t stream = ctx->saved_data["stream"].toInt();
        if (want_input || want_params) {
            const size_t nbytes = g_abi.backward_workspace_bytes(
                static_cast<int>(B), static_cast<int>(C), static_cast<int>(F), static_cast<int>(h),
                static_cast<int>(w), static_cast<int>(integrated.element_size()), want_input ? 1 : 0,
                want_params ? 1 : 0);
            at::Tensor ws = workspace(nbytes, integrated.device(), static_cast<uint64_t>(stream),
                                      ctx->saved_data["capturing"].toBool());
            const float reparam_h = static_cast<float>(ctx->saved_data["reparam_h"].toDouble());
            const float reparam_w = static_cast<float>(ctx->saved_data["reparam_w"].toDouble());
            const int normalize = ctx->saved_data["normalize"].toBool() ? 1 : 0;
            const int exact = ctx->saved_data["exact"].toBool() ? 1 : 0;
            const int64_t n = C * F;
            if (half) {
                const float* r = real.data_ptr<float>();
                float* gp = want_params ? grad_params.data_ptr<float>() : nullptr;
                check_rc(g_abi.backward_half(
                             integrated.data_ptr<float>(), r, r + n, r + 2 * n, r + 3 * n, grad_output.data_ptr(),
                             half_code(grad_output.scalar_type()), reparam_h, reparam_w, normalize, exact,
                             want_input ? grad_input.data_ptr() : nullptr, gp, gp ? gp + n : nullptr,
                             gp ? gp + 2 * n : nullptr, gp ? gp + 3 * n : nullptr, static_cast<int>(B),
                             static_cast<int>(C), static_cast<int>(F), static_cast<int>(h), static_cast<int>(w),
                             ptr_or_null(ws), nbytes, reinterpret_cast<void*>(stream)),
                         "box_convolution_backward_half");
            } else
            AT_DISPATCH_FLOATING_TYPES(integrated.scalar_type(), "boxconv_backward", [&] {
                const scalar_t* r = real.data_ptr<scalar_t>();
                scalar_t* gp = want_params ? grad_params.data_ptr<scalar_t>() : nullptr;
                check_rc(backward_fn<scalar_t>()(
                             integrated.data_ptr<scalar_t>(), r, r + n, r + 2 * n, r + 3 * n,
                             grad_output.data_ptr<scalar_t>(), nullptr, reparam_h, reparam_w, normalize, exact,
                             want_input ? grad_input.data_ptr<scalar_t>() : nullptr, gp, gp ? gp + n : nullptr,
                             gp ? gp + 2 * n : nullptr, gp ? gp + 3 * n : nullptr, static_cast<int>(B),
                             static_cast<int>(C), static_cast<int>(F), static_cast<int>(h), static_cast<int>(w),
                             ptr_or_null(ws), nbytes, reinterpret_cast<void*>(stream)),
                         "box_convolution_backward");
            });
        }
        torch::autograd::variable_list grads(14);             // one per argument of forward
        grads[0] = grad_input;
        if (any_param) {
            const auto parts = grad_params.unbind(0);
            for (int k = 0; k < 4; ++k)
                if (need[k]) grads[1 + k] = parts[k];
        }
        return grads;
    }
};

// The checks of BoxConv2d.forward -> BoxConvolutionFunction.apply -> box_convolution_forward in the
// reference (src/box_convolution_interface.cpp:19-34), same messages.
at::Tensor training_step(const at::Tensor& input, const at::Tensor& x_min, const at::Tensor& x_max,
                         const at::Tensor& y_min, const at::Tensor& y_max, double reparam_h, double reparam_w,
                         double max_h, double max_w, bool normalize, bool exact, bool clip, int64_t stream,
                         bool capturing) {
    TORCH_CHECK(g_abi.last_error != nullptr, "box_convolution: the native glue was not initialised");
    TORCH_CHECK(input.is_cuda(), "box_convolution: input is on '", input.device(),
                "'; this build runs on AMD GPUs only (no CPU path)");
    TORCH_CHECK(input.dim() == 4, "BoxConv2d: input must have 4 dimensions");
    const bool half = is_half(input.scalar_type());
    TORCH_CHECK(input.scalar_type() == at::kFloat || input.scalar_type() == at::kDouble || half,
                "box_convolution: input must be float32, float64, float16 or bfloat16, got ", input.scalar_type());
    const at::ScalarType param_type = half ? at::kFloat : input.scalar_type();
    const at::Tensor* params[4] = {&x_min, &x_max, &y_min, &y_max};
    for (const at::Tensor* p : params) {
        TORCH_CHECK(p->device() == input.device(), "BoxConv2d: input and parameters are on different devices");
        TORCH_CHECK(p->scalar_type() == param_type, "box_convolution: input and parameters have different dtypes (",
                    input.scalar_type(), ", ", p->scalar_type(), ")");
        TORCH_CHECK(!clip || p->is_contiguous(), "box_convolution: parameters must be contiguous to be clipped in place");
        TORCH_CHECK(p->dim() == 2, "BoxConv2d: all parameters must have 2 dimensions");
        TORCH_CHECK(p->size(0) == input.size(1),
                    "BoxConv2d: all parameters must have as many rows as there are input channels");
        TORCH_CHECK(p->size(1) == x_min.size(1), "BoxConv2d: all parameters must have equal number of columns");
    }
    TORCH_CHECK(input.size(2) >= 1 && input.size(3) >= 1, "BoxConv2d: input must be at least 1x1");
    TORCH_CHECK(reparam_h > 0 && reparam_w > 0, "box_convolution: reparametrization factors must be positive");
    if (clip)
        return TrainingStep::apply(input, x_min, x_max, y_min, y_max, reparam_h, reparam_w, max_h, max_w,
                                   normalize, exact, clip, stream, capturing);
    // only read: any layout will do (contiguous() is the tensor itself where it already is)
    return TrainingStep::apply(input, x_min.contiguous(), x_max.contiguous(), y_min.contiguous(),
                               y_max.contiguous(), reparam_h, reparam_w, max_h, max_w, normalize, exact, clip,
                               stream, capturing);
}

void init(uint64_t training_forward_f32, uint64_t training_forward_f64, uint64_t inference_forward_f32,
          uint64_t inference_forward_f64, uint64_t backward_f32, uint64_t backward_f64,
          uint64_t training_forward_half, uint64_t backward_half, uint64_t integral_workspace_bytes,
          uint64_t backward_workspace_bytes, uint64_t last_error) {
    g_abi.training_forward_f32 = reinterpret_cast<void*>(training_forward_f32);
    g_abi.training_forward_f64 = reinterpret_cast<void*>(training_forward_f64);
    g_abi.inference_forward_f32 = reinterpret_cast<void*>(inference_forward_f32);
    g_abi.inference_forward_f64 = reinterpret_cast<void*>(inference_forward_f64);
    g_abi.backward_f32 = reinterpret_cast<void*>(backward_f32);
    g_abi.backward_f64 = reinterpret_cast<void*>(backward_f64);
    g_abi.training_forward_half = reinterpret_cast<TrainingForwardHalfFn>(training_forward_half);
    g_abi.backward_half = reinterpret_cast<BackwardHalfFn>(backward_half);
    g_abi.integral_workspace_bytes = reinterpret_cast<IntegralWorkspaceFn>(integral_workspace_bytes);
    g_abi.backward_workspace_bytes = reinterpret_cast<BackwardWorkspaceFn>(backward_workspace_bytes);
    g_abi.last_error = reinterpret_cast<LastErrorFn>(last_error);
}

void release_workspaces() {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    g_workspaces.clear();
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("init", &init, "hand over the addresses of the C ABI entry points of libboxconv_hip.so");
    m.def("training_step", &training_step,
          "BoxConv2d.forward (training mode: clip = true; eval mode: clip = false) with its backward as a C++ "
          "autograd node");
    m.def("release_workspaces", &release_workspaces);
}
