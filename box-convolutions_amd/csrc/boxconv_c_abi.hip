// extern "C" entry points of libboxconv_hip.so (declared in include/boxconv.h): argument checks on
// the host, workspace carving, kernel launches. No torch types, no allocation, no synchronisation.

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "../../include/boxconv.h"
#include "boxconv_host.hpp"

namespace boxconv {

// ---- per-kernel timing ------------------------------------------------------------------------
namespace {
std::mutex g_prof_mutex;
std::atomic<bool> g_prof_armed{false};                     // read without the lock by every launch
std::string g_prof_name;                                   // empty: disarmed; guarded by the mutex
std::vector<std::pair<hipEvent_t, hipEvent_t>> g_prof_events;
hipEvent_t g_prof_open = nullptr;
int g_prof_every = 1;                                      // bracket one launch in this many
long g_prof_seen = 0;                                      // launches of the armed kernel so far
constexpr size_t kMaxProfiledLaunches = 1 << 16;
}  // namespace

void profile_before(const char* name, hipStream_t stream) {
    if (!g_prof_armed.load(std::memory_order_acquire)) return;   // fast path: not armed
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    if (g_prof_name != name || g_prof_events.size() >= kMaxProfiledLaunches) return;
    if (g_prof_seen++ % g_prof_every != 0) return;
    hipEvent_t start = nullptr;
    if (hipEventCreate(&start) != hipSuccess) return;
    (void)hipEventRecord(start, stream);
    g_prof_open = start;
}

void profile_after(const char* name, hipStream_t stream) {
    if (!g_prof_armed.load(std::memory_order_acquire)) return;
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    if (g_prof_open == nullptr || g_prof_name != name) return;
    hipEvent_t stop = nullptr;
    if (hipEventCreate(&stop) == hipSuccess) {
        (void)hipEventRecord(stop, stream);
        g_prof_events.emplace_back(g_prof_open, stop);
    } else {
        (void)hipEventDestroy(g_prof_open);
    }
    g_prof_open = nullptr;
}

}  // namespace boxconv

namespace {

thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int hip_result(hipError_t e, const char* what) {
    if (e == hipSuccess) return 0;
    return fail(static_cast<int>(e), "%s: %s", what, hipGetErrorString(e));
}

constexpr int64_t kMaxElems = (int64_t(1) << 31) - 1;

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

int check_dims(int batch, int in_planes, int num_filters, int h, int w) {
    if (batch < 0 || in_planes < 0 || num_filters < 0 || h < 1 || w < 1)
        return fail(BOXCONV_E_INVALID_ARGUMENT,
                    "invalid sizes: batch=%d in_planes=%d num_filters=%d h=%d w=%d", batch,
                    in_planes, num_filters, h, w);
    const int64_t big = static_cast<int64_t>(batch) * in_planes * std::max(num_filters, 1) *
                        static_cast<int64_t>(h + 1) * (w + 1);
    if (big > kMaxElems)
        return fail(BOXCONV_E_TOO_LARGE, "tensor of %lld elements exceeds 2^31-1",
                    static_cast<long long>(big));
    return 0;
}

// Walk the planes last to first in the second pass over a tensor (see integral_image_launch).
bool reverse_second_pass() { return boxconv::switches().bwd_reverse; }

// Workspace of the backward pass:
//   [column workspace M of grad_output: planes*F planes of (h+1) rows, or their integral images
//    of (h+1)(w+1) where the streaming pass does not apply]     only if grad_input is wanted
//   [aux doubles: band column sums of that integral image; gather path only]
//   [acc: C*F*5 doubles, times batch*bands when every streaming workgroup has its own slot]
//                                                              only if parameter gradients are wanted
struct BackwardLayout {
    size_t gint_off, aux_off, acc_off, total;
    int acc_slots;        // > 0: per-workgroup accumulation slots per (plane, filter), see grad_output_stream_launch
    bool streaming;       // grad_output_stream_kernel usable for this shape
};

BackwardLayout backward_layout(int batch, int in_planes, int num_filters, int h, int w,
                               int elem_size, bool need_input, bool need_params) {
    BackwardLayout L{};
    const int64_t planes = std::max<int64_t>(static_cast<int64_t>(batch) * in_planes, 1);
    const boxconv::StreamPlan sp = boxconv::plan_grad_output_stream(planes * num_filters, h, w, elem_size);
    L.streaming = sp.usable;
    size_t off = 0;
    L.gint_off = off;
    L.aux_off = off;
    if (need_input) {
        const size_t per_plane = L.streaming
            ? static_cast<size_t>(boxconv::column_workspace_plane(h, w))
            : static_cast<size_t>(h + 1) * (w + 1);
        off += align_up(static_cast<size_t>(planes) * num_filters * per_plane * elem_size, 256);
        L.aux_off = off;
        const int64_t aux = L.streaming ? int64_t(0)
                                        : boxconv::plan_integral(planes * num_filters, h, w).aux_doubles;
        off += align_up(static_cast<size_t>(aux) * 8, 256);
    }
    L.acc_off = off;
    L.acc_slots = (need_params && L.streaming) ? sp.nb * sp.parts : 0;
    if (need_params)
        off += align_up(static_cast<size_t>(in_planes) * num_filters * 5 * 8 *
                        (L.acc_slots > 0 ? static_cast<size_t>(batch) * L.acc_slots : 1), 256);
    L.total = off;
    return L;
}

template <class T>
int integral_image_impl(const T* in, T* out, int64_t planes, int h, int w, void* workspace,
                        size_t workspace_bytes, void* stream) {
    if (planes < 0 || h < 1 || w < 1)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "integral image: invalid sizes planes=%lld h=%d w=%d",
                    static_cast<long long>(planes), h, w);
    if (planes == 0) return 0;
    if (in == nullptr || out == nullptr)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "integral image: null tensor pointer");
    if (planes * static_cast<int64_t>(h + 1) * (w + 1) > kMaxElems)
        return fail(BOXCONV_E_TOO_LARGE, "integral image: output exceeds 2^31-1 elements");
    const size_t need = boxconv_integral_image_workspace_bytes(planes, h, w);
    if (need > 0 && (workspace == nullptr || workspace_bytes < need ||
                     reinterpret_cast<uintptr_t>(workspace) % 8 != 0))
        return fail(BOXCONV_E_WORKSPACE, "integral image: workspace of %zu bytes (8-byte aligned) required, got %zu",
                    need, workspace_bytes);
    return hip_result(boxconv::integral_image_launch<T>(in, out, planes, h, w,
                                                        static_cast<double*>(workspace),
                                                        boxconv::plan_integral(planes, h, w), false, false,
                                                        static_cast<hipStream_t>(stream)),
                      "integral image launch");
}

// ---- integral image without a caller-provided workspace ----------------------------------------
// The band column sums (and the hand-over words of the single-pass kernel) live in a fixed array
// in device memory instead of a workspace argument, for callers that cannot allocate one. Every
// GPU holds its own copy of the array at its own address; `scratch` itself is only the host-side
// name of the symbol, so the address is looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[BOXCONV_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Address of `scratch` on the current device (null + error message on failure).
void* static_scratch(int* rc) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { *rc = hip_result(e, "hipGetDevice"); return nullptr; }
    if (dev < 0 || dev >= kMaxDevices) {
        *rc = fail(BOXCONV_E_INVALID_ARGUMENT, "device index %d outside 0..%d", dev, kMaxDevices - 1);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            *rc = e != hipSuccess ? hip_result(e, "hipGetSymbolAddress(scratch)")
                                  : fail(BOXCONV_E_WORKSPACE, "hipGetSymbolAddress(scratch) returned null");
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    *rc = 0;
    return g_scratch_ptr[dev];
}

int integral_image_static_impl(const float* in, float* out, int64_t planes, int h, int w, void* stream) {
    if (planes < 0 || h < 1 || w < 1)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "integral image: invalid sizes planes=%lld h=%d w=%d",
                    static_cast<long long>(planes), h, w);
    if (planes == 0) return 0;
    const size_t need = boxconv_integral_image_workspace_bytes(planes, h, w);
    if (need > BOXCONV_STATIC_SCRATCH_BYTES)
        return fail(BOXCONV_E_TOO_LARGE,
                    "integral image without workspace: planes=%lld h=%d w=%d needs %zu bytes of scratch, "
                    "the built-in array holds %zu; use boxconv_integral_image_f32 with a workspace",
                    static_cast<long long>(planes), h, w, need,
                    static_cast<size_t>(BOXCONV_STATIC_SCRATCH_BYTES));
    int rc = 0;
    void* ws = need > 0 ? static_scratch(&rc) : nullptr;
    if (rc != 0) return rc;
    // Same checks and launches as the entry point with a workspace argument; the kernels rewrite
    // every scratch word they later read (column sums, or the hand-over markers, which a fill
    // kernel resets at every call), so nothing of the previous call is ever seen.
    return integral_image_impl<float>(in, out, planes, h, w, ws, need, stream);
}

// BoxConv2d.forward in training mode, natively: clip (+ stored -> real units), integral image,
// forward sampling; the clip rides on the launch that prepares the integral image's workspace.
template <class T>
int training_forward_impl(const T* input, T* x_min, T* x_max, T* y_min, T* y_max, T* real,
                          T* integ, T* output, int batch, int in_planes, int num_filters, int h,
                          int w, double reparam_h, double reparam_w, double max_h, double max_w,
                          int normalize, int exact, void* workspace, size_t workspace_bytes,
                          void* stream, bool project = true) {
    if (int rc = check_dims(batch, in_planes, num_filters, h, w)) return rc;
    const int n = in_planes * num_filters;
    if (n > 0 && (!x_min || !x_max || !y_min || !y_max || !real))
        return fail(BOXCONV_E_INVALID_ARGUMENT, "training forward: null parameter pointer");
    if (!(reparam_h > 0) || !(reparam_w > 0))
        return fail(BOXCONV_E_INVALID_ARGUMENT, "training forward: reparametrization factors must be positive");
    const int64_t planes = static_cast<int64_t>(batch) * in_planes;
    if (planes > 0 && (!input || !integ || (n > 0 && !output)))
        return fail(BOXCONV_E_INVALID_ARGUMENT, "training forward: null tensor pointer");
    const size_t need = boxconv_integral_image_workspace_bytes(planes, h, w);
    if (need > 0 && (workspace == nullptr || workspace_bytes < need ||
                     reinterpret_cast<uintptr_t>(workspace) % 8 != 0))
        return fail(BOXCONV_E_WORKSPACE, "training forward: workspace of %zu bytes (8-byte aligned) required, got %zu",
                    need, workspace_bytes);
    hipStream_t s = static_cast<hipStream_t>(stream);
    double* aux = static_cast<double*>(workspace);
    const boxconv::IntegralPlan plan = boxconv::plan_integral(planes, h, w);
    bool fused = false;
    if constexpr (std::is_same<T, float>::value) {
        // small planes: the clip job rides on the integral image's own launch
        if (boxconv::clip_rides_on_integral(plan, planes)) {
            fused = true;
            if (int rc = hip_result(boxconv::clip_and_plane_integral_launch<float>(
                    boxconv::clip_args<float>(x_min, x_max, y_min, y_max, real, n, reparam_h, reparam_w,
                                              max_h, max_w, exact != 0, project),
                    input, integ, planes, h, w, plan, s), "clip and integral image launch"))
                return rc;
        }
    }
    if (!fused) {
        bool prepared = false;
        if (int rc = hip_result(boxconv::clip_and_prepare_integral_launch<T>(
                boxconv::clip_args<T>(x_min, x_max, y_min, y_max, real, n, reparam_h, reparam_w, max_h,
                                      max_w, exact != 0, project),
                planes, w, aux, plan, &prepared, s), "clip launch"))
            return rc;
        if (planes == 0) return 0;
        if (int rc = hip_result(boxconv::integral_image_launch<T>(input, integ, planes, h, w, aux, plan,
                                                                  prepared, false, s),
                                "integral image launch"))
            return rc;
    }
    if (n == 0) return 0;
    const boxconv::Dims d{in_planes, num_filters, h, w, planes, 0};
    const boxconv::BoxParams<T> prm{real, real + n, real + 2 * n, real + 3 * n};
    return hip_result(boxconv::forward_launch<T>(integ, prm, output, d, normalize != 0, exact != 0, s),
                      "forward launch");
}

// The same for a float16 / bfloat16 input and output (TH): float32 bounds, float32 integral image.
template <class TH>
int training_forward_half_impl(const TH* input, float* x_min, float* x_max, float* y_min, float* y_max,
                               float* real, float* integ, TH* output, int batch, int in_planes,
                               int num_filters, int h, int w, double reparam_h, double reparam_w,
                               double max_h, double max_w, bool project, int normalize, int exact,
                               void* workspace, size_t workspace_bytes, void* stream) {
    const int n = in_planes * num_filters;
    const int64_t planes = static_cast<int64_t>(batch) * in_planes;
    hipStream_t s = static_cast<hipStream_t>(stream);
    double* aux = static_cast<double*>(workspace);
    const boxconv::IntegralPlan plan = boxconv::plan_integral(planes, h, w);
    const boxconv::ClipArgs<float> clip = boxconv::clip_args<float>(
        x_min, x_max, y_min, y_max, real, n, reparam_h, reparam_w, max_h, max_w, exact != 0, project);
    if (boxconv::clip_rides_on_integral(plan, planes)) {
        if (int rc = hip_result(boxconv::clip_and_plane_integral_launch<TH>(clip, input, integ, planes, h, w,
                                                                            plan, s),
                                "clip and integral image launch"))
            return rc;
    } else {
        bool prepared = false;
        if (int rc = hip_result(boxconv::clip_and_prepare_integral_launch<float>(clip, planes, w, aux, plan,
                                                                                &prepared, s), "clip launch"))
            return rc;
        if (planes == 0) return 0;
        if (int rc = hip_result(boxconv::integral_image_widening_launch<TH>(input, integ, planes, h, w, aux,
                                                                            plan, s, prepared),
                                "integral image launch"))
            return rc;
    }
    if (n == 0) return 0;
    const boxconv::Dims d{in_planes, num_filters, h, w, planes, 0};
    const boxconv::BoxParams<float> prm{real, real + n, real + 2 * n, real + 3 * n};
    return hip_result(boxconv::forward_fused_launch<TH>(integ, prm, output, static_cast<const TH*>(nullptr),
                                                        nullptr, nullptr, false, d, normalize != 0,
                                                        exact != 0, s),
                      "forward launch");
}

template <class TI>
int integral_image_widening_impl(const TI* in, float* out, int64_t planes, int h, int w,
                                 void* workspace, size_t workspace_bytes, void* stream) {
    const size_t need = boxconv_integral_image_workspace_bytes(planes, h, w);
    if (need > 0 && (workspace == nullptr || workspace_bytes < need ||
                     reinterpret_cast<uintptr_t>(workspace) % 8 != 0))
        return fail(BOXCONV_E_WORKSPACE, "integral image: workspace of %zu bytes (8-byte aligned) required, got %zu",
                    need, workspace_bytes);
    return hip_result(boxconv::integral_image_widening_launch<TI>(
                          in, out, planes, h, w, static_cast<double*>(workspace),
                          boxconv::plan_integral(planes, h, w), static_cast<hipStream_t>(stream)),
                      "integral image launch");
}

template <class T>
int forward_impl(const T* integ, const T* x_min, const T* x_max, const T* y_min, const T* y_max,
                 T* output, int batch, int in_planes, int num_filters, int h, int w,
                 int normalize, int exact, void* stream) {
    if (int rc = check_dims(batch, in_planes, num_filters, h, w)) return rc;
    if (static_cast<int64_t>(batch) * in_planes * num_filters == 0) return 0;
    if (!integ || !x_min || !x_max || !y_min || !y_max || !output)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "forward: null tensor pointer");
    boxconv::Dims d{in_planes, num_filters, h, w, static_cast<int64_t>(batch) * in_planes, 0};
    boxconv::BoxParams<T> prm{x_min, x_max, y_min, y_max};
    return hip_result(boxconv::forward_launch<T>(integ, prm, output, d, normalize != 0, exact != 0,
                                                 static_cast<hipStream_t>(stream)),
                      "forward launch");
}

// TG: element type of grad_output and grad_input (T, or f16_t / bf16_t with T = float).
template <class T, class TG>
int backward_impl(const T* integ, const T* x_min, const T* x_max, const T* y_min, const T* y_max,
                  const TG* grad_output, const T* /*output*/, float reparam_h, float reparam_w,
                  int normalize, int exact, TG* grad_input, T* gx_min, T* gx_max, T* gy_min,
                  T* gy_max, int batch, int in_planes, int num_filters, int h, int w,
                  void* workspace, size_t workspace_bytes, void* stream) {
    if (int rc = check_dims(batch, in_planes, num_filters, h, w)) return rc;
    const bool need_input = grad_input != nullptr;
    const bool need_params = gx_min || gx_max || gy_min || gy_max;
    if (!need_input && !need_params) return 0;
    if (!x_min || !x_max || !y_min || !y_max)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "backward: null parameter pointer");
    const int64_t nout = static_cast<int64_t>(batch) * in_planes * num_filters;
    if (nout > 0 && (!grad_output || (need_params && !integ)))
        return fail(BOXCONV_E_INVALID_ARGUMENT, "backward: null tensor pointer");
    const BackwardLayout L = backward_layout(batch, in_planes, num_filters, h, w, sizeof(T),
                                             need_input, need_params);
    if (L.total > 0 && (workspace == nullptr || workspace_bytes < L.total ||
                        reinterpret_cast<uintptr_t>(workspace) % 256 != 0))
        return fail(BOXCONV_E_WORKSPACE, "backward: workspace of %zu bytes (256-byte aligned) required, got %zu",
                    L.total, workspace_bytes);
    constexpr bool kSameType = std::is_same<T, TG>::value;
    if (!kSameType && !L.streaming)
        return fail(BOXCONV_E_TOO_LARGE, "backward: half-precision grad_output is read directly for rows of at "
                    "most %d columns; convert wider ones to float first", boxconv::kMaxRowStreamWidth);

    hipStream_t s = static_cast<hipStream_t>(stream);
    unsigned char* ws = static_cast<unsigned char*>(workspace);
    boxconv::BoxParams<T> prm{x_min, x_max, y_min, y_max};
    const int n_boxes = in_planes * num_filters;
    double* acc = need_params ? reinterpret_cast<double*>(ws + L.acc_off) : nullptr;
    double* aux = reinterpret_cast<double*>(ws + L.aux_off);
    T* gint = need_input ? reinterpret_cast<T*>(ws + L.gint_off) : nullptr;

    if (need_input && nout == 0)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "backward: grad_input requested with zero filters");
    if (need_params && L.acc_slots == 0)
        if (int rc = hip_result(boxconv::grad_params_begin(acc, n_boxes, s), "accumulator clear"))
            return rc;

    const int grad_dtype = std::is_same<TG, T>::value ? 0 : std::is_same<TG, boxconv::f16_t>::value ? 1 : 2;
    const boxconv::ParamFinish<T> finish{acc, batch, L.acc_slots, {gx_min, gx_max, gy_min, gy_max},
                                         n_boxes, reparam_h, reparam_w, normalize != 0, exact != 0,
                                         integ, grad_output, grad_dtype, h, w, num_filters};
    bool finished = false;
    const int64_t planes = static_cast<int64_t>(batch) * in_planes;
    const boxconv::Dims d{in_planes, num_filters, h, w, planes, 0};
    if (L.streaming) {
        // one pass over grad_output: parameter sums + column workspace, then grad_input, whose
        // launch finishes the parameter gradients on the side
        const boxconv::StreamPlan sp = boxconv::plan_grad_output_stream(planes * num_filters, h, w, sizeof(T));
        if (int rc = hip_result(boxconv::grad_output_stream_launch<T, TG>(
                integ, grad_output, prm, acc, L.acc_slots, gint, sp, d, exact != 0, s),
                "grad_output streaming launch"))
            return rc;
        if (need_input)
            if (int rc = hip_result(boxconv::grad_input_launch<T, TG>(
                    gint, sp.R, prm, grad_input, d, normalize != 0, exact != 0, s,
                    need_params ? &finish : nullptr, &finished),
                    "input-gradient launch"))
                return rc;
    } else if constexpr (kSameType) {
        // any width: gather kernels on true integral images
        if (need_params)
            if (int rc = hip_result(boxconv::grad_params_gather_launch<T>(
                    integ, grad_output, prm, acc, d, exact != 0, s),
                    "parameter-gradient launch"))
                return rc;
        if (need_input) {
            const boxconv::IntegralPlan plan = boxconv::plan_integral(planes * num_filters, h, w);
            if (int rc = hip_result(boxconv::integral_image_launch<T>(
                    grad_output, gint, planes * num_filters, h, w, aux, plan, false,
                    need_params && reverse_second_pass(), s),
                    "grad_output integral image launch"))
                return rc;
            if (int rc = hip_result(boxconv::grad_input_launch<T, T>(
                    gint, 0, prm, grad_input, d, normalize != 0, exact != 0, s),
                    "input-gradient launch"))
                return rc;
        }
    }
    if (need_params && !finished)
        if (int rc = hip_result(boxconv::grad_params_finish<T>(finish, prm, s),
                                "parameter-gradient finish"))
            return rc;
    return 0;
}

template <class T>
int clip_impl(T* x_min, T* x_max, T* y_min, T* y_max, T* real, int n, double reparam_h, double reparam_w,
              double max_h, double max_w, int exact, void* stream) {
    if (n < 0) return fail(BOXCONV_E_INVALID_ARGUMENT, "clip: negative element count");
    if (n == 0) return 0;
    if (!x_min || !x_max || !y_min || !y_max)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "clip: null parameter pointer");
    if (!(reparam_h != 0.0) || !(reparam_w != 0.0))
        return fail(BOXCONV_E_INVALID_ARGUMENT, "clip: reparametrization factor is zero");
    return hip_result(boxconv::clip_launch<T>(x_min, x_max, y_min, y_max, real, n, reparam_h, reparam_w,
                                              max_h, max_w, exact != 0,
                                              static_cast<hipStream_t>(stream)),
                      "clip launch");
}

}  // namespace

extern "C" {

int boxconv_abi_version(void) { return BOXCONV_ABI_VERSION; }

int boxconv_profile_arm(const char* kernel_name) { return boxconv_profile_arm_every(kernel_name, 1); }

int boxconv_profile_arm_every(const char* kernel_name, int every) {
    if (every < 1) return fail(BOXCONV_E_INVALID_ARGUMENT, "profile_arm_every: every must be >= 1");
    std::lock_guard<std::mutex> lock(boxconv::g_prof_mutex);
    boxconv::g_prof_every = every;
    boxconv::g_prof_seen = 0;
    for (auto& ev : boxconv::g_prof_events) {
        (void)hipEventDestroy(ev.first);
        (void)hipEventDestroy(ev.second);
    }
    boxconv::g_prof_events.clear();
    boxconv::g_prof_name = kernel_name ? kernel_name : "";
    boxconv::g_prof_armed.store(!boxconv::g_prof_name.empty(), std::memory_order_release);
    return 0;
}

int boxconv_profile_collect(double* total_ms, int* launches) {
    std::lock_guard<std::mutex> lock(boxconv::g_prof_mutex);
    double sum = 0.0;
    int n = 0;
    int rc = 0;
    for (auto& ev : boxconv::g_prof_events) {
        float ms = 0.0f;
        hipError_t e = hipEventSynchronize(ev.second);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, ev.first, ev.second);
        if (e == hipSuccess) { sum += ms; ++n; }
        else rc = hip_result(e, "profile collect");
        (void)hipEventDestroy(ev.first);
        (void)hipEventDestroy(ev.second);
    }
    boxconv::g_prof_events.clear();
    boxconv::g_prof_name.clear();
    boxconv::g_prof_armed.store(false, std::memory_order_release);
    if (total_ms) *total_ms = sum;
    if (launches) *launches = n;
    return rc;
}

const char* boxconv_last_error(void) { return g_error; }

void boxconv_reload_env(void) { boxconv::reload_switches(); }

size_t boxconv_integral_image_workspace_bytes(int64_t planes, int h, int w) {
    if (planes <= 0 || h < 1 || w < 1) return 0;
    return static_cast<size_t>(boxconv::plan_integral(planes, h, w).aux_doubles) * 8;
}

int boxconv_integral_image_f32(const float* in, float* out, int64_t planes, int h, int w,
                               void* workspace, size_t workspace_bytes, void* stream) {
    return integral_image_impl<float>(in, out, planes, h, w, workspace, workspace_bytes, stream);
}
int boxconv_integral_image_f64(const double* in, double* out, int64_t planes, int h, int w,
                               void* workspace, size_t workspace_bytes, void* stream) {
    return integral_image_impl<double>(in, out, planes, h, w, workspace, workspace_bytes, stream);
}

int boxconv_integral_image_int(const void* in, void* out, int dtype, int64_t planes, int h, int w,
                               void* stream) {
    if (planes < 0 || h < 1 || w < 1)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "integral image: invalid sizes planes=%lld h=%d w=%d",
                    static_cast<long long>(planes), h, w);
    if (dtype < BOXCONV_U8 || dtype > BOXCONV_I64)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "integral image: dtype %d is not one of BOXCONV_U8 .. BOXCONV_I64",
                    dtype);
    if (planes == 0) return 0;
    if (in == nullptr || out == nullptr)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "integral image: null tensor pointer");
    if (planes * static_cast<int64_t>(h + 1) * (w + 1) > kMaxElems || planes * static_cast<int64_t>(h) > kMaxElems)
        return fail(BOXCONV_E_TOO_LARGE, "integral image: output exceeds 2^31-1 elements");
    return hip_result(boxconv::integral_image_int_launch(in, out, dtype, planes, h, w,
                                                         static_cast<hipStream_t>(stream)),
                      "integer integral image launch");
}

int boxconv_probe_copy_bands(const float* src, float* dst, int64_t planes, int h, int w,
                             int rows_per_group, int rows_in_flight, void* stream) {
    if (planes < 1 || h < 1 || w < 256 || w > 4096 || w % 256 != 0 || rows_per_group < 1 ||
        h % rows_per_group != 0 || (rows_in_flight != 2 && rows_in_flight != 4 && rows_in_flight != 8) ||
        rows_per_group % rows_in_flight != 0)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "copy probe: invalid sizes planes=%lld h=%d w=%d rows=%d in flight=%d",
                    static_cast<long long>(planes), h, w, rows_per_group, rows_in_flight);
    if (src == nullptr || dst == nullptr)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "copy probe: null tensor pointer");
    if (planes * static_cast<int64_t>(h + 1) * w > kMaxElems)
        return fail(BOXCONV_E_TOO_LARGE, "copy probe: destination exceeds 2^31-1 elements");
    return hip_result(boxconv::probe_copy_bands_launch(src, dst, planes, h, w, rows_per_group, rows_in_flight,
                                                       static_cast<hipStream_t>(stream)),
                      "copy probe launch");
}

int boxconv_probe_grad_input_pattern(const float* column_workspace, float* out, const int* x_lo,
                                     const int* x_hi, int64_t planes, int in_planes, int num_filters, int h,
                                     int mode, void* stream) {
    if (planes < 1 || in_planes < 1 || num_filters < 1 || h < 8 || h % 8 != 0 || mode < 0 || mode > 2)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "grad-input pattern probe: invalid sizes planes=%lld in_planes=%d "
                    "num_filters=%d h=%d mode=%d", static_cast<long long>(planes), in_planes, num_filters, h, mode);
    if (mode == 2 && (h < 97 || planes < 8))
        return fail(BOXCONV_E_INVALID_ARGUMENT, "grad-input pattern probe: mode 2 needs h >= 97 and 8 planes");
    if (!column_workspace || !out || !x_lo || !x_hi)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "grad-input pattern probe: null pointer");
    if (planes * num_filters * static_cast<int64_t>(h + 1) * 1024 > kMaxElems)
        return fail(BOXCONV_E_TOO_LARGE, "grad-input pattern probe: workspace exceeds 2^31-1 elements");
    return hip_result(boxconv::probe_grad_input_pattern_launch(column_workspace, out, x_lo, x_hi, planes, in_planes,
                                                               num_filters, h, mode, static_cast<hipStream_t>(stream)),
                      "grad-input pattern probe launch");
}

int boxconv_integral_image_static_f32(const float* in, float* out, int64_t planes, int h, int w,
                                      void* stream) {
    return integral_image_static_impl(in, out, planes, h, w, stream);
}

int boxconv_forward_f32(const float* input_integrated, const float* x_min, const float* x_max,
                        const float* y_min, const float* y_max, float* output, int batch,
                        int in_planes, int num_filters, int h, int w, int normalize, int exact,
                        void* stream) {
    return forward_impl<float>(input_integrated, x_min, x_max, y_min, y_max, output, batch,
                               in_planes, num_filters, h, w, normalize, exact, stream);
}
int boxconv_forward_f64(const double* input_integrated, const double* x_min, const double* x_max,
                        const double* y_min, const double* y_max, double* output, int batch,
                        int in_planes, int num_filters, int h, int w, int normalize, int exact,
                        void* stream) {
    return forward_impl<double>(input_integrated, x_min, x_max, y_min, y_max, output, batch,
                                in_planes, num_filters, h, w, normalize, exact, stream);
}

int boxconv_integral_image_half_f32(const void* in, int input_dtype, float* out, int64_t planes,
                                    int h, int w, void* workspace, size_t workspace_bytes,
                                    void* stream) {
    if (planes < 0 || h < 1 || w < 1)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "integral image: invalid sizes planes=%lld h=%d w=%d",
                    static_cast<long long>(planes), h, w);
    if (input_dtype != BOXCONV_F16 && input_dtype != BOXCONV_BF16)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "integral image: input_dtype %d is neither BOXCONV_F16 nor BOXCONV_BF16",
                    input_dtype);
    if (planes == 0) return 0;
    if (in == nullptr || out == nullptr)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "integral image: null tensor pointer");
    if (planes * static_cast<int64_t>(h + 1) * (w + 1) > kMaxElems)
        return fail(BOXCONV_E_TOO_LARGE, "integral image: output exceeds 2^31-1 elements");
    if (!boxconv::integral_image_widening_applies(h, w))
        return fail(BOXCONV_E_TOO_LARGE, "integral image: half-precision input is read directly for rows "
                    "of at most %d columns and planes below 2 GiB; convert wider inputs to float first",
                    boxconv::kMaxWideningWidth);
    if (input_dtype == BOXCONV_F16)
        return integral_image_widening_impl(static_cast<const boxconv::f16_t*>(in), out, planes, h, w,
                                            workspace, workspace_bytes, stream);
    return integral_image_widening_impl(static_cast<const boxconv::bf16_t*>(in), out, planes, h, w,
                                        workspace, workspace_bytes, stream);
}

int boxconv_training_forward_f32(const float* input, float* x_min, float* x_max, float* y_min,
                                 float* y_max, float* real_parameters, float* input_integrated,
                                 float* output, int batch, int in_planes, int num_filters, int h,
                                 int w, double reparametrization_h, double reparametrization_w,
                                 double max_input_h, double max_input_w, int normalize, int exact,
                                 void* workspace, size_t workspace_bytes, void* stream) {
    return training_forward_impl<float>(input, x_min, x_max, y_min, y_max, real_parameters,
                                        input_integrated, output, batch, in_planes, num_filters, h, w,
                                        reparametrization_h, reparametrization_w, max_input_h,
                                        max_input_w, normalize, exact, workspace, workspace_bytes,
                                        stream);
}
int boxconv_training_forward_f64(const double* input, double* x_min, double* x_max, double* y_min,
                                 double* y_max, double* real_parameters, double* input_integrated,
                                 double* output, int batch, int in_planes, int num_filters, int h,
                                 int w, double reparametrization_h, double reparametrization_w,
                                 double max_input_h, double max_input_w, int normalize, int exact,
                                 void* workspace, size_t workspace_bytes, void* stream) {
    return training_forward_impl<double>(input, x_min, x_max, y_min, y_max, real_parameters,
                                         input_integrated, output, batch, in_planes, num_filters, h,
                                         w, reparametrization_h, reparametrization_w, max_input_h,
                                         max_input_w, normalize, exact, workspace, workspace_bytes,
                                         stream);
}

int boxconv_training_forward_half_f32(const void* input, int io_dtype, float* x_min, float* x_max,
                                      float* y_min, float* y_max, float* real_parameters,
                                      float* input_integrated, void* output, int batch, int in_planes,
                                      int num_filters, int h, int w, double reparametrization_h,
                                      double reparametrization_w, double max_input_h, double max_input_w,
                                      int clip, int normalize, int exact, void* workspace,
                                      size_t workspace_bytes, void* stream) {
    if (int rc = check_dims(batch, in_planes, num_filters, h, w)) return rc;
    if (io_dtype != BOXCONV_F16 && io_dtype != BOXCONV_BF16)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "half training forward: io_dtype %d is neither BOXCONV_F16 nor BOXCONV_BF16",
                    io_dtype);
    const int n = in_planes * num_filters;
    if (n > 0 && (!x_min || !x_max || !y_min || !y_max || !real_parameters))
        return fail(BOXCONV_E_INVALID_ARGUMENT, "half training forward: null parameter pointer");
    if (!(reparametrization_h > 0) || !(reparametrization_w > 0))
        return fail(BOXCONV_E_INVALID_ARGUMENT, "half training forward: reparametrization factors must be positive");
    const int64_t planes = static_cast<int64_t>(batch) * in_planes;
    if (planes > 0 && (!input || !input_integrated || (n > 0 && !output)))
        return fail(BOXCONV_E_INVALID_ARGUMENT, "half training forward: null tensor pointer");
    if (!boxconv::integral_image_widening_applies(h, w))
        return fail(BOXCONV_E_TOO_LARGE, "half training forward: half-precision input is read directly for rows "
                    "of at most %d columns and planes below 2 GiB; convert wider inputs to float first",
                    boxconv::kMaxWideningWidth);
    const size_t need = boxconv_integral_image_workspace_bytes(planes, h, w);
    if (need > 0 && (workspace == nullptr || workspace_bytes < need ||
                     reinterpret_cast<uintptr_t>(workspace) % 8 != 0))
        return fail(BOXCONV_E_WORKSPACE, "half training forward: workspace of %zu bytes (8-byte aligned) required, got %zu",
                    need, workspace_bytes);
    if (io_dtype == BOXCONV_F16)
        return training_forward_half_impl(static_cast<const boxconv::f16_t*>(input), x_min, x_max, y_min, y_max,
                                          real_parameters, input_integrated, static_cast<boxconv::f16_t*>(output),
                                          batch, in_planes, num_filters, h, w, reparametrization_h,
                                          reparametrization_w, max_input_h, max_input_w, clip != 0, normalize,
                                          exact, workspace, workspace_bytes, stream);
    return training_forward_half_impl(static_cast<const boxconv::bf16_t*>(input), x_min, x_max, y_min, y_max,
                                      real_parameters, input_integrated, static_cast<boxconv::bf16_t*>(output),
                                      batch, in_planes, num_filters, h, w, reparametrization_h,
                                      reparametrization_w, max_input_h, max_input_w, clip != 0, normalize,
                                      exact, workspace, workspace_bytes, stream);
}

int boxconv_inference_forward_f32(const float* input, const float* x_min, const float* x_max,
                                  const float* y_min, const float* y_max, float* real_parameters,
                                  float* input_integrated, float* output, int batch, int in_planes,
                                  int num_filters, int h, int w, double reparametrization_h,
                                  double reparametrization_w, int normalize, int exact, void* workspace,
                                  size_t workspace_bytes, void* stream) {
    // (the stored bounds are only read: the job does not project)
    return training_forward_impl<float>(input, const_cast<float*>(x_min), const_cast<float*>(x_max),
                                        const_cast<float*>(y_min), const_cast<float*>(y_max), real_parameters,
                                        input_integrated, output, batch, in_planes, num_filters, h, w,
                                        reparametrization_h, reparametrization_w, 0.0, 0.0, normalize, exact,
                                        workspace, workspace_bytes, stream, false);
}
int boxconv_inference_forward_f64(const double* input, const double* x_min, const double* x_max,
                                  const double* y_min, const double* y_max, double* real_parameters,
                                  double* input_integrated, double* output, int batch, int in_planes,
                                  int num_filters, int h, int w, double reparametrization_h,
                                  double reparametrization_w, int normalize, int exact, void* workspace,
                                  size_t workspace_bytes, void* stream) {
    return training_forward_impl<double>(input, const_cast<double*>(x_min), const_cast<double*>(x_max),
                                         const_cast<double*>(y_min), const_cast<double*>(y_max), real_parameters,
                                         input_integrated, output, batch, in_planes, num_filters, h, w,
                                         reparametrization_h, reparametrization_w, 0.0, 0.0, normalize, exact,
                                         workspace, workspace_bytes, stream, false);
}

int boxconv_forward_fused_f32(const float* input_integrated, const float* x_min,
                              const float* x_max, const float* y_min, const float* y_max,
                              void* output, int output_dtype, const void* residual,
                              const float* channel_scale, const float* channel_shift, int relu,
                              int batch, int in_planes, int num_filters, int h, int w,
                              int normalize, int exact, void* stream) {
    if (int rc = check_dims(batch, in_planes, num_filters, h, w)) return rc;
    if (output_dtype != BOXCONV_F32 && output_dtype != BOXCONV_F16 && output_dtype != BOXCONV_BF16)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "fused forward: unknown output_dtype %d", output_dtype);
    if (static_cast<int64_t>(batch) * in_planes * num_filters == 0) return 0;
    if (!input_integrated || !x_min || !x_max || !y_min || !y_max || !output)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "fused forward: null tensor pointer");
    const boxconv::Dims d{in_planes, num_filters, h, w, static_cast<int64_t>(batch) * in_planes, 0};
    const boxconv::BoxParams<float> prm{x_min, x_max, y_min, y_max};
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (output_dtype == BOXCONV_F32)
        e = boxconv::forward_fused_launch<float>(
            input_integrated, prm, static_cast<float*>(output), static_cast<const float*>(residual),
            channel_scale, channel_shift, relu != 0, d, normalize != 0, exact != 0, s);
    else if (output_dtype == BOXCONV_F16)
        e = boxconv::forward_fused_launch<boxconv::f16_t>(
            input_integrated, prm, static_cast<boxconv::f16_t*>(output),
            static_cast<const boxconv::f16_t*>(residual), channel_scale, channel_shift, relu != 0, d,
            normalize != 0, exact != 0, s);
    else
        e = boxconv::forward_fused_launch<boxconv::bf16_t>(
            input_integrated, prm, static_cast<boxconv::bf16_t*>(output),
            static_cast<const boxconv::bf16_t*>(residual), channel_scale, channel_shift, relu != 0, d,
            normalize != 0, exact != 0, s);
    return hip_result(e, "fused forward launch");
}

size_t boxconv_backward_workspace_bytes(int batch, int in_planes, int num_filters, int h, int w,
                                        int elem_size, int input_needs_grad,
                                        int params_need_grad) {
    if (batch < 0 || in_planes < 0 || num_filters < 0 || h < 1 || w < 1) return 0;
    if (elem_size != 4 && elem_size != 8) return 0;
    return backward_layout(batch, in_planes, num_filters, h, w, elem_size, input_needs_grad != 0,
                           params_need_grad != 0).total;
}

int boxconv_backward_f32(const float* input_integrated, const float* x_min, const float* x_max,
                         const float* y_min, const float* y_max, const float* grad_output,
                         const float* output, float reparametrization_h,
                         float reparametrization_w, int normalize, int exact, float* grad_input,
                         float* grad_x_min, float* grad_x_max, float* grad_y_min,
                         float* grad_y_max, int batch, int in_planes, int num_filters, int h,
                         int w, void* workspace, size_t workspace_bytes, void* stream) {
    return backward_impl<float, float>(input_integrated, x_min, x_max, y_min, y_max, grad_output, output,
                                reparametrization_h, reparametrization_w, normalize, exact,
                                grad_input, grad_x_min, grad_x_max, grad_y_min, grad_y_max, batch,
                                in_planes, num_filters, h, w, workspace, workspace_bytes, stream);
}
int boxconv_backward_f64(const double* input_integrated, const double* x_min, const double* x_max,
                         const double* y_min, const double* y_max, const double* grad_output,
                         const double* output, float reparametrization_h,
                         float reparametrization_w, int normalize, int exact, double* grad_input,
                         double* grad_x_min, double* grad_x_max, double* grad_y_min,
                         double* grad_y_max, int batch, int in_planes, int num_filters, int h,
                         int w, void* workspace, size_t workspace_bytes, void* stream) {
    return backward_impl<double, double>(input_integrated, x_min, x_max, y_min, y_max, grad_output, output,
                                 reparametrization_h, reparametrization_w, normalize, exact,
                                 grad_input, grad_x_min, grad_x_max, grad_y_min, grad_y_max, batch,
                                 in_planes, num_filters, h, w, workspace, workspace_bytes, stream);
}

int boxconv_backward_half_f32(const float* input_integrated, const float* x_min, const float* x_max,
                              const float* y_min, const float* y_max, const void* grad_output,
                              int io_dtype, float reparametrization_h, float reparametrization_w,
                              int normalize, int exact, void* grad_input, float* grad_x_min,
                              float* grad_x_max, float* grad_y_min, float* grad_y_max, int batch,
                              int in_planes, int num_filters, int h, int w, void* workspace,
                              size_t workspace_bytes, void* stream) {
    if (io_dtype == BOXCONV_F16)
        return backward_impl<float, boxconv::f16_t>(
            input_integrated, x_min, x_max, y_min, y_max, static_cast<const boxconv::f16_t*>(grad_output),
            nullptr, reparametrization_h, reparametrization_w, normalize, exact,
            static_cast<boxconv::f16_t*>(grad_input), grad_x_min, grad_x_max, grad_y_min, grad_y_max,
            batch, in_planes, num_filters, h, w, workspace, workspace_bytes, stream);
    if (io_dtype == BOXCONV_BF16)
        return backward_impl<float, boxconv::bf16_t>(
            input_integrated, x_min, x_max, y_min, y_max, static_cast<const boxconv::bf16_t*>(grad_output),
            nullptr, reparametrization_h, reparametrization_w, normalize, exact,
            static_cast<boxconv::bf16_t*>(grad_input), grad_x_min, grad_x_max, grad_y_min, grad_y_max,
            batch, in_planes, num_filters, h, w, workspace, workspace_bytes, stream);
    return fail(BOXCONV_E_INVALID_ARGUMENT, "backward: io_dtype %d is neither BOXCONV_F16 nor BOXCONV_BF16",
                io_dtype);
}

int boxconv_clip_parameters_f32(float* x_min, float* x_max, float* y_min, float* y_max, int n,
                                double reparametrization_h, double reparametrization_w,
                                double max_input_h, double max_input_w, int exact, void* stream) {
    return clip_impl<float>(x_min, x_max, y_min, y_max, nullptr, n, reparametrization_h,
                            reparametrization_w, max_input_h, max_input_w, exact, stream);
}
int boxconv_clip_parameters_f64(double* x_min, double* x_max, double* y_min, double* y_max, int n,
                                double reparametrization_h, double reparametrization_w,
                                double max_input_h, double max_input_w, int exact, void* stream) {
    return clip_impl<double>(x_min, x_max, y_min, y_max, nullptr, n, reparametrization_h,
                             reparametrization_w, max_input_h, max_input_w, exact, stream);
}

int boxconv_clip_reparametrize_f32(float* x_min, float* x_max, float* y_min, float* y_max,
                                   float* real_parameters, int n, double reparametrization_h,
                                   double reparametrization_w, double max_input_h,
                                   double max_input_w, int exact, void* stream) {
    if (n > 0 && real_parameters == nullptr)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "clip_reparametrize: null output pointer");
    return clip_impl<float>(x_min, x_max, y_min, y_max, real_parameters, n, reparametrization_h,
                            reparametrization_w, max_input_h, max_input_w, exact, stream);
}
int boxconv_clip_reparametrize_f64(double* x_min, double* x_max, double* y_min, double* y_max,
                                   double* real_parameters, int n, double reparametrization_h,
                                   double reparametrization_w, double max_input_h,
                                   double max_input_w, int exact, void* stream) {
    if (n > 0 && real_parameters == nullptr)
        return fail(BOXCONV_E_INVALID_ARGUMENT, "clip_reparametrize: null output pointer");
    return clip_impl<double>(x_min, x_max, y_min, y_max, real_parameters, n, reparametrization_h,
                             reparametrization_w, max_input_h, max_input_w, exact, stream);
}

}  // extern "C"
