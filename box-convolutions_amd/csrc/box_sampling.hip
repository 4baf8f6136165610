// Host-side pieces of the box-sampling kernels that do not depend on the element type; the
// kernels themselves are templates in box_sampling_impl.hpp, instantiated by box_sampling_inst.hip.

#include <atomic>
#include <mutex>

#include "box_sampling_impl.hpp"   // stream_lds_bytes; the templates in it are not instantiated here

namespace boxconv {

namespace {

Switches read_switches() {
    auto text = [](const char* name) { return std::getenv(name); };
    auto flag_unless_zero = [&](const char* name) { const char* e = text(name); return e == nullptr || e[0] != '0'; };
    auto threads = [&](const char* name, int fallback) {
        const char* e = text(name);
        const int n = e ? std::atoi(e) : fallback;
        return (n == 256 || n == 512) ? n : fallback;
    };
    Switches s{};
    const char* e = text("BOXCONV_FORCE_GATHER");
    s.force_gather = e != nullptr && e[0] == '1';
    s.gi_reverse = flag_unless_zero("BOXCONV_GI_REVERSE");
    s.bwd_reverse = flag_unless_zero("BOXCONV_BWD_REVERSE");
    e = text("BOXCONV_GI_SPLIT_FILTERS");
    s.gi_split_filters = e == nullptr || std::atoi(e) != 0;
    e = text("BOXCONV_INTEGRAL_LOOKBACK");
    s.lookback = e == nullptr || std::atoi(e) != 0;
    s.lookback_any_shape = e != nullptr && std::atoi(e) == 2;
    s.plane_integral = flag_unless_zero("BOXCONV_INTEGRAL_PLANE");
    s.stream_consecutive = flag_unless_zero("BOXCONV_STREAM_CONSEC");
    {
        const char* e = text("BOXCONV_STREAM_CONSEC");
        s.stream_consecutive_partial = e == nullptr || (e[0] != '0' && e[0] != '1');
    }
    s.stream_narrow_double = flag_unless_zero("BOXCONV_STREAM_F64_NARROW");
    s.interleave_workspace = flag_unless_zero("BOXCONV_M_INTERLEAVE");
    e = text("BOXCONV_STREAM_WGS");
    s.stream_workgroups = e != nullptr ? std::max(1, std::atoi(e)) : 2048;
    e = text("BOXCONV_INTEGRAL_SPIN");
    s.spin_limit = e != nullptr ? std::max(0, std::atoi(e)) : 64;
    s.fwd_threads = threads("BOXCONV_FWD_THREADS", 512);
    s.stream_threads = threads("BOXCONV_STREAM_THREADS", 256);
    e = text("BOXCONV_L_KEEP_MB");
    s.keep_tail_bytes = static_cast<int64_t>(e != nullptr ? std::max(0, std::atoi(e)) : 192) << 20;
    return s;
}

std::mutex g_switch_mutex;
std::atomic<bool> g_switches_read{false};
Switches g_switches;

constexpr int kLdsDevices = 64;
std::atomic<int64_t> g_lds_limit[kLdsDevices];     // 0 = not looked up yet, -1 = query failed

}  // namespace

const Switches& switches() {
    if (!g_switches_read.load(std::memory_order_acquire)) {
        std::lock_guard<std::mutex> lock(g_switch_mutex);
        if (!g_switches_read.load(std::memory_order_relaxed)) {
            g_switches = read_switches();
            g_switches_read.store(true, std::memory_order_release);
        }
    }
    return g_switches;
}

void reload_switches() {
    std::lock_guard<std::mutex> lock(g_switch_mutex);
    g_switches = read_switches();
    g_switches_read.store(true, std::memory_order_release);
}

size_t device_lds_limit() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kLdsDevices) return 0;
    int64_t v = g_lds_limit[dev].load(std::memory_order_relaxed);
    if (v == 0) {
        int bytes = 0;
        v = hipDeviceGetAttribute(&bytes, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess && bytes > 0
                ? bytes : -1;
        g_lds_limit[dev].store(v, std::memory_order_relaxed);
    }
    return v > 0 ? static_cast<size_t>(v) : 0;
}

namespace {

__global__ void fill_zero_kernel(double* __restrict__ p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.0;
}

}  // namespace

hipError_t grad_params_begin(double* acc, int n_boxes, hipStream_t stream) {
    if (n_boxes == 0) return hipSuccess;
    BOXCONV_LAUNCH("fill_zero", fill_zero_kernel, dim3((n_boxes * 5 + 255) / 256), dim3(256), 0,
                   stream, acc, n_boxes * 5);
    return hipGetLastError();
}

StreamPlan plan_grad_output_stream(int64_t planes_f, int h, int w, size_t elem_size) {
    StreamPlan sp{};
    const RowConfig rc = stream_row_config(std::max(w, 1), elem_size);
    sp.usable = row_kernels_apply(h, w, elem_size) &&
                stream_lds_bytes(rc.K, rc.nt, elem_size) <= kMaxDynamicLds;
    int nb = bands_for(std::max<int64_t>(planes_f, 1), h, 32, switches().stream_workgroups);
    int R = (h + nb - 1) / nb;
    R += R & 1;                                        // rows are handled in pairs
    sp.R = std::max(R, 2);
    sp.nb = (h + sp.R - 1) / sp.R;
    sp.parts = (rc.nt == 1024 || stream_double_wide_split(w, elem_size)) ? 2 : 1;
    return sp;
}

}  // namespace boxconv
