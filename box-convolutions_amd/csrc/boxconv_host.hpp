// Host-side declarations shared by the translation units of libboxconv_hip.so.
#pragma once
#include <cstdlib>

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

namespace boxconv {

// One call works on `planes` consecutive (batch, input plane) pairs starting at global index
// `plane0` (= b * C + c); all tensor pointers passed alongside already point at that first plane.
struct Dims {
    int C, F, h, w;      // input planes, filters per plane, image height, image width
    int64_t planes;      // (batch, plane) pairs covered by this call
    int64_t plane0;      // global index of the first one (selects the boxes: c = (plane0+p) % C)
    int64_t hw() const { return static_cast<int64_t>(h) * w; }
    int64_t integral_plane() const { return static_cast<int64_t>(h + 1) * (w + 1); }
};

// Four [C*F] arrays in real (pixel) units, device memory.
template <class T>
struct BoxParams {
    const T* xmin;
    const T* xmax;
    const T* ymin;
    const T* ymax;
};

struct IntegralPlan {
    int nb;                // horizontal bands per plane
    int R;                 // rows per band
    int64_t aux_doubles;   // scratch for the column sums of all bands but the last
    bool lookback;         // geometry fits the single-pass kernel (bands of <= 32 rows, one tile wide)
    bool plane_per_workgroup;  // planes of at most 192 rows and 256 columns: one workgroup scans a whole plane (float output)
};
// `want`: number of workgroups to aim for.
IntegralPlan plan_integral(int64_t planes, int h, int w, int64_t want = 1024);

// workspace_prepared: clip_and_prepare_integral_launch ran on this workspace with this plan and
// reported it prepared (the single-pass kernel then needs no launch to mark its hand-over words).
// reverse_order: walk the planes last to first. A kernel that re-reads what the previous kernel
// on the stream just streamed through finds the most recently touched planes still in the
// 256 MB memory-side cache if it starts with those.
template <class T>
hipError_t integral_image_launch(const T* in, T* out, int64_t planes, int h, int w, double* aux,
                                 const IntegralPlan& plan, bool workspace_prepared, bool reverse_order,
                                 hipStream_t stream);

// float32 integral image of a float16 / bfloat16 input (TI = f16_t or bf16_t), for the shapes
// integral_image_widening_applies() accepts (rows of at most 2048 columns, planes below 2 GiB).
struct f16_t;
struct bf16_t;
template <class TI>
hipError_t integral_image_widening_launch(const TI* in, float* out, int64_t planes, int h, int w,
                                          double* aux, const IntegralPlan& plan, hipStream_t stream,
                                          bool workspace_prepared = false);
bool integral_image_widening_applies(int h, int w);

// Integral image of an integer tensor (dtype: BOXCONV_U8 .. BOXCONV_I64 of include/boxconv.h),
// every entry the exact sum modulo 2^bits; no workspace. The grid holds planes * h workgroups.
constexpr int kIntU8 = 16, kIntI8 = 17, kIntI16 = 18, kIntI32 = 19, kIntI64 = 20;
hipError_t integral_image_int_launch(const void* in, void* out, int dtype, int64_t planes, int h, int w,
                                     hipStream_t stream);

// Plain copy with the grad_output pass's access pattern (see boxconv_probe_copy_bands in
// include/boxconv.h); the caller has checked the sizes.
hipError_t probe_copy_bands_launch(const float* src, float* dst, int64_t planes, int h, int w, int rows,
                                   int rows_in_flight, hipStream_t stream);

// The grad-input pass's loads and stores without its arithmetic (see
// boxconv_probe_grad_input_pattern in include/boxconv.h); the caller has checked the sizes.
hipError_t probe_grad_input_pattern_launch(const float* M, float* out, const int* xlo, const int* xhi,
                                           int64_t planes, int C, int F, int h, int mode, hipStream_t stream);

template <class T>
hipError_t forward_launch(const T* integ, BoxParams<T> prm, T* out, Dims d, bool normalize,
                          bool exact, hipStream_t stream);

// Forward with the output written as TO (float, f16_t or bf16_t; boxconv_device.hpp) and an
// optional fused tail: y = S * channel_scale[c*F+f] + channel_shift[c*F+f] + residual, then
// max(y, 0) if relu. Null pointers leave their piece out. Inference only.
template <class TO>
hipError_t forward_fused_launch(const float* integ, BoxParams<float> prm, TO* out, const TO* residual,
                                const float* channel_scale, const float* channel_shift, bool relu,
                                Dims d, bool normalize, bool exact, hipStream_t stream);

// The last step of the parameter gradients: from the five sums per box (or per box, batch item
// and band, see grad_output_stream_launch) to the four gradients.
template <class T>
struct ParamFinish {
    const double* acc;
    int batch, acc_slots;
    T* grad[4];            // w.r.t. x_min, x_max, y_min, y_max; null = not wanted
    int n_boxes;
    float reparam_h, reparam_w;
    bool normalize, exact;
    // For the one case in which sum(grad_output * output) has to follow the FORWARD split of a
    // box rather than the one the sums were taken with (see finalize_box): the integral image of
    // the input, grad_output with its element type (0: T, 1: float16, 2: bfloat16), the image size.
    const T* integ;
    const void* grad_out;
    int grad_dtype;
    int h, w, num_filters;
};

// The column workspace M of the backward pass (written by grad_output_stream_launch, read by
// grad_input_launch): per (plane, filter) h+1 rows of column_workspace_pitch(w) elements, so
// that every row starts 16-byte aligned.
inline int64_t column_workspace_pitch(int w) { return (static_cast<int64_t>(w) + 3) / 4 * 4; }
inline int64_t column_workspace_plane(int h, int w) {
    return (static_cast<int64_t>(h) + 1) * column_workspace_pitch(w);
}

// band_rows: 0 when `gint` holds true integral images, (h+1) x (w+1) per (plane, filter);
// otherwise `gint` is the column workspace M in bands of band_rows rows, each restarting at zero.
// finish (may be null): parameter-gradient sums that are complete when this launch starts; the
// row kernel then finishes them on the side (no launch of its own) and *finish_done is set.
// TO: element type of grad_in: T, or with T = float and the column workspace also f16_t / bf16_t.
template <class T, class TO>
hipError_t grad_input_launch(const T* gint, int band_rows, BoxParams<T> prm, TO* grad_in, Dims d,
                             bool normalize, bool exact, hipStream_t stream,
                             const ParamFinish<T>* finish = nullptr, bool* finish_done = nullptr);

// The streaming pass over grad_output (parameter-gradient sums and/or band-local integral).
struct StreamPlan {
    bool usable;             // false: width or LDS need outside what the streaming kernel covers
    int nb, R;               // bands per plane, rows per band (R even)
    int parts;               // workgroups that share a band for the parameter sums (1, or 2 for rows
                             // wider than 2048 columns): accumulation slots per (plane, filter) = nb * parts
};
StreamPlan plan_grad_output_stream(int64_t planes_f, int h, int w, size_t elem_size);

// acc may be null: no parameter sums. With acc_slots == sp.nb it is [all planes*F][nb][5] doubles
// and every workgroup stores its five partial sums in its own slot (nothing to clear, no atomics,
// results reproducible bit for bit); with acc_slots == 0 it is [C*F*5] doubles, cleared by
// grad_params_begin, and workgroups add atomically. grad_params_finish takes the same two values.
// column_workspace ([planes*F] planes of column_workspace_plane(h, w) elements) may be null: no
// workspace for the gradient w.r.t. the input. At least one of the two must be given.
// TG: element type of grad_out: T, or with T = float also f16_t / bf16_t (widened on load).
template <class T, class TG>
hipError_t grad_output_stream_launch(const T* integ, const TG* grad_out, BoxParams<T> prm,
                                     double* acc, int acc_slots, T* column_workspace,
                                     const StreamPlan& sp, Dims d, bool exact, hipStream_t stream);

hipError_t grad_params_begin(double* acc, int n_boxes, hipStream_t stream);
template <class T>
hipError_t grad_params_gather_launch(const T* integ, const T* grad_out, BoxParams<T> prm,
                                     double* acc, Dims d, bool exact, hipStream_t stream);
template <class T>
hipError_t grad_params_finish(const ParamFinish<T>& finish, BoxParams<T> prm, hipStream_t stream);

// One clip job: n boxes, bounds stored divided by reparam_*; real: null, or [4][n] receiving the
// clipped bounds times their reparametrization factor.
template <class T>
struct ClipArgs {
    T* xmin; T* xmax; T* ymin; T* ymax;
    T* real;
    int n;
    double reparam_h, reparam_w, max_h, max_w, min_size;
    int project;          // 0: the stored bounds are left as they are (only `real` is written)
};
template <class T>
ClipArgs<T> clip_args(T* xmin, T* xmax, T* ymin, T* ymax, T* real, int n, double reparam_h,
                      double reparam_w, double max_h, double max_w, bool exact, bool project = true);

// The clip job and whatever the integral-image launch that follows needs done to `aux`
// beforehand, in one launch. *prepared: pass it on to integral_image_launch.
template <class T>
hipError_t clip_and_prepare_integral_launch(const ClipArgs<T>& clip, int64_t planes, int w,
                                            double* aux, const IntegralPlan& plan, bool* prepared,
                                            hipStream_t stream);

// Small planes with float output (clip_rides_on_integral): the clip job in the launch of the
// integral image itself, which needs no preparation there. TI: float, f16_t or bf16_t.
bool clip_rides_on_integral(const IntegralPlan& plan, int64_t planes);
template <class TI>
hipError_t clip_and_plane_integral_launch(const ClipArgs<float>& clip, const TI* in, float* out,
                                          int64_t planes, int h, int w, const IntegralPlan& plan,
                                          hipStream_t stream);

// real: null, or [4][n] receiving the clipped bounds times their reparametrization factor.
template <class T>
hipError_t clip_launch(T* xmin, T* xmax, T* ymin, T* ymax, T* real, int n, double reparam_h,
                       double reparam_w, double max_h, double max_w, bool exact,
                       hipStream_t stream);

// Measurement and test switches (environment variables BOXCONV_*). They are read ONCE, at the
// first call that needs them, and again only by reload_switches() (exported as
// boxconv_reload_env): no entry point calls getenv on its way to a launch.
struct Switches {
    bool force_gather;        // BOXCONV_FORCE_GATHER=1: per-pixel gather kernels for every shape
    bool gi_reverse;          // BOXCONV_GI_REVERSE=0 clears it: grad-input walks the planes first to last
    bool bwd_reverse;         // BOXCONV_BWD_REVERSE=0 clears it: the same for the gather path's second pass
    bool gi_split_filters;    // BOXCONV_GI_SPLIT_FILTERS=0 clears it: no filter sharing in small grad-input launches
    bool lookback;            // BOXCONV_INTEGRAL_LOOKBACK=0 clears it: no single-pass integral image
    bool lookback_any_shape;  // BOXCONV_INTEGRAL_LOOKBACK=2: single pass for every shape it covers
    bool plane_integral;      // BOXCONV_INTEGRAL_PLANE=0 clears it: no plane-per-workgroup integral image
    bool stream_consecutive;  // BOXCONV_STREAM_CONSEC=0 clears it: no consecutive-column variant of the grad_output pass at all
    bool stream_consecutive_partial;  // BOXCONV_STREAM_CONSEC=1 clears it: that variant only for rows that fill its workgroup exactly
    bool stream_narrow_double;  // BOXCONV_STREAM_F64_NARROW=0 clears it: float64 rows with three or four columns per lane and one launch like float32
    bool interleave_workspace;  // BOXCONV_M_INTERLEAVE=0 clears it: rows of the column workspace in their natural order
    int stream_workgroups;    // BOXCONV_STREAM_WGS: workgroups the grad_output pass aims for when it cuts planes into bands (2048)
    int spin_limit;           // BOXCONV_INTEGRAL_SPIN: polls of a hand-over word before re-summing (64)
    int fwd_threads;          // BOXCONV_FWD_THREADS: 256 or 512 (512)
    int stream_threads;       // BOXCONV_STREAM_THREADS: 256 or 512 (256)
    int64_t keep_tail_bytes;  // BOXCONV_L_KEEP_MB: end of the column workspace stored with the ordinary cache policy (192 MB)
};
const Switches& switches();
void reload_switches();       // not synchronised with calls in flight on other threads

// True when the environment asks for the gather kernels (one thread per output pixel, no LDS
// row staging) instead of the row-streaming ones; the gather kernels also serve widths the
// row-streaming kernels do not cover.
inline bool force_gather_kernels() { return switches().force_gather; }

// LDS bytes one workgroup may use on the current device (hipDeviceAttributeMaxSharedMemoryPerBlock,
// looked up once per device; 0 if the query fails, which sends every shape to the gather kernels).
size_t device_lds_limit();

// Optional per-kernel timing (see boxconv_profile_arm in include/boxconv.h). When a kernel name is
// armed, every launch of that kernel is bracketed by a pair of HIP events on its stream.
void profile_before(const char* name, hipStream_t stream);
void profile_after(const char* name, hipStream_t stream);

#define BOXCONV_LAUNCH(NAME, KERNEL, GRID, BLOCK, LDS, STREAM, ...)              \
    do {                                                                          \
        ::boxconv::profile_before(NAME, STREAM);                                  \
        hipLaunchKernelGGL(KERNEL, GRID, BLOCK, LDS, STREAM, __VA_ARGS__);        \
        ::boxconv::profile_after(NAME, STREAM);                                   \
    } while (0)

constexpr int kMaxRowStreamWidth = 4096;       // float32 rows; float64 rows half of that
constexpr int kMaxScanRowsWidth = 4096;        // widest row the one-workgroup-per-row integral kernels take
constexpr int kMaxWideningWidth = 2048;        // widest float16 / bfloat16 row the integral image reads directly
constexpr size_t kMaxDynamicLds = 160 * 1024;  // LDS of a gfx950 CU, all of which one workgroup may use
                                               // (the library is built for gfx950 only; launches also
                                               // check device_lds_limit())

}  // namespace boxconv
