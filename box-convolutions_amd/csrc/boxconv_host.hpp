// Host-side declarations shared by the translation units of libboxconv_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

namespace boxconv {

struct Dims {
    int B, C, F, h, w;   // batch, input planes, filters per plane, image height, image width
    int64_t planes() const { return static_cast<int64_t>(B) * C; }
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
};
IntegralPlan plan_integral(int64_t planes, int h, int w);

template <class T>
hipError_t integral_image_launch(const T* in, T* out, int64_t planes, int h, int w, double* aux,
                                 hipStream_t stream);

template <class T>
hipError_t forward_launch(const T* integ, BoxParams<T> prm, T* out, Dims d, bool normalize,
                          bool exact, hipStream_t stream);

template <class T>
hipError_t grad_input_launch(const T* gint, BoxParams<T> prm, T* grad_in, Dims d, bool normalize,
                             bool exact, hipStream_t stream);

// acc: [C*F*5] doubles of scratch (cleared by the launch itself with a fill kernel).
// g[k] may be null for a gradient that is not wanted.
template <class T>
hipError_t grad_params_launch(const T* integ, const T* grad_out, BoxParams<T> prm, double* acc,
                              T* gxmin, T* gxmax, T* gymin, T* gymax, Dims d, float reparam_h,
                              float reparam_w, bool normalize, bool exact, hipStream_t stream);

template <class T>
hipError_t clip_launch(T* xmin, T* xmax, T* ymin, T* ymax, int n, double reparam_h,
                       double reparam_w, double max_h, double max_w, bool exact,
                       hipStream_t stream);

// True when the environment asks for the gather kernels (one thread per output pixel, no LDS
// row staging) instead of the row-streaming ones; the gather kernels also serve widths the
// row-streaming kernels do not cover.
bool force_gather_kernels();

constexpr int kMaxRowStreamWidth = 2048;
constexpr size_t kMaxDynamicLds = 64 * 1024;   // dynamic LDS a launch may request without opting in to more

}  // namespace boxconv
