// Parameter clipping for gfx950 (projected-gradient step on the four box bounds).
// Replaces cpu::clipParameters, src/box_convolution.cpp:729-763 (CUDA: box_convolution_cuda_misc.cu:190-236)
// and its wrapper src/box_convolution_interface.cpp:397-415. One launch handles the x pair and the
// y pair of every box; arithmetic is in double as in the reference. The same launch can also
// write the clipped bounds in real pixel units (stored * reparametrization, the multiplication the
// reference does in box_convolution/box_convolution_function.py:21-27 with four torch ops).

#include "boxconv_device.hpp"
#include "boxconv_host.hpp"

namespace boxconv {

namespace {

// Confine both bounds to [-(max_size+1), max_size-1] pixels, and if the box got thinner than
// min_size - 0.9999 pixels, re-centre it at that thickness. Bounds are stored divided by
// `reparam`. The midpoint is rounded to T before use, as the reference does.
template <class T>
__device__ __forceinline__ void clip_pair(T& pmin, T& pmax, double reparam, double min_size,
                                          double max_size) {
    const double inv = 1.0 / reparam;
    const double floor_v = -(max_size + 1) * inv;
    const double ceil_v = (max_size - 1) * inv;
    double lo = fmax(floor_v, fmin(ceil_v, static_cast<double>(pmin)));
    double hi = fmax(floor_v, fmin(ceil_v, static_cast<double>(pmax)));
    const double gap = (min_size - 0.9999) * inv;
    if (lo + gap > hi) {
        const T mean = static_cast<T>(0.5 * (lo + hi));
        lo = mean - 0.5 * gap;
        hi = mean + 0.5 * gap;
    }
    pmin = static_cast<T>(lo);
    pmax = static_cast<T>(hi);
}

template <class T>
__global__ void __launch_bounds__(256)
clip_kernel(T* __restrict__ xmin, T* __restrict__ xmax, T* __restrict__ ymin, T* __restrict__ ymax,
            T* __restrict__ real /* [4][n] or null */, int n, double reparam_h, double reparam_w,
            double max_h, double max_w, double min_size) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    T a = xmin[i], b = xmax[i];
    clip_pair(a, b, reparam_h, min_size, max_h);
    xmin[i] = a; xmax[i] = b;
    T c = ymin[i], d = ymax[i];
    clip_pair(c, d, reparam_w, min_size, max_w);
    ymin[i] = c; ymax[i] = d;
    if (real != nullptr) {
        // a T tensor times a Python float: the scalar is rounded to T, then one T multiplication
        const T sh = static_cast<T>(reparam_h), sw = static_cast<T>(reparam_w);
        real[i] = a * sh; real[n + i] = b * sh; real[2 * n + i] = c * sw; real[3 * n + i] = d * sw;
    }
}

}  // namespace

template <class T>
hipError_t clip_launch(T* xmin, T* xmax, T* ymin, T* ymax, T* real, int n, double reparam_h,
                       double reparam_w, double max_h, double max_w, bool exact,
                       hipStream_t stream) {
    if (n == 0) return hipSuccess;
    // float literals widened to double (src/box_convolution_interface.cpp:405-406)
    const double min_size = static_cast<double>(exact ? 1.001f : 2.001f);
    BOXCONV_LAUNCH("clip", (clip_kernel<T>), dim3((n + 255) / 256), dim3(256), 0, stream, xmin, xmax,
                   ymin, ymax, real, n, reparam_h, reparam_w, max_h, max_w, min_size);
    return hipGetLastError();
}

template hipError_t clip_launch<float>(float*, float*, float*, float*, float*, int, double, double,
                                       double, double, bool, hipStream_t);
template hipError_t clip_launch<double>(double*, double*, double*, double*, double*, int, double,
                                        double, double, double, bool, hipStream_t);

}  // namespace boxconv
