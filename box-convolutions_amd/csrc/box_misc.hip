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

template <class T>
__global__ void __launch_bounds__(256) clip_kernel(ClipArgs<T> c) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < c.n) clip_box(c, i);
}

}  // namespace

template <class T>
ClipArgs<T> clip_args(T* xmin, T* xmax, T* ymin, T* ymax, T* real, int n, double reparam_h,
                      double reparam_w, double max_h, double max_w, bool exact) {
    // float literals widened to double (src/box_convolution_interface.cpp:405-406)
    const double min_size = static_cast<double>(exact ? 1.001f : 2.001f);
    return ClipArgs<T>{xmin, xmax, ymin, ymax, real, n, reparam_h, reparam_w, max_h, max_w, min_size};
}

template <class T>
hipError_t clip_launch(T* xmin, T* xmax, T* ymin, T* ymax, T* real, int n, double reparam_h,
                       double reparam_w, double max_h, double max_w, bool exact,
                       hipStream_t stream) {
    if (n == 0) return hipSuccess;
    BOXCONV_LAUNCH("clip", (clip_kernel<T>), dim3((n + 255) / 256), dim3(256), 0, stream,
                   clip_args(xmin, xmax, ymin, ymax, real, n, reparam_h, reparam_w, max_h, max_w, exact));
    return hipGetLastError();
}

template hipError_t clip_launch<float>(float*, float*, float*, float*, float*, int, double, double,
                                       double, double, bool, hipStream_t);
template hipError_t clip_launch<double>(double*, double*, double*, double*, double*, int, double,
                                        double, double, double, bool, hipStream_t);
template ClipArgs<float> clip_args<float>(float*, float*, float*, float*, float*, int, double, double,
                                          double, double, bool);
template ClipArgs<double> clip_args<double>(double*, double*, double*, double*, double*, int, double,
                                            double, double, double, bool);

}  // namespace boxconv
