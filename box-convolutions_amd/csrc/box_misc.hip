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

// Plain copy with the access pattern of the grad_output pass: a workgroup of w/4 lanes streams
// `rows` consecutive rows of one plane, 16 bytes per lane and row, `U` rows in flight, from planes
// of h rows into planes of h+1 rows (row 0 is left alone), non-temporal stores, XCD-contiguous
// workgroup ids. What this reaches is what the memory system gives a kernel with that pattern.
typedef float probe_f4 __attribute__((ext_vector_type(4)));

template <int U>
__global__ void __launch_bounds__(1024)
probe_copy_bands_kernel(const float* __restrict__ src, float* __restrict__ dst, int h, int w, int rows,
                        int nb, int64_t per_xcd, int64_t total) {
    const unsigned vid = xcd_contiguous_id(per_xcd);
    if (vid >= total) return;
    const int band = static_cast<int>(vid % static_cast<unsigned>(nb));
    const int64_t p = vid / static_cast<unsigned>(nb);
    const float* s = src + (p * h + static_cast<int64_t>(band) * rows) * w + 4 * threadIdx.x;
    float* d = dst + (p * (h + 1) + static_cast<int64_t>(band) * rows + 1) * w + 4 * threadIdx.x;
    for (int r = 0; r < rows; r += U) {
        probe_f4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = *reinterpret_cast<const probe_f4*>(s + static_cast<int64_t>(r + u) * w);
#pragma unroll
        for (int u = 0; u < U; ++u)
            __builtin_nontemporal_store(v[u], reinterpret_cast<probe_f4*>(d + static_cast<int64_t>(r + u) * w));
    }
}

}  // namespace

hipError_t probe_copy_bands_launch(const float* src, float* dst, int64_t planes, int h, int w, int rows,
                                   int rows_in_flight, hipStream_t stream) {
    const int nb = h / rows;
    const int64_t total = planes * nb;
    const int64_t per_xcd = (total + kXcds - 1) / kXcds;
    const dim3 grid(static_cast<unsigned>(per_xcd * kXcds)), block(w / 4);
    if (rows_in_flight == 2)
        BOXCONV_LAUNCH("probe_copy_bands", (probe_copy_bands_kernel<2>), grid, block, 0, stream, src, dst, h, w,
                       rows, nb, per_xcd, total);
    else if (rows_in_flight == 4)
        BOXCONV_LAUNCH("probe_copy_bands", (probe_copy_bands_kernel<4>), grid, block, 0, stream, src, dst, h, w,
                       rows, nb, per_xcd, total);
    else if (rows_in_flight == 8)
        BOXCONV_LAUNCH("probe_copy_bands", (probe_copy_bands_kernel<8>), grid, block, 0, stream, src, dst, h, w,
                       rows, nb, per_xcd, total);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

template <class T>
ClipArgs<T> clip_args(T* xmin, T* xmax, T* ymin, T* ymax, T* real, int n, double reparam_h,
                      double reparam_w, double max_h, double max_w, bool exact, bool project) {
    // float literals widened to double (src/box_convolution_interface.cpp:405-406)
    const double min_size = static_cast<double>(exact ? 1.001f : 2.001f);
    return ClipArgs<T>{xmin, xmax, ymin, ymax, real, n, reparam_h, reparam_w, max_h, max_w, min_size,
                       project ? 1 : 0};
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
                                          double, double, bool, bool);
template ClipArgs<double> clip_args<double>(double*, double*, double*, double*, double*, int, double,
                                            double, double, double, bool, bool);

}  // namespace boxconv
