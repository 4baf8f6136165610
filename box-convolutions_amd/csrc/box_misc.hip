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

// The loads and stores of the grad-input pass without its arithmetic: a workgroup of 256 lanes
// owns 8 output rows of one plane (rows of 1024 floats, 16 bytes per lane) and reads, for each of
// F filters, the 9 rows from i0 + xlo[f] - 1 and the 9 rows from i0 + xhi[f] of that filter's
// plane of M (h + 1 rows), clamped to [0, h]; it writes the 8 rows of their blend.
// mode 0: both runs (the kernel's pattern); 1: the bottom run only (every row of M is then read
// once); 2: the bottom run from M, the top run from the first 97 rows of the XCD's first planes
// (a few MB that stay in the L2: what the second read costs when it always hits).
template <int MODE>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3)))
probe_grad_input_pattern_kernel(const float* __restrict__ M, float* __restrict__ out, const int* __restrict__ xlo,
                                const int* __restrict__ xhi, int C, int F, int h, int64_t per_xcd, int64_t total) {
    unsigned vid = xcd_contiguous_id(per_xcd);
    if (vid >= total) return;
    vid = static_cast<unsigned>(total) - 1u - vid;                  // last to first, like the kernel
    const unsigned groups = static_cast<unsigned>(h / 8);
    const int i0 = static_cast<int>(vid % groups) * 8;
    const int64_t p = vid / groups;
    const int c = static_cast<int>(p % C);
    probe_f4 acc[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) acc[r] = probe_f4{0.f, 0.f, 0.f, 0.f};
    const int64_t mplane = static_cast<int64_t>(h + 1) * 1024;
#pragma unroll 1
    for (int f = 0; f < F; ++f) {
        const int lo = xlo[c * F + f], hi = xhi[c * F + f];
        const float* plane = M + (p * F + f) * mplane + 4 * threadIdx.x;
        const float* resident = M + (static_cast<int64_t>(blockIdx.x % kXcds) * F + f) * mplane + 4 * threadIdx.x;
        probe_f4 T[9], B[9];
#pragma unroll
        for (int r = 0; r <= 8; ++r) {
            const int rt = min(max(i0 + r + lo - 1, 0), h), rb = min(max(i0 + r + hi, 0), h);
            if (MODE == 0) T[r] = *reinterpret_cast<const probe_f4*>(plane + static_cast<int64_t>(rt) * 1024);
            if (MODE == 2) T[r] = *reinterpret_cast<const probe_f4*>(resident + static_cast<int64_t>((rt * 7) % 97) * 1024);
            B[r] = *reinterpret_cast<const probe_f4*>(plane + static_cast<int64_t>(rb) * 1024);
        }
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            if (MODE == 1) acc[r] += B[r] + 0.25f * (B[r + 1] - B[r]);
            else acc[r] += (B[r] - T[r + 1]) + 0.25f * (B[r + 1] - B[r]) + 0.5f * (T[r + 1] - T[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < 8; ++r)
        *reinterpret_cast<probe_f4*>(out + (p * h + i0 + r) * 1024 + 4 * threadIdx.x) = acc[r];
}

}  // namespace

hipError_t probe_grad_input_pattern_launch(const float* M, float* out, const int* xlo, const int* xhi,
                                           int64_t planes, int C, int F, int h, int mode, hipStream_t stream) {
    const int64_t total = planes * (h / 8);
    const int64_t per_xcd = (total + kXcds - 1) / kXcds;
    const dim3 grid(static_cast<unsigned>(per_xcd * kXcds)), block(256);
    if (mode == 0)
        BOXCONV_LAUNCH("probe_grad_input_pattern", (probe_grad_input_pattern_kernel<0>), grid, block, 0, stream, M, out,
                       xlo, xhi, C, F, h, per_xcd, total);
    else if (mode == 1)
        BOXCONV_LAUNCH("probe_grad_input_pattern", (probe_grad_input_pattern_kernel<1>), grid, block, 0, stream, M, out,
                       xlo, xhi, C, F, h, per_xcd, total);
    else if (mode == 2)
        BOXCONV_LAUNCH("probe_grad_input_pattern", (probe_grad_input_pattern_kernel<2>), grid, block, 0, stream, M, out,
                       xlo, xhi, C, F, h, per_xcd, total);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

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
