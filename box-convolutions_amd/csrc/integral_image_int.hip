// Integral image of integer tensors for gfx950 (uint8, int8, int16, int32, int64).
//
// The reference's CPU function takes every ATen type (AT_DISPATCH_ALL_TYPES,
// src/integral_image.cpp:14): for an integer tensor the running row sum is an int64 and every
// entry is stored back in the tensor's own type, i.e. the exact sum modulo 2^bits
// (src/integral_image.cpp:20-37). Integer addition is associative, so any summation order gives
// those bits; sums are carried in uint32 for the types of up to 32 bits and in uint64 for int64,
// whose wrap-around is exactly that modulo.
//
// BoxConv2d never integrates integers; this path exists for callers of the native
// integral_image function and is not tuned like the floating-point one: two launches,
//   1. int_row_prefix_kernel: one workgroup per (plane, row): prefix sums along the row
//      (4 columns per lane, DPP wave scan, wave totals through LDS) into out[r+1][1..w];
//   2. int_col_prefix_kernel: one lane per (plane, column): running sum down the rows, in place
//      (lane-consecutive columns: coalesced), which also clears row 0.
// The output is written once and read and written once more: 4 passes worth of bytes.

#include <type_traits>

#include "boxconv_device.hpp"
#include "boxconv_host.hpp"

namespace boxconv {

namespace {

template <class T> struct IntAcc { using type = unsigned; };
template <> struct IntAcc<long long> { using type = unsigned long long; };

template <class T, class A>
__global__ void __launch_bounds__(256)
int_row_prefix_kernel(const T* __restrict__ in, T* __restrict__ out, int h, int w) {
    __shared__ A wave_tot[2][4];
    const int64_t pr = blockIdx.x;                 // plane * h + row
    const int64_t p = pr / h;
    const int r = static_cast<int>(pr % h);
    const T* src = in + pr * w;
    T* dst = out + (p * (h + 1) + r + 1) * (static_cast<int64_t>(w) + 1);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (tid == 0) dst[0] = T(0);
    A carry = 0;
    int buf = 0;
    for (int c0 = 0; c0 < w; c0 += 1024, buf ^= 1) {
        const int c = c0 + 4 * tid;
        A v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = c + k < w ? static_cast<A>(src[c + k]) : A(0);   // sign-extends
        v[1] += v[0]; v[2] += v[1]; v[3] += v[2];
        const A incl = wave_inclusive_scan(v[3]);
        if (lane == 63) wave_tot[buf][wave] = incl;
        __syncthreads();
        A left = carry + (incl - v[3]), total = carry;
#pragma unroll
        for (int wv = 0; wv < 4; ++wv) {
            const A t = wave_tot[buf][wv];
            if (wv < wave) left += t;
            total += t;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (c + k < w) dst[c + k + 1] = static_cast<T>(left + v[k]);
        carry = total;
    }
}

template <class T, class A>
__global__ void __launch_bounds__(256)
int_col_prefix_kernel(T* __restrict__ out, int64_t planes, int h, int w) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= planes * w) return;
    const int64_t p = idx / w;
    const int c = static_cast<int>(idx % w) + 1;
    const int64_t W1 = static_cast<int64_t>(w) + 1;
    T* col = out + p * (h + 1) * W1 + c;
    col[0] = T(0);
    if (c == 1) col[-1] = T(0);
    A run = 0;
    int r = 1;
    for (; r + 3 <= h; r += 4) {
        A x[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) x[k] = static_cast<A>(col[(r + k) * W1]);
#pragma unroll
        for (int k = 0; k < 4; ++k) { run += x[k]; col[(r + k) * W1] = static_cast<T>(run); }
    }
    for (; r <= h; ++r) { run += static_cast<A>(col[r * W1]); col[r * W1] = static_cast<T>(run); }
}

template <class T>
hipError_t launch_int(const void* in, void* out, int64_t planes, int h, int w, hipStream_t stream) {
    using A = typename IntAcc<T>::type;
    BOXCONV_LAUNCH("int_row_prefix", (int_row_prefix_kernel<T, A>), dim3(static_cast<unsigned>(planes * h)),
                   dim3(256), 0, stream, static_cast<const T*>(in), static_cast<T*>(out), h, w);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    BOXCONV_LAUNCH("int_col_prefix", (int_col_prefix_kernel<T, A>),
                   dim3(static_cast<unsigned>((planes * w + 255) / 256)), dim3(256), 0, stream,
                   static_cast<T*>(out), planes, h, w);
    return hipGetLastError();
}

}  // namespace

hipError_t integral_image_int_launch(const void* in, void* out, int dtype, int64_t planes, int h, int w,
                                     hipStream_t stream) {
    if (planes == 0) return hipSuccess;
    switch (dtype) {
        case kIntU8:  return launch_int<unsigned char>(in, out, planes, h, w, stream);
        case kIntI8:  return launch_int<signed char>(in, out, planes, h, w, stream);
        case kIntI16: return launch_int<short>(in, out, planes, h, w, stream);
        case kIntI32: return launch_int<int>(in, out, planes, h, w, stream);
        case kIntI64: return launch_int<long long>(in, out, planes, h, w, stream);
        default:      return hipErrorInvalidValue;
    }
}

}  // namespace boxconv
