// Device-side helpers shared by the gfx950 kernels: box parameter splitting, clamps, wave64 scans
// and reductions. Wave size is 64 everywhere (CDNA); nothing here is written for 32-wide waves.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace boxconv {

constexpr int kWave = 64;

__device__ __forceinline__ int clampi(int v, int lo, int hi) { return max(lo, min(v, hi)); }

// Integer offsets are confined to +-2^28 so that `pixel + offset` cannot overflow; every use is
// clamped to the image afterwards, so this never changes a result for images below 2^28 pixels
// per side.
__device__ __forceinline__ int to_offset(float v) {
    return static_cast<int>(fminf(fmaxf(v, -268435456.0f), 268435456.0f));
}
__device__ __forceinline__ int to_offset(double v) {
    return static_cast<int>(fmin(fmax(v, -268435456.0), 268435456.0));
}

// One box, split into whole-pixel offsets and fractional border weights.
//   rows  t = clamp(i + xlo), b = clamp(i + xhi);   cols  l = clamp(j + ylo), r = clamp(j + yhi)
template <class T>
struct BoxSplit {
    int xlo, xhi, ylo, yhi;
    T fxlo, fxhi, fylo, fyhi;
};

// Forward split (reference: src/box_convolution.cpp:22-38).
template <class T>
__device__ __forceinline__ BoxSplit<T> split_forward(T xmin, T xmax, T ymin, T ymax) {
    BoxSplit<T> s;
    T v;
    v = ceil(xmin);  s.fxlo = v - xmin; s.xlo = to_offset(v);
    v = ceil(ymin);  s.fylo = v - ymin; s.ylo = to_offset(v);
    v = floor(xmax); s.fxhi = xmax - v; s.xhi = to_offset(v) + 1;
    v = floor(ymax); s.fyhi = ymax - v; s.yhi = to_offset(v) + 1;
    return s;
}

// Split of the box mirrored through the origin, used for the gradient w.r.t. the input
// (reference: src/box_convolution.cpp:51-67; the float expressions are kept literally).
template <class T>
__device__ __forceinline__ BoxSplit<T> split_grad_input(T xmin, T xmax, T ymin, T ymax) {
    BoxSplit<T> s;
    T v;
    v = ceil(-xmax);          s.fxlo = v + xmax;          s.xlo = to_offset(v);
    v = ceil(-ymax);          s.fylo = v + ymax;          s.ylo = to_offset(v);
    v = floor(-xmin) + T(1);  s.fxhi = -xmin + T(1) - v;  s.xhi = to_offset(v);
    v = floor(-ymin) + T(1);  s.fyhi = -ymin + T(1) - v;  s.yhi = to_offset(v);
    return s;
}

// Split used for the gradient w.r.t. the box bounds (reference: src/box_convolution.cpp:80-96,
// which pairs it with 1-based pixel loops). Returned here already shifted to 0-based pixels:
// xlo = ceil(xmin - 1) + 1, xhi = floor(xmax) + 1, so the same row/column selection as the
// forward pass applies.
template <class T>
__device__ __forceinline__ BoxSplit<T> split_grad_params(T xmin, T xmax, T ymin, T ymax) {
    BoxSplit<T> s;
    T v;
    v = ceil(xmin - T(1)); s.fxlo = v - xmin + T(1); s.xlo = to_offset(v) + 1;
    v = ceil(ymin - T(1)); s.fylo = v - ymin + T(1); s.ylo = to_offset(v) + 1;
    v = floor(xmax);       s.fxhi = xmax - v;        s.xhi = to_offset(v) + 1;
    v = floor(ymax);       s.fyhi = ymax - v;        s.yhi = to_offset(v) + 1;
    return s;
}

// 1 / ((xmax-xmin+1) * (ymax-ymin+1)), either factor optional; rounded mode shrinks the box to
// whole pixels first (reference: src/box_convolution.cpp:765-793).
template <class T>
__device__ __forceinline__ T inverse_extent(T xmin, T xmax, T ymin, T ymax, bool exact,
                                            bool use_x, bool use_y) {
    if (!exact) {
        xmin = ceil(xmin); ymin = ceil(ymin);
        xmax = floor(xmax); ymax = floor(ymax);
    }
    T acc = T(1);
    if (use_x) { T e = xmax - xmin; e += T(1); acc *= e; }
    if (use_y) { T e = ymax - ymin; e += T(1); acc *= e; }
    return T(1) / acc;
}

// ---------------------------------------------------------------------------------------------
// Cross-lane data movement (DPP). `Ctrl` values used: 0x111..0x11f row_shr:1..15,
// 0x142 row_bcast:15, 0x143 row_bcast:31. A lane whose source lane does not exist reads 0
// (bound_ctrl); a lane in a row disabled by RowMask keeps `keep`.
template <int Ctrl, int RowMask>
__device__ __forceinline__ int dpp_move(int keep, int v) {
    return __builtin_amdgcn_update_dpp(keep, v, Ctrl, RowMask, 0xf, true);
}
template <int Ctrl, int RowMask>
__device__ __forceinline__ double dpp_move(double keep, double v) {
    const int lo = dpp_move<Ctrl, RowMask>(__double2loint(keep), __double2loint(v));
    const int hi = dpp_move<Ctrl, RowMask>(__double2hiint(keep), __double2hiint(v));
    return __hiloint2double(hi, lo);
}
template <int Ctrl, int RowMask>
__device__ __forceinline__ float dpp_move(float keep, float v) {
    return __int_as_float(dpp_move<Ctrl, RowMask>(__float_as_int(keep), __float_as_int(v)));
}

// Inclusive prefix sum across the 64 lanes of a wave. All lanes must be active.
template <class A>
__device__ __forceinline__ A wave_inclusive_scan(A x) {
    // within each row of 16 lanes (every row enabled, so `keep` is never used: pass x itself
    // and no register has to be cleared first)
    x += dpp_move<0x111, 0xf>(x, x);
    x += dpp_move<0x112, 0xf>(x, x);
    x += dpp_move<0x114, 0xf>(x, x);
    x += dpp_move<0x118, 0xf>(x, x);
    const A zero = A(0);
    x += dpp_move<0x142, 0xa>(zero, x);   // lane 15 of rows 0,2 into rows 1,3
    x += dpp_move<0x143, 0xc>(zero, x);   // lane 31 into rows 2,3
    return x;
}

// Sum over the wave, valid in lane 63 (and only there). All lanes must be active.
template <class A>
__device__ __forceinline__ A wave_sum_to_last(A x) { return wave_inclusive_scan(x); }

template <class A>
__device__ __forceinline__ A read_lane(A v, int lane);
template <>
__device__ __forceinline__ double read_lane<double>(double v, int lane) {
    const int lo = __builtin_amdgcn_readlane(__double2loint(v), lane);
    const int hi = __builtin_amdgcn_readlane(__double2hiint(v), lane);
    return __hiloint2double(hi, lo);
}
template <>
__device__ __forceinline__ float read_lane<float>(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// Workgroup index remapped so that a contiguous range of work items lands on one XCD.
// Hardware hands consecutive workgroup ids to the 8 XCDs in turn; item ids are decoded with the
// slowest-varying coordinate first, so giving XCD x the range [x*per, (x+1)*per) keeps all the
// work that shares one integral plane inside one XCD's L2. Launch with 8*per workgroups,
// per = ceil(total/8); ids >= total must exit.
constexpr int kXcds = 8;
__device__ __forceinline__ int64_t xcd_contiguous_id(int64_t per_xcd) {
    const int64_t id = blockIdx.x;
    return (id % kXcds) * per_xcd + id / kXcds;
}

}  // namespace boxconv
