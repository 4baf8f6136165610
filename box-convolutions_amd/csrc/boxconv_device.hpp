// Device-side helpers shared by the gfx950 kernels: box parameter splitting, clamps, wave64 scans
// and reductions. Wave size is 64 everywhere (CDNA); nothing here is written for 32-wide waves.
#pragma once

#include "boxconv_host.hpp"

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

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
__device__ __forceinline__ unsigned dpp_move(unsigned keep, unsigned v) {
    return static_cast<unsigned>(dpp_move<Ctrl, RowMask>(static_cast<int>(keep), static_cast<int>(v)));
}
template <int Ctrl, int RowMask>
__device__ __forceinline__ unsigned long long dpp_move(unsigned long long keep, unsigned long long v) {
    const int lo = dpp_move<Ctrl, RowMask>(static_cast<int>(keep), static_cast<int>(v));
    const int hi = dpp_move<Ctrl, RowMask>(static_cast<int>(keep >> 32), static_cast<int>(v >> 32));
    return (static_cast<unsigned long long>(static_cast<unsigned>(hi)) << 32) | static_cast<unsigned>(lo);
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

// The same for float with the two row broadcasts written as single instructions: an addition
// whose first operand comes through DPP and which leaves the rows outside the row mask
// untouched. (From the generic form above the compiler makes a zeroed register, a DPP move and
// an addition for each of them.) The wait states a DPP read needs after the write of its source
// are part of the statement, since the compiler does not look inside it.
template <>
__device__ __forceinline__ float wave_inclusive_scan<float>(float x) {
    x += dpp_move<0x111, 0xf>(x, x);
    x += dpp_move<0x112, 0xf>(x, x);
    x += dpp_move<0x114, 0xf>(x, x);
    x += dpp_move<0x118, 0xf>(x, x);
    asm volatile("s_nop 1\n\tv_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf" : "+v"(x));
    asm volatile("s_nop 1\n\tv_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf" : "+v"(x));
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

// ---------------------------------------------------------------------------------------------
// Pointer plus a byte offset held in a 32-bit register. Global accesses written this way use a
// scalar base and one VGPR offset, LDS accesses an immediate base; no per-access address math.
template <class P>
__device__ __forceinline__ P* at_bytes(P* base, unsigned bytes) {
    using Byte = std::conditional_t<std::is_const<P>::value, const char, char>;
    return reinterpret_cast<P*>(reinterpret_cast<Byte*>(base) + bytes);
}

// Global memory is reached through raw buffer instructions: a scalar descriptor (base, size in
// bytes), a scalar byte offset and one 32-bit VGPR byte offset per access, so there is no
// per-lane 64-bit address arithmetic. The hardware checks the VGPR offset against the size: a
// load at or beyond it returns 0 and a store there is dropped.
constexpr int kCacheDefault = 0, kCacheStream = 2;   // buffer cache policy bits: 2 = non-temporal
template <class T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const T* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(base), 0, static_cast<int>(bytes), 0x00020000);
}

// One row of a stack of rows: descriptor plus scalar offset. Must be wave-uniform.
struct RowRef {
    __amdgpu_buffer_rsrc_t rs;
    int soff;
};

// A stack of equally long rows of T in global memory (`cols` elements of each row reachable,
// rows `pitch` elements apart, the whole stack below 4 GiB).
//   BY_OFFSET: one descriptor spans the stack and a row is selected by its scalar byte offset.
//              Only for stacks where every column slot of every lane is a valid column (there
//              is no per-row bounds check). Measured: good for stores, slower than per-row
//              descriptors for loads, so loads never use it.
//   else     : one descriptor per row, sized to the row, so that the bounds check masks the
//              column slots past its end.
// A row that does not `exist` gets size 0: loads give 0, stores vanish, no branch needed.
template <class T, bool BY_OFFSET>
struct Rows {
    T* base;
    unsigned pitch_bytes, row_bytes, stack_bytes;
    __device__ __forceinline__ Rows(T* base_, int64_t pitch, int cols, int nrows)
        : base(base_), pitch_bytes(static_cast<unsigned>(pitch * sizeof(T))),
          row_bytes(static_cast<unsigned>(cols) * static_cast<unsigned>(sizeof(T))),
          stack_bytes(static_cast<unsigned>(nrows - 1) * pitch_bytes + row_bytes) {}
    __device__ __forceinline__ RowRef row(int r, bool exists = true) const {
        const unsigned offset = static_cast<unsigned>(r) * pitch_bytes;
        if constexpr (BY_OFFSET)
            return {make_buffer(base, exists ? stack_bytes : 0u), static_cast<int>(offset)};
        else
            return {make_buffer(at_bytes(base, offset), exists ? row_bytes : 0u), 0};
    }
};
template <class T> using LoadRows = Rows<const T, false>;

template <int POLICY>
__device__ __forceinline__ float buffer_load(const RowRef& r, int off, float) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r.rs, off, r.soff, POLICY));
}
template <int POLICY>
__device__ __forceinline__ double buffer_load(const RowRef& r, int off, double) {
    return __builtin_bit_cast(double, __builtin_amdgcn_raw_buffer_load_b64(r.rs, off, r.soff, POLICY));
}
template <int POLICY>
__device__ __forceinline__ void buffer_store(float v, const RowRef& r, int off) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r.rs, off, r.soff, POLICY);
}
template <int POLICY>
__device__ __forceinline__ void buffer_store(double v, const RowRef& r, int off) {
    typedef unsigned v2u __attribute__((__vector_size__(8)));
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u, v), r.rs, off, r.soff, POLICY);
}

// 16-bit storage types for kernels that compute in float but read or write half precision
// (IEEE binary16 and bfloat16). Conversions round to nearest even.
struct f16_t { unsigned short bits; };
struct bf16_t { unsigned short bits; };
__device__ __forceinline__ float widen(float v) { return v; }
__device__ __forceinline__ double widen(double v) { return v; }
__device__ __forceinline__ float widen(f16_t v) {
    return static_cast<float>(__builtin_bit_cast(_Float16, v.bits));
}
__device__ __forceinline__ float widen(bf16_t v) {
    return __builtin_bit_cast(float, static_cast<unsigned>(v.bits) << 16);
}
__device__ __forceinline__ void narrow(float v, float& o) { o = v; }
__device__ __forceinline__ void narrow(double v, double& o) { o = v; }
__device__ __forceinline__ void narrow(float v, f16_t& o) {
    // The conversion is kept a separate instruction: left to the compiler it is merged with the
    // multiplication in front of it into one mixed-precision operation that rounds once
    // (differing from "float32 result, then converted" on ties) and measured slower.
    unsigned r;
    asm("v_cvt_f16_f32 %0, %1" : "=v"(r) : "v"(v));
    o.bits = static_cast<unsigned short>(r);
}
__device__ __forceinline__ void narrow(float v, bf16_t& o) {
    o.bits = __builtin_bit_cast(unsigned short, static_cast<__bf16>(v));
}
template <int POLICY>
__device__ __forceinline__ f16_t buffer_load(const RowRef& r, int off, f16_t) {
    return {static_cast<unsigned short>(__builtin_amdgcn_raw_buffer_load_b16(r.rs, off, r.soff, POLICY))};
}
template <int POLICY>
__device__ __forceinline__ bf16_t buffer_load(const RowRef& r, int off, bf16_t) {
    return {static_cast<unsigned short>(__builtin_amdgcn_raw_buffer_load_b16(r.rs, off, r.soff, POLICY))};
}
template <int POLICY>
__device__ __forceinline__ void buffer_store(f16_t v, const RowRef& r, int off) {
    __builtin_amdgcn_raw_buffer_store_b16(v.bits, r.rs, off, r.soff, POLICY);
}
template <int POLICY>
__device__ __forceinline__ void buffer_store(bf16_t v, const RowRef& r, int off) {
    __builtin_amdgcn_raw_buffer_store_b16(v.bits, r.rs, off, r.soff, POLICY);
}

// K consecutive elements per lane starting at byte offset `off` of a row of `limit` bytes. A
// lane whose run lies inside the row stores it with one wide instruction (16, 12 or 8 bytes;
// dword alignment suffices); the at most one lane per row whose run straddles the end goes
// element by element, each store checked against the row size. WHOLE: every lane's run lies
// inside the row, nothing to test.
//
// A buffer store of more than 8 bytes per lane reads its data registers over several cycles
// after issue. Observed once: with a scalar offset register on the store (the stacked descriptors
// of `Rows` above), a conversion to double scheduled right behind a 16-byte store replaced the
// first two dwords of the data in some lanes (row h of the column workspace at width 2048). The
// working hypothesis is a store-data hazard that the compiler's hazard recogniser does not cover
// for this form; it has not been confirmed beyond that observation and the fact that wait states
// behind the store remove it. settle_wide_store therefore takes the data registers as an operand
// of the wait-state statement: their live range then extends past the wait states, so no
// instruction that overwrites them can be scheduled in between.
template <class V>
__device__ __forceinline__ void settle_wide_store(const V& data) { asm volatile("s_nop 1" : : "v"(data)); }

template <int POLICY, int K>
__device__ __forceinline__ void buffer_store_wide(const float (&v)[K], const RowRef& r, int off) {
    typedef unsigned v4u __attribute__((__vector_size__(16)));
    typedef unsigned v3u __attribute__((__vector_size__(12)));
    typedef unsigned v2u __attribute__((__vector_size__(8)));
    if constexpr (K % 4 == 0) {
#pragma unroll
        for (int k = 0; k < K; k += 4) {
            const v4u pack = {__builtin_bit_cast(unsigned, v[k]), __builtin_bit_cast(unsigned, v[k + 1]),
                              __builtin_bit_cast(unsigned, v[k + 2]), __builtin_bit_cast(unsigned, v[k + 3])};
            __builtin_amdgcn_raw_buffer_store_b128(pack, r.rs, off + 4 * k, r.soff, POLICY);
            settle_wide_store(pack);
        }
    } else if constexpr (K == 3) {
        const v3u pack = {__builtin_bit_cast(unsigned, v[0]), __builtin_bit_cast(unsigned, v[1]),
                          __builtin_bit_cast(unsigned, v[2])};
        __builtin_amdgcn_raw_buffer_store_b96(pack, r.rs, off, r.soff, POLICY);
        settle_wide_store(pack);
    } else if constexpr (K == 2) {
        const v2u pack = {__builtin_bit_cast(unsigned, v[0]), __builtin_bit_cast(unsigned, v[1])};
        __builtin_amdgcn_raw_buffer_store_b64(pack, r.rs, off, r.soff, POLICY);
    } else {
#pragma unroll
        for (int k = 0; k < K; ++k) buffer_store<POLICY>(v[k], r, off + 4 * k);
    }
}
template <int POLICY, bool WHOLE, int K>
__device__ __forceinline__ void buffer_store_run(const float (&v)[K], const RowRef& r, int off, int limit) {
    if (WHOLE || off + 4 * K <= limit) {
        buffer_store_wide<POLICY, K>(v, r, off);
    } else {
#pragma unroll
        for (int k = 0; k < K; ++k) buffer_store<POLICY>(v[k], r, off + 4 * k);
    }
}
template <int POLICY, bool WHOLE, int K>
__device__ __forceinline__ void buffer_store_run(const double (&v)[K], const RowRef& r, int off, int limit) {
    (void)limit;
#pragma unroll
    for (int k = 0; k < K; ++k) buffer_store<POLICY>(v[k], r, off + 8 * k);
}

// K consecutive elements per lane, element by element, each checked against the row size.
// (There is deliberately no 16-byte variant: this toolchain lowers the 128-bit raw buffer LOAD
// builtin to a 32-bit load. 16-byte loads go through load_quad below.)
template <int POLICY, class T, int K>
__device__ __forceinline__ void buffer_load_run(T (&v)[K], const RowRef& r, int off) {
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = buffer_load<POLICY>(r, off + static_cast<int>(sizeof(T)) * k, T());
}

// Four consecutive elements from a 16-byte aligned address with one (float) or two (double)
// 16-byte non-temporal global loads.
__device__ __forceinline__ void load_quad(const float* p, float (&v)[4]) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const f4 q = __builtin_nontemporal_load(reinterpret_cast<const f4*>(p));
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
}
__device__ __forceinline__ void load_quad(const double* p, double (&v)[4]) {
    typedef double d2 __attribute__((ext_vector_type(2)));
    const d2 q0 = __builtin_nontemporal_load(reinterpret_cast<const d2*>(p));
    const d2 q1 = __builtin_nontemporal_load(reinterpret_cast<const d2*>(p) + 1);
    v[0] = q0.x; v[1] = q0.y; v[2] = q1.x; v[3] = q1.y;
}

// ---------------------------------------------------------------------------------------------
// Parameter clipping (reference cpu::clipParameters, src/box_convolution.cpp:729-763).
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

// Box i of a clip job: both pairs clipped in place (if the job projects), and optionally written in
// real pixel units.
template <class T>
__device__ __forceinline__ void clip_box(const ClipArgs<T>& c, int i) {
    T a = c.xmin[i], b = c.xmax[i];
    T lo = c.ymin[i], hi = c.ymax[i];
    if (c.project) {                                   // (off: the bounds are only converted, nothing is stored to them)
        clip_pair(a, b, c.reparam_h, c.min_size, c.max_h);
        c.xmin[i] = a; c.xmax[i] = b;
        clip_pair(lo, hi, c.reparam_w, c.min_size, c.max_w);
        c.ymin[i] = lo; c.ymax[i] = hi;
    }
    if (c.real != nullptr) {
        // a T tensor times a Python float: the scalar is rounded to T, then one T multiplication
        const T sh = static_cast<T>(c.reparam_h), sw = static_cast<T>(c.reparam_w);
        const int n = c.n;
        c.real[i] = a * sh; c.real[n + i] = b * sh; c.real[2 * n + i] = lo * sw; c.real[3 * n + i] = hi * sw;
    }
}

// The same for half-precision sources (one 8-byte load), widened to float.
__device__ __forceinline__ void unpack_quad(unsigned lo, unsigned hi, f16_t (&h)[4]) {
    h[0].bits = static_cast<unsigned short>(lo & 0xffffu); h[1].bits = static_cast<unsigned short>(lo >> 16);
    h[2].bits = static_cast<unsigned short>(hi & 0xffffu); h[3].bits = static_cast<unsigned short>(hi >> 16);
}
template <class H>
__device__ __forceinline__ void load_quad_half(const H* p, float (&v)[4]) {
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    const u2 q = __builtin_nontemporal_load(reinterpret_cast<const u2*>(p));
    f16_t raw[4];
    unpack_quad(q.x, q.y, raw);
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = widen(H{raw[k].bits});
}
__device__ __forceinline__ void load_quad(const f16_t* p, float (&v)[4]) { load_quad_half(p, v); }
__device__ __forceinline__ void load_quad(const bf16_t* p, float (&v)[4]) { load_quad_half(p, v); }

// K consecutive elements of type TI per lane, element by element, converted to T.
template <int POLICY, class TI, class T, int K>
__device__ __forceinline__ void buffer_load_run_as(T (&v)[K], const RowRef& r, int off) {
#pragma unroll
    for (int k = 0; k < K; ++k)
        v[k] = static_cast<T>(widen(buffer_load<POLICY>(r, off + static_cast<int>(sizeof(TI)) * k, TI())));
}

// Workgroup index remapped so that a contiguous range of work items lands on one XCD.
// Hardware hands consecutive workgroup ids to the 8 XCDs in turn; item ids are decoded with the
// slowest-varying coordinate first, so giving XCD x the range [x*per, (x+1)*per) keeps all the
// work that shares one integral plane inside one XCD's L2. Launch with 8*per workgroups,
// per = ceil(total/8); ids >= total must exit.
constexpr int kXcds = 8;
// A grid has fewer than 2^31 workgroups, so 32-bit arithmetic is exact (and much cheaper than
// 64-bit division in scalar code).
__device__ __forceinline__ unsigned xcd_contiguous_id(int64_t per_xcd) {
    const unsigned id = blockIdx.x;
    return (id % kXcds) * static_cast<unsigned>(per_xcd) + id / kXcds;
}

}  // namespace boxconv
