// Shared by the translation units that hold the box-sampling kernels: lane/slot addressing, row
// loads, the LDS row-pair layout, the gather helpers, and the host-side choice of workgroup shape.
// Apart from the argument block SampleArgs, which crosses translation units, everything here
// lives in an unnamed namespace: each translation unit gets its own copy.
#pragma once

#include <cstdlib>
#include <type_traits>

#include "boxconv_device.hpp"
#include "boxconv_host.hpp"

namespace boxconv {

namespace {

extern __shared__ __align__(16) unsigned char smem_raw[];

// Largest workgroup of the row-streaming kernels (16 waves, for rows of 2049 to 4096 columns;
// up to 2048 columns at most 8). A wide row is spread over more lanes rather than over more than
// 4 columns per lane: per-lane state (sliding rows, prefetched rows, accumulators) scales with the
// columns per lane, and these kernels hide HBM latency with occupancy.
constexpr int kMaxRowThreads = 1024;
constexpr int kMaxRowWaves = kMaxRowThreads / 64;

}  // namespace

template <class T>
struct SampleArgs {
    const T* src;         // integral planes, (h+1) x (w+1) each, contiguous
    BoxParams<T> prm;
    T* dst;               // forward: [planes,F,h,w]; grad input: [planes,h,w]; grad_output pass: M
    const T* grad_out;    // param grads only: [planes,F,h,w]
    double* acc;          // param grads only: [C*F*5], or [planes*F*acc_slots*5] workgroup slots
    int acc_slots;        // param grads only: slots per (plane, filter), 0 = atomics on [C*F*5]
    int off_R;            // grad input only: rows per band of the column workspace M (each band restarts at zero)
    int64_t mpitch;       // elements between rows of M (a multiple of 4)
    int vec_out;          // grad input only: rows of dst are 16-byte aligned
    int band_major;       // forward only: work items ordered (plane, band, filter) instead of (plane, filter, band)
    int stream_out;       // forward only: the output is stored with the non-temporal policy
    int C, F, h, w;
    int nb, R;            // bands per plane and rows per band
    int64_t plane0;       // global index of the first plane (selects the boxes)
    int64_t total;        // workgroups with work
    int64_t per_xcd;      // ceil(total / 8)
    int normalize;
    int reverse;          // grad input only: walk the work items last to first
    int64_t keep_tail;    // grad_output pass only: bytes at the end of each XCD's share of the
                          // band-local integral that are stored with the ordinary cache policy
    int m_bands;          // rows of M interleaved over this many bands (0: rows in their natural order)
    int m_shift;          // log2 of the rows per band of M (interleaved layout only)
};

namespace {

// Where row r (0..h) of a plane of the column workspace M lives. Natural order: row r. Interleaved
// (planes of nb bands of exactly R = 2^m_shift rows): row 0 stays, row 1 + b*R + k (row k of band
// b) goes to 1 + k*nb + b, so that the nb workgroups that write the bands of one plane side by
// side, all at row k of their band at about the same time, write nb adjacent rows: the memory
// system takes writes that cluster in address space faster than as many streams 256 KB apart
// (a plain copy with either layout: 190 against 201 us for the headline's 1074 MB).
template <class T>
__device__ __forceinline__ int workspace_row(const SampleArgs<T>& a, int r) {
    if (a.m_bands == 0) return r;
    const int rr = r - 1;
    const int il = 1 + (rr & ((1 << a.m_shift) - 1)) * a.m_bands + (rr >> a.m_shift);
    return r == 0 ? 0 : il;
}

// Two rows of the same column, adjacent in LDS: every LDS access of the row kernels moves the
// values of both rows of the current row pair at once.
template <class T>
struct alignas(2 * sizeof(T)) RowPair {
    T r0, r1;
};

// Per-lane column slots. Lane `tid` owns integral columns q = 1 + tid + NT*k (pixel columns
// j = q - 1), k < K, NT = workgroup size. q1 = (1 + tid) * sizeof(T) is the byte offset of the
// lane's first column in a row of T; the other slots are compile-time distances away, so one
// register addresses all of them (instruction offsets for LDS and for buffers).
// FULL: w == K * NT, so every (lane, k) slot is a valid column and no bounds checks are compiled
// in; otherwise a slot is valid iff its byte offset is <= w * sizeof(T).
template <class T>
__device__ __forceinline__ int lane_q1() {
    return (1 + static_cast<int>(threadIdx.x)) * static_cast<int>(sizeof(T));
}
template <class T, int NT>
__device__ __forceinline__ constexpr int slot_bytes(int k) {
    return NT * k * static_cast<int>(sizeof(T));
}
template <class T, int NT, bool FULL>
__device__ __forceinline__ bool slot_valid(int q1, int k, unsigned row_bytes) {
    return FULL || static_cast<unsigned>(q1 + slot_bytes<T, NT>(k)) <= row_bytes;
}
template <class T, int NT, int POLICY>
__device__ __forceinline__ T load_slot(const RowRef& r, int q1, int k) {
    return buffer_load<POLICY>(r, q1 + slot_bytes<T, NT>(k), T());
}
template <class T, int NT, int POLICY>
__device__ __forceinline__ void store_slot(T v, const RowRef& r, int q1, int k) {
    buffer_store<POLICY>(v, r, q1 + slot_bytes<T, NT>(k));
}

// Columns 1.. of one row into the lane's slots; slots past the end of the row read 0.
template <class T, int NT, int K>
__device__ __forceinline__ void load_row(const RowRef& r, int q1, T (&dst)[K]) {
#pragma unroll
    for (int k = 0; k < K; ++k) dst[k] = load_slot<T, NT, kCacheDefault>(r, q1, k);
}

// The four rows that become new when the window moves from output rows (i-2, i-1) to (i, i+1):
// I[t(i)], I[t(i+1)], I[b(i+1)], I[b(i+2)].
template <class T, int NT, int K, bool FULL>
__device__ __forceinline__ void load_pair(const LoadRows<T>& rows, int i, int xlo, int xhi,
                                          int h, int q1, T (&t0)[K], T (&t1)[K], T (&b1)[K],
                                          T (&b2)[K]) {
    load_row<T, NT, K>(rows.row(clampi(i + xlo, 0, h)), q1, t0);
    load_row<T, NT, K>(rows.row(clampi(i + 1 + xlo, 0, h)), q1, t1);
    load_row<T, NT, K>(rows.row(clampi(i + 1 + xhi, 0, h)), q1, b1);
    load_row<T, NT, K>(rows.row(clampi(i + 2 + xhi, 0, h)), q1, b2);
}

template <class T, bool EXACT>
__device__ __forceinline__ T blend(T lo_adv, T lo, T hi, T hi_adv, T flo, T fhi) {
    // two fused multiply-adds onto the main difference (written as one sum of two products it
    // costs a multiply, a fused multiply-add and an add)
    T v = hi - lo;
    if (EXACT) {
        v += fhi * (hi_adv - hi);
        v += flo * (lo - lo_adv);
    }
    return v;
}

// Row vectors V(i), V(i+1) into LDS. Layout: V[q+1] for q = -1..w+1 with V(-1) = V(0) = 0 (written
// once by clear_row_pads) and V(w+1) = V(w), so a clamped column pair is always two adjacent
// entries.
template <class T, int NT, int K, bool FULL>
__device__ __forceinline__ void publish_rows(RowPair<T>* __restrict__ V, const T (&v0)[K],
                                             const T (&v1)[K], int w, unsigned row_bytes, int q1) {
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const RowPair<T> pr{v0[k], v1[k]};
        if (slot_valid<T, NT, FULL>(q1, k, row_bytes)) *at_bytes(V + 1 + NT * k, 2 * q1) = pr;
        if (FULL ? (k == K - 1 && static_cast<int>(threadIdx.x) == NT - 1)
                 : (static_cast<unsigned>(q1 + slot_bytes<T, NT>(k)) == row_bytes))
            V[w + 2] = pr;
    }
}
template <class T>
__device__ __forceinline__ void clear_row_pads(RowPair<T>* vbuf, int vlen) {
    if (threadIdx.x < 4) vbuf[(threadIdx.x >> 1) * vlen + (threadIdx.x & 1)] = RowPair<T>{T(0), T(0)};
}

// LDS byte offsets of the column pairs (lAdv, l) = (lo, lo+1) and (r, rAdv) = (hi, hi+1) of the
// lane's pixels.
template <class T, int NT, int K>
__device__ __forceinline__ void column_taps(unsigned (&lo)[K], unsigned (&hi)[K], int ylo, int yhi,
                                            int w) {
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const int j = static_cast<int>(threadIdx.x) + NT * k;
        lo[k] = static_cast<unsigned>(clampi(j + ylo, 0, w + 1)) * static_cast<unsigned>(sizeof(RowPair<T>));
        hi[k] = static_cast<unsigned>(clampi(j + yhi, -1, w) + 1) * static_cast<unsigned>(sizeof(RowPair<T>));
    }
}

// Box sums of one pixel column slot for both rows of the pair.
template <class T, bool EXACT>
__device__ __forceinline__ RowPair<T> sample_columns(const RowPair<T>* __restrict__ V, unsigned lo,
                                                     unsigned hi, T fylo, T fyhi) {
    const RowPair<T>* L = at_bytes(V, lo);
    const RowPair<T>* H = at_bytes(V, hi);
    const RowPair<T> l = L[1], r = H[0];
    RowPair<T> la = l, ra = r;
    if (EXACT) { la = L[0]; ra = H[1]; }
    return {blend<T, EXACT>(la.r0, l.r0, r.r0, ra.r0, fylo, fyhi),
            blend<T, EXACT>(la.r1, l.r1, r.r1, ra.r1, fylo, fyhi)};
}

template <class T>
struct BoxOfWorkgroup {
    T xmin, xmax, ymin, ymax;
};
// The box bounds are read through the constant address space: no kernel that samples boxes
// writes them, and a load the compiler may treat as invariant becomes a scalar load when its
// index is the same for the whole wave. Scalar loads are counted apart from the vector memory
// loads, so fetching a box does not wait for (or hold up) the row loads in flight around it.
template <class T>
__device__ __forceinline__ T load_invariant(const T* p) {
    typedef const T __attribute__((address_space(4))) * ConstPtr;
    return *(ConstPtr)(p);
}
template <class T>
__device__ __forceinline__ BoxOfWorkgroup<T> load_box(const BoxParams<T>& prm, int k_par) {
    return {load_invariant(prm.xmin + k_par), load_invariant(prm.xmax + k_par),
            load_invariant(prm.ymin + k_par), load_invariant(prm.ymax + k_par)};
}

using Flip0 = std::integral_constant<int, 0>;
using Flip1 = std::integral_constant<int, 1>;

// ---------------------------------------------------------------------------------------------
// Gather kernels: one thread per output pixel, the 16 integral samples are read straight from
// global memory. Any width; also the cross-check implementation for the row-streaming kernels.
template <class T, bool EXACT>
__device__ __forceinline__ T gather_V(const T* __restrict__ plane, int64_t pitch, int ta, int t,
                                      int b, int ba, int q, T fxlo, T fxhi) {
    const T vt = plane[t * pitch + q], vb = plane[b * pitch + q];
    T vta = T(0), vba = T(0);
    if (EXACT) { vta = plane[ta * pitch + q]; vba = plane[ba * pitch + q]; }
    return blend<T, EXACT>(vta, vt, vb, vba, fxlo, fxhi);
}

template <class T, bool EXACT>
__device__ __forceinline__ T gather_box(const T* __restrict__ plane, const BoxSplit<T>& s, int i,
                                        int j, int h, int w) {
    const int64_t pitch = w + 1;
    const int t = clampi(i + s.xlo, 0, h), ta = clampi(i + s.xlo - 1, 0, h);
    const int b = clampi(i + s.xhi, 0, h), ba = clampi(i + s.xhi + 1, 0, h);
    const int l = clampi(j + s.ylo, 0, w), la = clampi(j + s.ylo - 1, 0, w);
    const int r = clampi(j + s.yhi, 0, w), ra = clampi(j + s.yhi + 1, 0, w);
    const T vl = gather_V<T, EXACT>(plane, pitch, ta, t, b, ba, l, s.fxlo, s.fxhi);
    const T vr = gather_V<T, EXACT>(plane, pitch, ta, t, b, ba, r, s.fxlo, s.fxhi);
    T vla = T(0), vra = T(0);
    if (EXACT) {
        vla = gather_V<T, EXACT>(plane, pitch, ta, t, b, ba, la, s.fxlo, s.fxhi);
        vra = gather_V<T, EXACT>(plane, pitch, ta, t, b, ba, ra, s.fxlo, s.fxhi);
    }
    return blend<T, EXACT>(vla, vl, vr, vra, s.fylo, s.fyhi);
}

// ---------------------------------------------------------------------------------------------
// Workgroup shapes the row kernels are compiled for: (threads, columns per lane).
//   (64,1) widths up to 64; (128,1) up to 128; (64,3..4) up to 256; (128,3..4) up to 512;
//   (256,3..4) and (512,2..4) up to 2048; (1024,3..4) up to 4096 (float32 only; the fused
//   grad_output pass does not fit the 128 registers a lane gets at 16 waves, so there its two
//   halves run as two launches).
// Rows of up to 512 columns go to one or two waves with three or four columns per lane rather
// than to four or eight waves with one or two: the per-wave part of a row pair (scan steps,
// address and loop overhead, the waits of a workgroup-wide barrier) does not shrink with the
// columns a lane holds, and small images are bound by exactly that (measured, grad_output pass at
// 128 rows: 256 columns 55 -> 36 us, 384 columns 48 -> 30 us, 512 columns 48 -> 36 us; forward
// 23 -> 20, 25 -> 15, 24 -> 22 us). Up to 128 columns one column per lane stays (two per lane on
// one wave measured the same or slower).
// Wider rows: each kernel has a preferred size (measured at width 1024: 512 threads for forward,
// 256 for the grad_output pass); rows too wide for 4 columns per lane at that size take 512
// threads, which bounds the register footprint and the length of the per-lane float
// accumulation chains.
struct RowConfig { int nt; int K; bool full; };
inline RowConfig row_config(int w, int prefer) {
    RowConfig c;
    if (w <= 128) {
        c.nt = w <= 64 ? 64 : 128; c.K = 1;
    } else if (w <= 512) {
        c.nt = w <= 256 ? 64 : 128;
        c.K = (w + c.nt - 1) / c.nt;                   // 3 or 4
    } else if (w > 2048) {
        c.nt = 1024;
        c.K = std::min(std::max((w + 1023) / 1024, 3), 4);
    } else {
        // fewest column slots (K * threads) that cover the row; the preferred size wins ties
        const int other = prefer == 256 ? 512 : 256;
        const int kp = (w + prefer - 1) / prefer, ko = (w + other - 1) / other;
        const bool use_other = kp > 4 || (ko <= 4 && ko * other < kp * prefer);
        c.nt = use_other ? other : prefer;
        c.K = std::min(std::max(use_other ? ko : kp, 1), 4);
    }
    c.full = (c.K * c.nt == w);
    return c;
}

// The row kernels address a plane with 32-bit byte offsets and hold a full row per workgroup.
inline bool row_kernels_apply(int h, int w, size_t elem_size) {
    const uint64_t plane_bytes = (static_cast<uint64_t>(h) + 1) * (static_cast<uint64_t>(w) + 1) * elem_size;
    // rows of more than 2048 columns: float32 (and 16-bit) elements only
    const int max_w = elem_size <= 4 ? kMaxRowStreamWidth : kMaxRowStreamWidth / 2;
    return w <= max_w && plane_bytes < (1ull << 31) && !force_gather_kernels();
}

// The grad-input kernel runs right after the pass that wrote the integral of grad_output; the
// planes written last are the ones most likely still held by the memory-side cache.
inline bool reverse_grad_input() { return switches().gi_reverse; }

// The grad_output pass keeps the most state per column of all row kernels. With 8-byte elements
// three or four columns per lane need 200 to 580 registers more than a lane has: the kernels ran
// out of scratch memory, at 8 times the time of their float counterparts instead of twice. Rows of
// up to 1024 doubles therefore get at most two columns per lane (a lane's state is then what four
// columns are in floats).
// Rows of 1025 to 2048 doubles: the two jobs of the grad_output pass as two launches, the
// parameter sums by two workgroups of 512 threads per band that own half of the columns each
// (two columns per lane), the column workspace by one workgroup with three or four columns per
// lane; neither spills.
inline bool stream_double_wide_split(int w, size_t elem_size) {
    return elem_size == 8 && w > 1024 && w <= 2048 && switches().stream_narrow_double;
}
inline RowConfig stream_row_config(int w, size_t elem_size) {
    if (elem_size == 8 && w <= 1024 && switches().stream_narrow_double) {
        RowConfig c;
        if (w <= 128)      { c.nt = w <= 64 ? 64 : 128; c.K = 1; }
        else if (w <= 256) { c.nt = 128; c.K = 2; }
        else if (w <= 512) { c.nt = 256; c.K = 2; }
        else               { c.nt = 512; c.K = 2; }
        c.full = (c.K * c.nt == w);
        return c;
    }
    return row_config(w, switches().stream_threads);
}

inline int bands_for(int64_t independent, int h, int min_rows, int64_t want) {
    int nb = static_cast<int>(std::min<int64_t>((want + independent - 1) / std::max<int64_t>(independent, 1),
                                                std::max(1, h / min_rows)));
    return std::max(nb, 1);
}

template <class T>
SampleArgs<T> base_args(BoxParams<T> prm, const Dims& d) {
    SampleArgs<T> a{};
    a.prm = prm; a.C = d.C; a.F = d.F; a.h = d.h; a.w = d.w; a.plane0 = d.plane0;
    return a;
}

// The interleaved layout of M applies to planes that are cut into whole bands of a power-of-two
// number of rows; both launches that touch M derive it from (h, rows per band) alone.
template <class T>
void set_workspace_layout(SampleArgs<T>& a, int h, int band_rows) {
    a.m_bands = 0; a.m_shift = 0;
    if (!switches().interleave_workspace || band_rows < 2 || (band_rows & (band_rows - 1)) != 0 ||
        h % band_rows != 0 || h / band_rows < 2)
        return;
    a.m_bands = h / band_rows;
    while ((1 << a.m_shift) < band_rows) ++a.m_shift;
}

template <class T>
void finish_args(SampleArgs<T>& a, int64_t total) {
    a.total = total;
    a.per_xcd = (total + kXcds - 1) / kXcds;
}

// (row_config never asks for a shape that is not listed here)
#define BOXCONV_DISPATCH_K34(KERNEL, NT, K, ...)                                     \
    if ((K) == 3) { KERNEL(NT, 3, __VA_ARGS__); } else { KERNEL(NT, 4, __VA_ARGS__); }
#define BOXCONV_DISPATCH_SHAPE(KERNEL, RC, ...)                                      \
    if ((RC).nt == 64) {                                                             \
        if ((RC).K == 1) { KERNEL(64, 1, __VA_ARGS__); }                             \
        else { BOXCONV_DISPATCH_K34(KERNEL, 64, (RC).K, __VA_ARGS__) }               \
    } else if ((RC).nt == 128) {                                                     \
        if ((RC).K == 1) { KERNEL(128, 1, __VA_ARGS__); }                            \
        else if ((RC).K == 2) { BOXCONV_DISPATCH_K2(KERNEL, 128, __VA_ARGS__) }      \
        else { BOXCONV_DISPATCH_K34(KERNEL, 128, (RC).K, __VA_ARGS__) }              \
    } else if ((RC).nt == 256) {                                                     \
        if ((RC).K == 2) { BOXCONV_DISPATCH_K2(KERNEL, 256, __VA_ARGS__) }           \
        else { BOXCONV_DISPATCH_K34(KERNEL, 256, (RC).K, __VA_ARGS__) }              \
    } else if ((RC).nt == 512) {                                                     \
        if ((RC).K == 2) { KERNEL(512, 2, __VA_ARGS__); }                            \
        else { BOXCONV_DISPATCH_K34(KERNEL, 512, (RC).K, __VA_ARGS__) }              \
    } else {                                                                         \
        BOXCONV_DISPATCH_WIDE(KERNEL, (RC).K, __VA_ARGS__)                           \
    }
// two columns per lane on two or four waves: only the grad_output pass, for 8-byte arithmetic,
// instantiates these (it redefines the macro around its dispatch)
#define BOXCONV_DISPATCH_K2(KERNEL, NT, ...) { return hipErrorInvalidValue; }
// 1024 threads: instantiated for 4-byte arithmetic only (`T` is the launch function's type)
#define BOXCONV_DISPATCH_WIDE(KERNEL, K, ...)                                        \
    if constexpr (sizeof(T) <= 4) { BOXCONV_DISPATCH_K34(KERNEL, 1024, K, __VA_ARGS__) } \
    else { return hipErrorInvalidValue; }
#define BOXCONV_DISPATCH_SHAPE_EXACT_FULL(KERNEL, RC, EXACT)                         \
    if (EXACT) {                                                                     \
        if ((RC).full) { BOXCONV_DISPATCH_SHAPE(KERNEL, RC, true, true) }            \
        else           { BOXCONV_DISPATCH_SHAPE(KERNEL, RC, true, false) }           \
    } else {                                                                         \
        if ((RC).full) { BOXCONV_DISPATCH_SHAPE(KERNEL, RC, false, true) }           \
        else           { BOXCONV_DISPATCH_SHAPE(KERNEL, RC, false, false) }          \
    }

}  // namespace

}  // namespace boxconv
