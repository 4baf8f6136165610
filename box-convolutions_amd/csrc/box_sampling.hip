// Box-filter sampling kernels for gfx950: forward output, gradient w.r.t. the input and
// gradient w.r.t. the four box bounds. They replace
//   cpu::boxConvUpdateOutput        src/box_convolution.cpp:100-261  (CUDA: box_convolution_cuda_forward.cu:28-251)
//   cpu::boxConvUpdateGradInput     src/box_convolution.cpp:286-456  (+ tmpArray.sum(2), box_convolution_interface.cpp:274)
//   cpu::boxConvAccGradParameters   src/box_convolution.cpp:480-715  (+ the ATen mul_/sum/addcmul_ chain,
//                                   box_convolution_interface.cpp:313-391)
// and fold the three parameter splits (src/box_convolution.cpp:14-98) and computeArea (:765-793)
// into the kernels.
//
// Math. With I the integral image, a box sum with fractional bounds is separable:
//   V(i)[q] = (I[b][q] - I[t][q]) + fxhi*(I[bAdv][q] - I[b][q]) + fxlo*(I[t][q] - I[tAdv][q])
//   S(i,j)  = (V[r] - V[l]) + fyhi*(V[rAdv] - V[r]) + fylo*(V[l] - V[lAdv])
// with t = clamp(i+xlo), tAdv = clamp(i+xlo-1), b = clamp(i+xhi), bAdv = clamp(i+xhi+1) in [0,h]
// and l, lAdv, r, rAdv alike in [0,w]. Expanding S gives exactly the reference's nine terms
// (main area, four fractional borders, four corner pixels); the corner guards of the reference
// are the cases where an advanced index clamps onto the plain one and the term vanishes.
// The derivatives of S are the same expressions applied to one-row or one-column differences:
//   dS/dxmax =  H(I[bAdv]-I[b]),  dS/dxmin = -H(I[t]-I[tAdv]),   H(X) = S's column formula on X
//   dS/dymax =  V[rAdv]-V[r],     dS/dymin = -(V[l]-V[lAdv]).
//
// Row streaming. Column 0 of I is zero, so V(i) has w interesting entries. A workgroup owns a
// band of output rows at full width: each lane keeps I[t(i-1)] and I[b(i)] of its columns in
// registers, loads only the two new rows I[t(i)], I[b(i+1)] per output row (coalesced), writes
// V(i) to LDS, and after one barrier every output pixel reads its four V entries from LDS.
// That is 2 global loads per output pixel instead of 16 gathers. The row after next is
// requested before the barrier so its latency overlaps the LDS phase.
//
// Workgroup ids are remapped (xcd_contiguous_id) so all filters and bands of one input plane run
// on one XCD and its integral plane stays in that XCD's L2.

#include <cstdlib>

#include "boxconv_device.hpp"
#include "boxconv_host.hpp"

namespace boxconv {

bool force_gather_kernels() {
    const char* e = std::getenv("BOXCONV_FORCE_GATHER");
    return e != nullptr && e[0] == '1';
}

namespace {

extern __shared__ __align__(16) unsigned char smem_raw[];

template <class T>
struct SampleArgs {
    const T* src;         // integral planes, (h+1) x (w+1) each, contiguous
    BoxParams<T> prm;
    T* dst;               // forward: [B,C,F,h,w]; grad input: [B,C,h,w]
    const T* grad_out;    // param grads only: [B,C,F,h,w]
    double* acc;          // param grads only: [C*F*5]
    int C, F, h, w;
    int nb, R;            // bands per plane and rows per band
    int64_t total;        // workgroups with work
    int64_t per_xcd;      // ceil(total / 8)
    int normalize;
};

template <class T, int K>
__device__ __forceinline__ void load_row(const T* __restrict__ plane, int64_t pitch, int row,
                                         int w, int q0, int nt, T (&dst)[K]) {
    const T* r = plane + static_cast<int64_t>(row) * pitch;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const int q = q0 + nt * k;
        dst[k] = (q <= w) ? r[q] : T(0);
    }
}

template <class T, bool EXACT>
__device__ __forceinline__ T blend(T lo_adv, T lo, T hi, T hi_adv, T flo, T fhi) {
    T v = hi - lo;
    if (EXACT) v += fhi * (hi_adv - hi) + flo * (lo - lo_adv);
    return v;
}

// Row vector into LDS. Layout: V[q+1] for q = -1..w+1 with V(-1) = V(0) = 0 and V(w+1) = V(w), so
// a clamped column pair is always two adjacent entries.
template <class T, int K>
__device__ __forceinline__ void publish_row(T* __restrict__ V, const T (&val)[K], int w, int q0,
                                            int nt) {
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const int q = q0 + nt * k;
        if (q <= w) {
            V[q + 1] = val[k];
            if (q == w) V[w + 2] = val[k];
        }
    }
    if (q0 == 1) { V[0] = T(0); V[1] = T(0); }
}

struct ColumnTaps { int lo, hi; };   // LDS indices of (lAdv, l) = (lo, lo+1) and (r, rAdv) = (hi, hi+1)
__device__ __forceinline__ ColumnTaps column_taps(int j, int ylo, int yhi, int w) {
    ColumnTaps c;
    c.lo = clampi(j + ylo, 0, w + 1);        // V index of lAdv; l is the next entry
    c.hi = clampi(j + yhi, -1, w) + 1;       // V index of r; rAdv is the next entry
    return c;
}

// ---------------------------------------------------------------------------------------------
// Forward. Work item = (plane p, filter f, band). blockDim = nt, K = ceil(w / nt) <= template K.
template <class T, int K, bool EXACT>
__global__ void __launch_bounds__(256) forward_rows_kernel(SampleArgs<T> a) {
    const int64_t vid = xcd_contiguous_id(a.per_xcd);
    if (vid >= a.total) return;
    const int band = static_cast<int>(vid % a.nb);
    const int64_t pf = vid / a.nb;
    const int f = static_cast<int>(pf % a.F);
    const int64_t p = pf / a.F;
    const int k_par = static_cast<int>(p % a.C) * a.F + f;
    const int h = a.h, w = a.w, nt = blockDim.x, q0 = 1 + threadIdx.x;

    const T xmin = a.prm.xmin[k_par], xmax = a.prm.xmax[k_par];
    const T ymin = a.prm.ymin[k_par], ymax = a.prm.ymax[k_par];
    const BoxSplit<T> s = split_forward(xmin, xmax, ymin, ymax);
    const T scale = a.normalize ? inverse_extent(xmin, xmax, ymin, ymax, EXACT, true, true) : T(1);

    const int64_t pitch = w + 1;
    const T* plane = a.src + p * static_cast<int64_t>(h + 1) * pitch;
    T* out = a.dst + pf * static_cast<int64_t>(h) * w;
    T* vbuf = reinterpret_cast<T*>(smem_raw);
    const int vlen = w + 3;

    const int i0 = band * a.R;
    const int i1 = min(h, i0 + a.R);

    T pT[K], pB[K], nT[K], nB[K];
    load_row<T, K>(plane, pitch, clampi(i0 + s.xlo - 1, 0, h), w, q0, nt, pT);
    load_row<T, K>(plane, pitch, clampi(i0 + s.xhi, 0, h), w, q0, nt, pB);
    load_row<T, K>(plane, pitch, clampi(i0 + s.xlo, 0, h), w, q0, nt, nT);
    load_row<T, K>(plane, pitch, clampi(i0 + s.xhi + 1, 0, h), w, q0, nt, nB);

    for (int i = i0; i < i1; ++i) {
        T* V = vbuf + ((i - i0) & 1) * vlen;
        T fT[K] = {}, fB[K] = {};
        if (i + 1 < i1) {
            load_row<T, K>(plane, pitch, clampi(i + 1 + s.xlo, 0, h), w, q0, nt, fT);
            load_row<T, K>(plane, pitch, clampi(i + 2 + s.xhi, 0, h), w, q0, nt, fB);
        }
        T val[K];
#pragma unroll
        for (int k = 0; k < K; ++k) val[k] = blend<T, EXACT>(pT[k], nT[k], pB[k], nB[k], s.fxlo, s.fxhi);
        publish_row<T, K>(V, val, w, q0, nt);
        __syncthreads();

        T* orow = out + static_cast<int64_t>(i) * w;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int j = static_cast<int>(threadIdx.x) + nt * k;
            if (j < w) {
                const ColumnTaps c = column_taps(j, s.ylo, s.yhi, w);
                const T o = blend<T, EXACT>(V[c.lo], V[c.lo + 1], V[c.hi], V[c.hi + 1], s.fylo, s.fyhi);
                __builtin_nontemporal_store(o * scale, orow + j);
            }
        }
#pragma unroll
        for (int k = 0; k < K; ++k) { pT[k] = nT[k]; pB[k] = nB[k]; nT[k] = fT[k]; nB[k] = fB[k]; }
    }
}

// ---------------------------------------------------------------------------------------------
// Gradient w.r.t. the input. Work item = (plane p = (b,c), band of RB rows); the F mirrored boxes
// are visited in order and summed in registers, so no [B,C,F,h,w] temporary exists.
template <class T, int K, int RB, bool EXACT>
__global__ void __launch_bounds__(256) grad_input_rows_kernel(SampleArgs<T> a) {
    const int64_t vid = xcd_contiguous_id(a.per_xcd);
    if (vid >= a.total) return;
    const int band = static_cast<int>(vid % a.nb);
    const int64_t p = vid / a.nb;
    const int c_in = static_cast<int>(p % a.C);
    const int h = a.h, w = a.w, nt = blockDim.x, q0 = 1 + threadIdx.x;
    const int64_t pitch = w + 1;
    const int64_t ipl = static_cast<int64_t>(h + 1) * pitch;
    T* vbuf = reinterpret_cast<T*>(smem_raw);
    const int vlen = w + 3;
    const int i0 = band * RB;

    T acc[RB][K];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int k = 0; k < K; ++k) acc[r][k] = T(0);

    int flip = 0;
    for (int f = 0; f < a.F; ++f) {
        const int k_par = c_in * a.F + f;
        const T xmin = a.prm.xmin[k_par], xmax = a.prm.xmax[k_par];
        const T ymin = a.prm.ymin[k_par], ymax = a.prm.ymax[k_par];
        const BoxSplit<T> s = split_grad_input(xmin, xmax, ymin, ymax);
        const T scale = a.normalize ? inverse_extent(xmin, xmax, ymin, ymax, EXACT, true, true) : T(1);
        const T* plane = a.src + (p * a.F + f) * ipl;

        T pT[K], pB[K], nT[K], nB[K];
        load_row<T, K>(plane, pitch, clampi(i0 + s.xlo - 1, 0, h), w, q0, nt, pT);
        load_row<T, K>(plane, pitch, clampi(i0 + s.xhi, 0, h), w, q0, nt, pB);
        load_row<T, K>(plane, pitch, clampi(i0 + s.xlo, 0, h), w, q0, nt, nT);
        load_row<T, K>(plane, pitch, clampi(i0 + s.xhi + 1, 0, h), w, q0, nt, nB);

#pragma unroll
        for (int r = 0; r < RB; ++r) {
            const int i = i0 + r;
            if (i < h) {                                   // uniform across the workgroup
                T* V = vbuf + flip * vlen;
                flip ^= 1;
                T fT[K] = {}, fB[K] = {};
                if (r + 1 < RB && i + 1 < h) {
                    load_row<T, K>(plane, pitch, clampi(i + 1 + s.xlo, 0, h), w, q0, nt, fT);
                    load_row<T, K>(plane, pitch, clampi(i + 2 + s.xhi, 0, h), w, q0, nt, fB);
                }
                T val[K];
#pragma unroll
                for (int k = 0; k < K; ++k)
                    val[k] = blend<T, EXACT>(pT[k], nT[k], pB[k], nB[k], s.fxlo, s.fxhi);
                publish_row<T, K>(V, val, w, q0, nt);
                __syncthreads();
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    const int j = static_cast<int>(threadIdx.x) + nt * k;
                    if (j < w) {
                        const ColumnTaps c = column_taps(j, s.ylo, s.yhi, w);
                        const T o = blend<T, EXACT>(V[c.lo], V[c.lo + 1], V[c.hi], V[c.hi + 1],
                                                    s.fylo, s.fyhi);
                        acc[r][k] += o * scale;
                    }
                }
#pragma unroll
                for (int k = 0; k < K; ++k) { pT[k] = nT[k]; pB[k] = nB[k]; nT[k] = fT[k]; nB[k] = fB[k]; }
            }
        }
    }

    T* out = a.dst + p * static_cast<int64_t>(h) * w;
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        const int i = i0 + r;
        if (i < h) {
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const int j = static_cast<int>(threadIdx.x) + nt * k;
                if (j < w) out[static_cast<int64_t>(i) * w + j] = acc[r][k];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Sum of 5 per-lane values over the workgroup, then one atomic per value.
__device__ __forceinline__ void block_accumulate5(const double (&v)[5], double* __restrict__ dst,
                                                  double* __restrict__ lds /* [4*5] */) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = (blockDim.x + 63) >> 6;
#pragma unroll
    for (int n = 0; n < 5; ++n) {
        const double tot = wave_sum_to_last(v[n]);
        if (lane == 63) lds[wave * 5 + n] = tot;
    }
    __syncthreads();
    if (threadIdx.x < 5) {
        double tot = 0.0;
        for (int wv = 0; wv < waves; ++wv) tot += lds[wv * 5 + threadIdx.x];
        unsafeAtomicAdd(dst + threadIdx.x, tot);
    }
}

// Gradient w.r.t. the box bounds. Work item = (plane p, filter f, band). Accumulates, per (c,f):
//   [0] sum g*dS/dxmin  [1] sum g*dS/dxmax  [2] sum g*dS/dymin  [3] sum g*dS/dymax  [4] sum g*S
// Lanes accumulate in T over their pixels of the band, the workgroup sum is taken in double and
// leaves through one atomic per value.
template <class T, int K, bool EXACT>
__global__ void __launch_bounds__(256) grad_params_rows_kernel(SampleArgs<T> a) {
    const int64_t vid = xcd_contiguous_id(a.per_xcd);
    const bool live = vid < a.total;
    // No early return: every lane reaches the wave-wide sums below.
    const int64_t wid = live ? vid : 0;
    const int band = static_cast<int>(wid % a.nb);
    const int64_t pf = wid / a.nb;
    const int f = static_cast<int>(pf % a.F);
    const int64_t p = pf / a.F;
    const int k_par = static_cast<int>(p % a.C) * a.F + f;
    const int h = a.h, w = a.w, nt = blockDim.x, q0 = 1 + threadIdx.x;

    const T xmin = a.prm.xmin[k_par], xmax = a.prm.xmax[k_par];
    const T ymin = a.prm.ymin[k_par], ymax = a.prm.ymax[k_par];
    const BoxSplit<T> s = split_grad_params(xmin, xmax, ymin, ymax);

    const int64_t pitch = w + 1;
    const T* plane = a.src + p * static_cast<int64_t>(h + 1) * pitch;
    const T* gout = a.grad_out + pf * static_cast<int64_t>(h) * w;
    const int vlen = w + 3;
    T* vbuf = reinterpret_cast<T*>(smem_raw);                       // [2][3][vlen]
    double* red = reinterpret_cast<double*>(smem_raw + ((2 * 3 * vlen * sizeof(T) + 15) / 16) * 16);

    const int i0 = band * a.R;
    const int i1 = live ? min(h, i0 + a.R) : i0;

    T sum[5] = {T(0), T(0), T(0), T(0), T(0)};

    T pT[K], pB[K], nT[K], nB[K];
    load_row<T, K>(plane, pitch, clampi(i0 + s.xlo - 1, 0, h), w, q0, nt, pT);
    load_row<T, K>(plane, pitch, clampi(i0 + s.xhi, 0, h), w, q0, nt, pB);
    load_row<T, K>(plane, pitch, clampi(i0 + s.xlo, 0, h), w, q0, nt, nT);
    load_row<T, K>(plane, pitch, clampi(i0 + s.xhi + 1, 0, h), w, q0, nt, nB);

    for (int i = i0; i < i1; ++i) {
        T* V = vbuf + ((i - i0) & 1) * 3 * vlen;
        T* DT = V + vlen;
        T* DB = DT + vlen;
        T fT[K] = {}, fB[K] = {}, g[K];
        if (i + 1 < i1) {
            load_row<T, K>(plane, pitch, clampi(i + 1 + s.xlo, 0, h), w, q0, nt, fT);
            load_row<T, K>(plane, pitch, clampi(i + 2 + s.xhi, 0, h), w, q0, nt, fB);
        }
        const T* grow = gout + static_cast<int64_t>(i) * w;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int j = static_cast<int>(threadIdx.x) + nt * k;
            g[k] = (j < w) ? grow[j] : T(0);
        }
        T val[K], dt[K], db[K];
#pragma unroll
        for (int k = 0; k < K; ++k) {
            val[k] = blend<T, EXACT>(pT[k], nT[k], pB[k], nB[k], s.fxlo, s.fxhi);
            dt[k] = nT[k] - pT[k];
            db[k] = nB[k] - pB[k];
        }
        publish_row<T, K>(V, val, w, q0, nt);
        publish_row<T, K>(DT, dt, w, q0, nt);
        publish_row<T, K>(DB, db, w, q0, nt);
        __syncthreads();
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int j = static_cast<int>(threadIdx.x) + nt * k;
            if (j < w) {
                const ColumnTaps c = column_taps(j, s.ylo, s.yhi, w);
                const T vla = V[c.lo], vl = V[c.lo + 1], vr = V[c.hi], vra = V[c.hi + 1];
                const T S = blend<T, EXACT>(vla, vl, vr, vra, s.fylo, s.fyhi);
                const T dxmin = -blend<T, EXACT>(DT[c.lo], DT[c.lo + 1], DT[c.hi], DT[c.hi + 1], s.fylo, s.fyhi);
                const T dxmax = blend<T, EXACT>(DB[c.lo], DB[c.lo + 1], DB[c.hi], DB[c.hi + 1], s.fylo, s.fyhi);
                const T dymin = -(vl - vla);
                const T dymax = vra - vr;
                sum[0] += g[k] * dxmin;
                sum[1] += g[k] * dxmax;
                sum[2] += g[k] * dymin;
                sum[3] += g[k] * dymax;
                sum[4] += g[k] * S;
            }
        }
#pragma unroll
        for (int k = 0; k < K; ++k) { pT[k] = nT[k]; pB[k] = nB[k]; nT[k] = fT[k]; nB[k] = fB[k]; }
    }

    __syncthreads();
    const double v[5] = {static_cast<double>(sum[0]), static_cast<double>(sum[1]),
                         static_cast<double>(sum[2]), static_cast<double>(sum[3]),
                         static_cast<double>(sum[4])};
    block_accumulate5(v, a.acc + static_cast<int64_t>(k_par) * 5, red);
}

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

template <class T, bool EXACT>
__global__ void __launch_bounds__(256) forward_gather_kernel(SampleArgs<T> a) {
    const int64_t hw = static_cast<int64_t>(a.h) * a.w;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= a.total) return;
    const int64_t pf = idx / hw;
    const int pix = static_cast<int>(idx % hw);
    const int i = pix / a.w, j = pix % a.w;
    const int64_t p = pf / a.F;
    const int k_par = static_cast<int>(p % a.C) * a.F + static_cast<int>(pf % a.F);
    const T xmin = a.prm.xmin[k_par], xmax = a.prm.xmax[k_par];
    const T ymin = a.prm.ymin[k_par], ymax = a.prm.ymax[k_par];
    const BoxSplit<T> s = split_forward(xmin, xmax, ymin, ymax);
    const T scale = a.normalize ? inverse_extent(xmin, xmax, ymin, ymax, EXACT, true, true) : T(1);
    const T* plane = a.src + p * static_cast<int64_t>(a.h + 1) * (a.w + 1);
    a.dst[idx] = gather_box<T, EXACT>(plane, s, i, j, a.h, a.w) * scale;
}

template <class T, bool EXACT>
__global__ void __launch_bounds__(256) grad_input_gather_kernel(SampleArgs<T> a) {
    const int64_t hw = static_cast<int64_t>(a.h) * a.w;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= a.total) return;
    const int64_t p = idx / hw;
    const int pix = static_cast<int>(idx % hw);
    const int i = pix / a.w, j = pix % a.w;
    const int c_in = static_cast<int>(p % a.C);
    const int64_t ipl = static_cast<int64_t>(a.h + 1) * (a.w + 1);
    T acc = T(0);
    for (int f = 0; f < a.F; ++f) {
        const int k_par = c_in * a.F + f;
        const T xmin = a.prm.xmin[k_par], xmax = a.prm.xmax[k_par];
        const T ymin = a.prm.ymin[k_par], ymax = a.prm.ymax[k_par];
        const BoxSplit<T> s = split_grad_input(xmin, xmax, ymin, ymax);
        const T scale = a.normalize ? inverse_extent(xmin, xmax, ymin, ymax, EXACT, true, true) : T(1);
        acc += gather_box<T, EXACT>(a.src + (p * a.F + f) * ipl, s, i, j, a.h, a.w) * scale;
    }
    a.dst[idx] = acc;
}

// grid: (ceil(h*w/256) blocks per (p,f) plane) * planes*F; a block never straddles two planes.
template <class T, bool EXACT>
__global__ void __launch_bounds__(256) grad_params_gather_kernel(SampleArgs<T> a, int blocks_per_plane) {
    __shared__ double red[4 * 5];
    const int h = a.h, w = a.w;
    const int64_t pf = blockIdx.x / blocks_per_plane;
    const int pix = static_cast<int>(blockIdx.x % blocks_per_plane) * blockDim.x + threadIdx.x;
    const int64_t p = pf / a.F;
    const int k_par = static_cast<int>(p % a.C) * a.F + static_cast<int>(pf % a.F);
    double v[5] = {0, 0, 0, 0, 0};
    if (pix < h * w) {
        const int i = pix / w, j = pix % w;
        const BoxSplit<T> s = split_grad_params(a.prm.xmin[k_par], a.prm.xmax[k_par],
                                                a.prm.ymin[k_par], a.prm.ymax[k_par]);
        const int64_t pitch = w + 1;
        const T* plane = a.src + p * static_cast<int64_t>(h + 1) * pitch;
        const int t = clampi(i + s.xlo, 0, h), ta = clampi(i + s.xlo - 1, 0, h);
        const int b = clampi(i + s.xhi, 0, h), ba = clampi(i + s.xhi + 1, 0, h);
        const int cols[4] = {clampi(j + s.ylo - 1, 0, w), clampi(j + s.ylo, 0, w),
                             clampi(j + s.yhi, 0, w), clampi(j + s.yhi + 1, 0, w)};
        T V[4], DT[4], DB[4];
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            const T vta = plane[ta * pitch + cols[n]], vt = plane[t * pitch + cols[n]];
            const T vb = plane[b * pitch + cols[n]], vba = plane[ba * pitch + cols[n]];
            V[n] = blend<T, EXACT>(vta, vt, vb, vba, s.fxlo, s.fxhi);
            DT[n] = vt - vta;
            DB[n] = vba - vb;
        }
        const T g = a.grad_out[pf * static_cast<int64_t>(h) * w + pix];
        v[0] = static_cast<double>(g * -blend<T, EXACT>(DT[0], DT[1], DT[2], DT[3], s.fylo, s.fyhi));
        v[1] = static_cast<double>(g * blend<T, EXACT>(DB[0], DB[1], DB[2], DB[3], s.fylo, s.fyhi));
        v[2] = static_cast<double>(g * -(V[1] - V[0]));
        v[3] = static_cast<double>(g * (V[3] - V[2]));
        v[4] = static_cast<double>(g * blend<T, EXACT>(V[0], V[1], V[2], V[3], s.fylo, s.fyhi));
    }
    block_accumulate5(v, a.acc + static_cast<int64_t>(k_par) * 5, red);
}

// ---------------------------------------------------------------------------------------------
__global__ void fill_zero_kernel(double* __restrict__ p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.0;
}

// Turns the five sums per box into the four gradients (reference:
// src/box_convolution_interface.cpp:345-391): optional 1/area, the d(1/area) term
// sum(g*out) * (+-1)/(extent along the parameter's axis), and the reparametrization scale.
template <class T>
__global__ void param_grad_finalize_kernel(const double* __restrict__ acc, BoxParams<T> prm,
                                           T* g0, T* g1, T* g2, T* g3, int n, float reparam_h,
                                           float reparam_w, int normalize, int exact) {
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= n) return;
    const T xmin = prm.xmin[k], xmax = prm.xmax[k], ymin = prm.ymin[k], ymax = prm.ymax[k];
    const bool ex = exact != 0;
    const T inv_area = normalize ? inverse_extent(xmin, xmax, ymin, ymax, ex, true, true) : T(1);
    const T s = normalize ? static_cast<T>(acc[k * 5 + 4]) * inv_area : T(0);   // sum(g * output)
    T* outp[4] = {g0, g1, g2, g3};
#pragma unroll
    for (int which = 0; which < 4; ++which) {
        if (outp[which] == nullptr) continue;
        T g = static_cast<T>(acc[k * 5 + which]);
        if (normalize) {
            g *= inv_area;
            const bool is_x = which < 2;
            const T inv_ext = inverse_extent(xmin, xmax, ymin, ymax, ex, is_x, !is_x);
            const T sign = (which == 1 || which == 3) ? T(-1) : T(1);
            g = g + sign * s * inv_ext;
        }
        g *= static_cast<T>(static_cast<double>(which < 2 ? reparam_h : reparam_w));
        outp[which][k] = g;
    }
}

// ---------------------------------------------------------------------------------------------
struct RowConfig { int nt; int K; };
inline RowConfig row_config(int w) {
    RowConfig c;
    c.nt = std::min(256, ((w + 63) / 64) * 64);
    const int k = (w + c.nt - 1) / c.nt;
    c.K = k <= 1 ? 1 : k <= 2 ? 2 : k <= 4 ? 4 : 8;
    return c;
}

inline int bands_for(int64_t independent, int h, int min_rows, int64_t want) {
    int nb = static_cast<int>(std::min<int64_t>((want + independent - 1) / std::max<int64_t>(independent, 1),
                                                std::max(1, h / min_rows)));
    return std::max(nb, 1);
}

template <class T>
void finish_args(SampleArgs<T>& a, int64_t total) {
    a.total = total;
    a.per_xcd = (total + kXcds - 1) / kXcds;
}

#define BOXCONV_DISPATCH_K(KERNEL, K, ...)                                           \
    switch (K) {                                                                     \
        case 1: KERNEL(1, __VA_ARGS__); break;                                       \
        case 2: KERNEL(2, __VA_ARGS__); break;                                       \
        case 4: KERNEL(4, __VA_ARGS__); break;                                       \
        default: KERNEL(8, __VA_ARGS__); break;                                      \
    }

}  // namespace

template <class T>
hipError_t forward_launch(const T* integ, BoxParams<T> prm, T* out, Dims d, bool normalize,
                          bool exact, hipStream_t stream) {
    const int64_t planes_f = d.planes() * d.F;
    if (planes_f == 0 || d.hw() == 0) return hipSuccess;
    SampleArgs<T> a{};
    a.src = integ; a.prm = prm; a.dst = out; a.C = d.C; a.F = d.F; a.h = d.h; a.w = d.w;
    a.normalize = normalize ? 1 : 0;

    if (d.w > kMaxRowStreamWidth || force_gather_kernels()) {
        finish_args(a, planes_f * d.hw());
        const dim3 grid(static_cast<unsigned>((a.total + 255) / 256));
        if (exact) hipLaunchKernelGGL((forward_gather_kernel<T, true>), grid, dim3(256), 0, stream, a);
        else       hipLaunchKernelGGL((forward_gather_kernel<T, false>), grid, dim3(256), 0, stream, a);
        return hipGetLastError();
    }

    const RowConfig rc = row_config(d.w);
    a.nb = bands_for(planes_f, d.h, 16, 4096);
    a.R = (d.h + a.nb - 1) / a.nb;
    a.nb = (d.h + a.R - 1) / a.R;
    finish_args(a, planes_f * a.nb);
    const dim3 grid(static_cast<unsigned>(a.per_xcd * kXcds));
    const size_t lds = 2 * static_cast<size_t>(d.w + 3) * sizeof(T);
#define LAUNCH_FWD(KK, EX) \
    hipLaunchKernelGGL((forward_rows_kernel<T, KK, EX>), grid, dim3(rc.nt), lds, stream, a)
    if (exact) { BOXCONV_DISPATCH_K(LAUNCH_FWD, rc.K, true) } else { BOXCONV_DISPATCH_K(LAUNCH_FWD, rc.K, false) }
#undef LAUNCH_FWD
    return hipGetLastError();
}

template <class T>
hipError_t grad_input_launch(const T* gint, BoxParams<T> prm, T* grad_in, Dims d, bool normalize,
                             bool exact, hipStream_t stream) {
    if (d.planes() == 0 || d.hw() == 0) return hipSuccess;
    SampleArgs<T> a{};
    a.src = gint; a.prm = prm; a.dst = grad_in; a.C = d.C; a.F = d.F; a.h = d.h; a.w = d.w;
    a.normalize = normalize ? 1 : 0;

    if (d.w > kMaxRowStreamWidth || force_gather_kernels()) {
        finish_args(a, d.planes() * d.hw());
        const dim3 grid(static_cast<unsigned>((a.total + 255) / 256));
        if (exact) hipLaunchKernelGGL((grad_input_gather_kernel<T, true>), grid, dim3(256), 0, stream, a);
        else       hipLaunchKernelGGL((grad_input_gather_kernel<T, false>), grid, dim3(256), 0, stream, a);
        return hipGetLastError();
    }

    constexpr int RB = 8;
    const RowConfig rc = row_config(d.w);
    a.nb = (d.h + RB - 1) / RB;
    a.R = RB;
    finish_args(a, d.planes() * a.nb);
    const dim3 grid(static_cast<unsigned>(a.per_xcd * kXcds));
    const size_t lds = 2 * static_cast<size_t>(d.w + 3) * sizeof(T);
#define LAUNCH_GI(KK, EX) \
    hipLaunchKernelGGL((grad_input_rows_kernel<T, KK, RB, EX>), grid, dim3(rc.nt), lds, stream, a)
    if (exact) { BOXCONV_DISPATCH_K(LAUNCH_GI, rc.K, true) } else { BOXCONV_DISPATCH_K(LAUNCH_GI, rc.K, false) }
#undef LAUNCH_GI
    return hipGetLastError();
}

template <class T>
hipError_t grad_params_launch(const T* integ, const T* grad_out, BoxParams<T> prm, double* acc,
                              T* gxmin, T* gxmax, T* gymin, T* gymax, Dims d, float reparam_h,
                              float reparam_w, bool normalize, bool exact, hipStream_t stream) {
    const int n = d.C * d.F;
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((n * 5 + 255) / 256), dim3(256), 0, stream, acc, n * 5);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;

    const int64_t planes_f = d.planes() * d.F;
    if (planes_f > 0 && d.hw() > 0) {
        SampleArgs<T> a{};
        a.src = integ; a.prm = prm; a.grad_out = grad_out; a.acc = acc;
        a.C = d.C; a.F = d.F; a.h = d.h; a.w = d.w; a.normalize = normalize ? 1 : 0;
        const size_t lds = ((2 * 3 * static_cast<size_t>(d.w + 3) * sizeof(T) + 15) / 16) * 16
                           + 4 * 5 * sizeof(double);
        if (d.w > kMaxRowStreamWidth || lds > kMaxDynamicLds || force_gather_kernels()) {
            const int bpp = static_cast<int>((d.hw() + 255) / 256);
            finish_args(a, planes_f * bpp);
            const dim3 grid(static_cast<unsigned>(a.total));
            if (exact) hipLaunchKernelGGL((grad_params_gather_kernel<T, true>), grid, dim3(256), 0, stream, a, bpp);
            else       hipLaunchKernelGGL((grad_params_gather_kernel<T, false>), grid, dim3(256), 0, stream, a, bpp);
        } else {
            const RowConfig rc = row_config(d.w);
            a.nb = bands_for(planes_f, d.h, 16, 4096);
            a.R = (d.h + a.nb - 1) / a.nb;
            a.nb = (d.h + a.R - 1) / a.R;
            finish_args(a, planes_f * a.nb);
            const dim3 grid(static_cast<unsigned>(a.per_xcd * kXcds));
#define LAUNCH_GP(KK, EX) \
    hipLaunchKernelGGL((grad_params_rows_kernel<T, KK, EX>), grid, dim3(rc.nt), lds, stream, a)
            if (exact) { BOXCONV_DISPATCH_K(LAUNCH_GP, rc.K, true) } else { BOXCONV_DISPATCH_K(LAUNCH_GP, rc.K, false) }
#undef LAUNCH_GP
        }
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }

    hipLaunchKernelGGL((param_grad_finalize_kernel<T>), dim3((n + 127) / 128), dim3(128), 0, stream,
                       acc, prm, gxmin, gxmax, gymin, gymax, n, reparam_h, reparam_w,
                       normalize ? 1 : 0, exact ? 1 : 0);
    return hipGetLastError();
}

#define BOXCONV_INSTANTIATE(T)                                                                     \
    template hipError_t forward_launch<T>(const T*, BoxParams<T>, T*, Dims, bool, bool, hipStream_t); \
    template hipError_t grad_input_launch<T>(const T*, BoxParams<T>, T*, Dims, bool, bool, hipStream_t); \
    template hipError_t grad_params_launch<T>(const T*, const T*, BoxParams<T>, double*, T*, T*, T*, \
                                              T*, Dims, float, float, bool, bool, hipStream_t);

BOXCONV_INSTANTIATE(float)
BOXCONV_INSTANTIATE(double)

}  // namespace boxconv
