// Box-filter sampling kernels for gfx950 (templates; instantiated by box_sampling_inst.hip, once
// per element type and part, so that the instantiations compile in parallel): forward output, gradient w.r.t. the input and
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
// registers and loads only the new rows I[t(i)], I[b(i+1)] per output row (coalesced raw buffer
// loads: scalar row descriptor, one offset register per lane). Two output rows are handled per
// barrier, and the loads of the next two are issued before the barrier. The two rows of a pair
// sit interleaved in LDS, so one LDS access serves both.
//   forward / grad input: V(i), V(i+1) go to LDS; every output pixel reads its four V entries.
//   parameter gradients : the rows of grad_output go to LDS instead and every column q reads
//       the four grad_output entries whose box edges fall on q (the transposed access), so V and
//       the two row differences never leave registers: sum_j g[j]*H(X)[j] = sum_q X[q]*Ht(g)[q].
// The workgroup size NT and the columns per lane K are template parameters (row_config picks the
// tightest shape for a width), which turns every slot distance into an instruction offset.
//
// Workgroup ids are remapped (xcd_contiguous_id) so all filters and bands of one input plane run
// on one XCD and its integral plane stays in that XCD's L2.

#pragma once

#include "box_sampling_common.hpp"

namespace boxconv {

namespace {

// Turns the five sums per box into the four gradients (reference:
// src/box_convolution_interface.cpp:345-391): optional 1/area, the d(1/area) term
// sum(g*out) * (+-1)/(extent along the parameter's axis), and the reparametrization scale.
// One wave per box. slots == 0: acc holds the five sums per box. Otherwise acc holds one slot of
// five partial sums per (batch item b, box, band): [(b*n + box)*slots + band][5]; the wave adds
// them in a fixed order.
template <class T>
struct FinalizeArgs {
    const double* acc;     // null: nothing to do
    int batch, slots;
    T* g[4];               // gradients w.r.t. x_min, x_max, y_min, y_max; null = not wanted
    int n;                 // boxes
    float reparam_h, reparam_w;
    int normalize, exact;
    const T* integ;        // integral image of the input, [batch][n / F planes][(h+1) x (w+1)]
    const void* grad_out;  // [batch][n][h x w], elements of T (grad_dtype 0), f16_t (1) or bf16_t (2)
    int grad_dtype, h, w, F;
};

// sum over batch and pixels of grad_output * (box sum with the FORWARD split, rounded mode), for
// box k, by one wave; the total is valid in lane 63. Only used for the rare boxes described in
// finalize_box: a plain loop over the pixels, 4 integral-image samples each.
template <class T>
__device__ __forceinline__ double forward_split_sum(const FinalizeArgs<T>& fa, const BoxParams<T>& prm,
                                                 int k, int lane) {
    const T xmin = prm.xmin[k], xmax = prm.xmax[k], ymin = prm.ymin[k], ymax = prm.ymax[k];
    const BoxSplit<T> s = split_forward(xmin, xmax, ymin, ymax);
    const int h = fa.h, w = fa.w;
    const int64_t hw = static_cast<int64_t>(h) * w, ipl = static_cast<int64_t>(h + 1) * (w + 1);
    const int c = k / fa.F, C = fa.n / fa.F;
    double sum = 0.0;
    for (int b = 0; b < fa.batch; ++b) {
        const T* plane = fa.integ + (static_cast<int64_t>(b) * C + c) * ipl;
        const int64_t g0 = (static_cast<int64_t>(b) * fa.n + k) * hw;
        for (int64_t pix = lane; pix < hw; pix += 64) {
            const int i = static_cast<int>(pix / w), j = static_cast<int>(pix % w);
            T g;
            if (fa.grad_dtype == 1)      g = static_cast<T>(widen(static_cast<const f16_t*>(fa.grad_out)[g0 + pix]));
            else if (fa.grad_dtype == 2) g = static_cast<T>(widen(static_cast<const bf16_t*>(fa.grad_out)[g0 + pix]));
            else                         g = static_cast<const T*>(fa.grad_out)[g0 + pix];
            sum += static_cast<double>(g * gather_box<T, false>(plane, s, i, j, h, w));
        }
    }
    return wave_sum_to_last(sum);
}

template <class T>
__device__ __forceinline__ void finalize_box(const FinalizeArgs<T>& fa, const BoxParams<T>& prm,
                                             int k, int lane) {
    double sum[5] = {0.0, 0.0, 0.0, 0.0, 0.0};
    if (fa.slots > 0) {
        const int per_box = fa.batch * fa.slots;
        for (int e = lane; e < per_box; e += 64) {
            const int b = e / fa.slots, band = e % fa.slots;
            const double* part = fa.acc + ((static_cast<int64_t>(b) * fa.n + k) * fa.slots + band) * 5;
#pragma unroll
            for (int m = 0; m < 5; ++m) sum[m] += part[m];
        }
#pragma unroll
        for (int m = 0; m < 5; ++m) sum[m] = wave_sum_to_last(sum[m]);
    } else {
#pragma unroll
        for (int m = 0; m < 5; ++m) sum[m] = fa.acc[k * 5 + m];
    }
    const T xmin = prm.xmin[k], xmax = prm.xmax[k], ymin = prm.ymin[k], ymax = prm.ymax[k];
    const bool ex = fa.exact != 0;
    // sum[4] = sum(grad_output * box sum) was taken with the split of the parameter-gradient pass
    // (src/box_convolution.cpp:80-96); the reference multiplies grad_output with the saved forward
    // OUTPUT (src/box_convolution_interface.cpp:355-358), i.e. the forward split (:22-38). The two
    // cut a box at different whole pixels only when a lower bound lies so closely above an integer
    // that `bound - 1` rounds to the integer below. In exact mode the border weights make up for
    // it to the last digits; in rounded mode a whole row or column of the box is at stake, and the
    // sum is taken again with the forward split (wave-uniform branch, next to never taken).
    if (fa.normalize && !ex && fa.integ != nullptr && fa.grad_out != nullptr &&
        (ceil(xmin) != ceil(xmin - T(1)) + T(1) || ceil(ymin) != ceil(ymin - T(1)) + T(1)))
        sum[4] = forward_split_sum(fa, prm, k, lane);
    if (lane != 63) return;
    const T inv_area = fa.normalize ? inverse_extent(xmin, xmax, ymin, ymax, ex, true, true) : T(1);
    const T s = fa.normalize ? static_cast<T>(sum[4]) * inv_area : T(0);   // sum(g * output)
#pragma unroll
    for (int which = 0; which < 4; ++which) {
        if (fa.g[which] == nullptr) continue;
        T g = static_cast<T>(sum[which]);
        if (fa.normalize) {
            g *= inv_area;
            const bool is_x = which < 2;
            const T inv_ext = inverse_extent(xmin, xmax, ymin, ymax, ex, is_x, !is_x);
            const T sign = (which == 1 || which == 3) ? T(-1) : T(1);
            g = g + sign * s * inv_ext;
        }
        g *= static_cast<T>(static_cast<double>(which < 2 ? fa.reparam_h : fa.reparam_w));
        fa.g[which][k] = g;
    }
}

template <class T>
__global__ void __launch_bounds__(64)
param_grad_finalize_kernel(FinalizeArgs<T> fa, BoxParams<T> prm) {
    finalize_box(fa, prm, static_cast<int>(blockIdx.x), static_cast<int>(threadIdx.x));
}

// ---------------------------------------------------------------------------------------------
// Gradient w.r.t. the input from the column workspace M that grad_output_stream_kernel leaves:
//   M[pf][r][c], r = 0..h, rows `mpitch` elements apart (a multiple of 4: rows are 16-byte aligned)
//   M[pf][r][c] = sum over the rows i' of the band that row r lies in, i' < r, of A(i')[c],
// A(i')[c] being row i' of grad_output filtered along the row with the mirrored box (the adjoint
// of the forward's column formula). Integral row r (1..h) belongs to band (r-1)/off_R and row 0
// to band 0; each band restarts at zero. The running sum over ALL rows above r is therefore
// I[r] = M[r] + base(band(r)), base(b) = sum of the bottom rows M[(b'+1)*off_R] of the bands b' < b,
// and
//   grad_input(i, c) = sum_f scale_f * ((I[b] - I[t]) + fxhi*(I[bAdv] - I[b]) + fxlo*(I[t] - I[tAdv]))[c]
// with t = clamp(i+xlo), tAdv = clamp(i+xlo-1), b = clamp(i+xhi), bAdv = clamp(i+xhi+1) in [0,h]
// from the split of the mirrored box (reference src/box_convolution.cpp:51-67, :286-456; the sum
// over filters is tmpArray.sum(2), src/box_convolution_interface.cpp:274).
//
// Everything is local to a column: no LDS, no barriers, any tiling. A lane owns 4 consecutive
// columns (one 16-byte load per row); 2^LQ lanes side by side cover a strip of 4*2^LQ columns
// and RB consecutive output rows; a workgroup holds NTX / 2^LQ such row groups (one for rows of
// 256 columns and more: then every row index is wave-uniform and stays in scalar registers).
// Per filter a lane loads the RB+1 rows i0+xlo-1 .. and the RB+1 rows i0+xhi .. (all in flight
// together); both runs are shorter than a band, so each starts in one band and crosses into the
// next at most once:
//   I_t[r] = M_t[r] + [row beyond the first band of the run] * E_t          (relative to that band)
//   I_b[r] = M_b[r] + off_b + [row beyond ...] * E_b,   off_b = base(band_b) - base(band_t),
// E = bottom row of the band being left; off_b is summed in double.
//
// FS > 1 (small problems): threadIdx.y selects one of FS sets of threads; set g visits the
// filters g, g + FS, ... and the FS partial sums are added in that order through LDS at the end.
// A small launch cannot fill the chip with workgroups, and a workgroup that walks through all F
// filters alone is one chain of F memory round trips.
template <class T>
struct alignas(sizeof(T) >= 4 ? 16 : 4 * sizeof(T)) Quad {
    T v[4];
};

// TO: element type of grad_input (T, or a 16-bit type when T is float: a.dst then points at
// elements of TO and the sums are rounded to it in the store).
template <class T, class TO, int LQ, int RB, bool EXACT, int FS>
__global__ void __launch_bounds__((LQ > 6 ? (1 << LQ) : 64) * FS)
grad_input_cols_kernel(SampleArgs<T> a, FinalizeArgs<T> fin) {
    constexpr int NTX = LQ > 6 ? (1 << LQ) : 64;
    constexpr int RG = NTX >> LQ;                    // row groups per workgroup
    // Rides along: the first fin.n workgroups each finish the parameter gradients of one box from
    // the sums the preceding launch left (one wave's work; saves a launch of its own).
    if (fin.acc != nullptr && blockIdx.x < static_cast<unsigned>(fin.n) && threadIdx.x < 64 &&
        threadIdx.y == 0)
        finalize_box(fin, a.prm, static_cast<int>(blockIdx.x), static_cast<int>(threadIdx.x));
    unsigned vid = xcd_contiguous_id(a.per_xcd);
    if (vid >= a.total) return;
    if (a.reverse) vid = static_cast<unsigned>(a.total) - 1u - vid;
    const int h = a.h, w = a.w;
    const unsigned strips = static_cast<unsigned>((w + (4 << LQ) - 1) / (4 << LQ));
    const int strip = static_cast<int>(vid % strips);
    vid /= strips;
    const unsigned nbands = a.nb;
    const int band = static_cast<int>(vid % nbands);
    const int64_t p = vid / nbands;
    const int c_in = static_cast<int>(static_cast<unsigned>(a.plane0 + p) % static_cast<unsigned>(a.C));
    const int tid = threadIdx.x;
    const int rg = RG > 1 ? tid >> LQ : 0;
    const int i0 = (band * RG + rg) * RB;
    const int c0 = strip * (4 << LQ) + 4 * (tid & ((1 << LQ) - 1));
    const bool lane_in = c0 < w;
    const int cl = lane_in ? c0 : 0;                 // idle lanes read column 0 and store nothing
    const int64_t mpitch = a.mpitch;
    const int64_t mplane = static_cast<int64_t>(h + 1) * mpitch;
    const int fgroup = FS > 1 ? __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.y)) : 0;
    const int R = a.off_R;

    T acc[RB][4];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[r][v] = T(0);

#pragma unroll 1
    for (int f = fgroup; f < a.F; f += FS) {
        const BoxOfWorkgroup<T> bx = load_box(a.prm, c_in * a.F + f);
        const BoxSplit<T> s = split_grad_input(bx.xmin, bx.xmax, bx.ymin, bx.ymax);
        const T scale = a.normalize
            ? inverse_extent(bx.xmin, bx.xmax, bx.ymin, bx.ymax, EXACT, true, true) : T(1);
        const T* plane = a.src + (p * a.F + f) * mplane + cl;
        auto load_row = [&](int row) {
            return *reinterpret_cast<const Quad<T>*>(plane + static_cast<int64_t>(workspace_row(a, row)) * mpitch);
        };

        // rows of the two runs; rt[r+1], rb[r] are the plain and rt[r], rb[r+1] the advanced rows
        // of output row i0 + r
        int rt[RB + 1], rb[RB + 1];
        Quad<T> Tq[RB + 1], Bq[RB + 1];
#pragma unroll
        for (int r = 0; r <= RB; ++r) {
            rt[r] = clampi(i0 + r + s.xlo - 1, 0, h);
            rb[r] = clampi(i0 + r + s.xhi, 0, h);
            Tq[r] = load_row(rt[r]);
            Bq[r] = load_row(rb[r]);
        }

        T off_b[4] = {T(0), T(0), T(0), T(0)};
        if (R > 0) {
            const int band_t = max(rt[0] - 1, 0) / R, band_b = max(rb[0] - 1, 0) / R;
            const int last_t = (band_t + 1) * R, last_b = (band_b + 1) * R;   // last row of each first band
            if (band_t != band_b) {
                double sum[4] = {0.0, 0.0, 0.0, 0.0};
                for (int b = min(band_t, band_b); b < max(band_t, band_b); ++b) {
                    const Quad<T> bottom = load_row(min(h, (b + 1) * R));
#pragma unroll
                    for (int v = 0; v < 4; ++v) sum[v] += static_cast<double>(bottom.v[v]);
                }
#pragma unroll
                for (int v = 0; v < 4; ++v) off_b[v] = static_cast<T>(band_b > band_t ? sum[v] : -sum[v]);
            }
            if (rt[RB] > last_t) {                   // the top run crosses into the next band
                const Quad<T> e = load_row(min(h, last_t));
#pragma unroll
                for (int r = 0; r <= RB; ++r) {
                    const T c = T(rt[r] > last_t);
#pragma unroll
                    for (int v = 0; v < 4; ++v) Tq[r].v[v] += c * e.v[v];
                }
            }
            if (rb[RB] > last_b) {
                const Quad<T> e = load_row(min(h, last_b));
#pragma unroll
                for (int r = 0; r <= RB; ++r) {
                    const T c = T(rb[r] > last_b);
#pragma unroll
                    for (int v = 0; v < 4; ++v) Bq[r].v[v] += c * e.v[v];
                }
            }
        }

#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                T val = blend<T, EXACT>(Tq[r].v[v], Tq[r + 1].v[v], Bq[r].v[v], Bq[r + 1].v[v], s.fxlo, s.fxhi);
                val += off_b[v];
                acc[r][v] += scale * val;
            }
    }

    if constexpr (FS > 1) {
        // partial sums of the sets 1..FS-1 go through LDS and are added by set 0 in set order
        T* part = reinterpret_cast<T*>(smem_raw);
        if (fgroup > 0) {
#pragma unroll
            for (int r = 0; r < RB; ++r)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    part[(((fgroup - 1) * RB + r) * 4 + v) * NTX + tid] = acc[r][v];
        }
        __syncthreads();
        if (fgroup > 0) return;
        for (int g = 1; g < FS; ++g)
#pragma unroll
            for (int r = 0; r < RB; ++r)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    acc[r][v] += part[(((g - 1) * RB + r) * 4 + v) * NTX + tid];
    }

    if (!lane_in) return;
    TO* out = reinterpret_cast<TO*>(a.dst) + p * static_cast<int64_t>(h) * w + c0;
    const bool wide_store = a.vec_out != 0 && c0 + 4 <= w;
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        const int i = i0 + r;
        if (i >= h) break;
        TO* orow = out + static_cast<int64_t>(i) * w;
        Quad<TO> q;
#pragma unroll
        for (int v = 0; v < 4; ++v) narrow(acc[r][v], q.v[v]);
        if (wide_store) {
            *reinterpret_cast<Quad<TO>*>(orow) = q;
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (c0 + v < w) orow[v] = q.v[v];
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Sum of 5 per-lane values over the workgroup; the totals are added to dst atomically or, when
// dst is a slot that only this workgroup writes, simply stored.
__device__ __forceinline__ void block_accumulate5(const double (&v)[5], double* __restrict__ dst,
                                                  double* __restrict__ lds /* [waves*5] */,
                                                  bool atomic = true) {
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
        if (atomic) unsafeAtomicAdd(dst + threadIdx.x, tot);
        else dst[threadIdx.x] = tot;
    }
}

// Streaming pass over grad_output. Work item = (plane p, filter f, band of R rows). Each row of
// grad_output is read from HBM once, placed in LDS, and used for both products of the backward
// pass:
//
// (PARAMS) the five sums per box that the parameter gradients need,
//   [0] sum g*dS/dxmin  [1] sum g*dS/dxmax  [2] sum g*dS/dymin  [3] sum g*dS/dymax  [4] sum g*S
// by transposed access: for X in {V, DT = I[t]-I[tAdv], DB = I[bAdv]-I[b]} (per-column values of
// the current output row, held in registers by the lane that owns column q),
//   sum_j g[j]*H(X)[j] = sum_{q=1..w} X[q]*W[q] + X[w]*tail,
//   W[q] = (gr - gl) + fyhi*(grA - gr) + fylo*(gl - glA),
//   gr = g[q-yhi], grA = g[q-yhi-1], gl = g[q-ylo], glA = g[q-ylo+1]   (0 outside [0,w)).
// W[w] as written counts some pixels whose box edge is clamped onto column w with the wrong
// weight; `tail` = sum_j g[j]*delta[j] fixes that with a per-column constant
//   delta[j] = (1-fyhi)[j > w-yhi] + fyhi[j > w-yhi-1] - (1-fylo)[j > w-ylo] - fylo[j > w-ylo+1].
// Likewise dS/dymax = sum_q V[q]*(grA - gr) + V[w]*g[w-yhi] and
//          dS/dymin = -sum_q V[q]*(gl - glA) - V[w]*g[w-ylo+1].
// Column 0 of the integral image is zero, so clamping at the left edge needs no correction.
//
// (SCAN) what the gradient w.r.t. the input needs from grad_output, the column workspace M:
//   A(i)[c] = sum_j g(i)[j] * (weight of input column c in the box of output pixel j)
//           = sum_{q > c} W[q] + tail            (the adjoint of the forward's column formula:
//             the input row enters through its prefix X[q] = sum_{c < q} x[c], so the weight of
//             x[c] is the sum of the W[q] of all prefixes that contain it; `tail` belongs to q = w),
//   M[i+1][c] = sum of A(i')[c] over the rows i' <= i of this band          (band-local running sum)
// with the same W[q] as above, so the four grad_output taps per column are shared with PARAMS.
// W(i), W(i+1) go to LDS as a row pair, are read back K consecutive columns per lane, and
// A = (sum of all W + tail) - (exclusive prefix of W) is a lane prefix, a DPP wave scan and the
// totals of the waves to the left. Bands do not depend on each other, so nothing has to be known
// about the rows above: the grad-input kernel adds the bottom rows of the bands above when it
// loads a row. A lane stores its K consecutive columns as one run into 16-byte aligned rows
// (pitch rounded up to 4 elements), so a wave writes 64*K contiguous elements per row.
// The boxes behind W are those of the parameter-gradient split; the reference's grad-input
// pass splits the mirrored box (src/box_convolution.cpp:51-67), whose whole-pixel part can
// differ when x_min - 1 rounds in T (it is then one pixel off with a border weight that makes up
// for it in exact mode only). A workgroup whose box is such a case computes a second set of
// weights for M from the mirrored split.
//
// LDS: [2 buffers][K*nt + 8] RowPair grad_output rows (4 zero pairs in front, >= 4 behind),
//      [2][2][4] X[w] triples, [K*nt] tail weights, [K*nt] RowPair W rows, [8*5] doubles,
//      [2][2][8] wave totals, [2][2][8] wave tails (one set per LDS buffer).
constexpr int kGPad = 4;

template <class T>
struct StreamLds {
    RowPair<T>* grow;   // [2][glen]
    RowPair<T>* wrow;   // [K*nt] W(i), W(i+1) by pixel column
    T* xw;              // [2][2][4]
    T* delta;           // [K*nt] tail weight of pixel column j
    double* red;        // [5 * kMaxRowWaves]
    T* wave_tot;        // [2 buffers][2 rows][kMaxRowWaves]
    T* wave_tail;       // [2 buffers][2 rows][kMaxRowWaves]
    int glen;
};

__host__ __device__ constexpr size_t stream_lds_elems(int K, int nt) {
    const size_t glen = static_cast<size_t>(K) * nt + 8;
    return 4 * glen + 2 * static_cast<size_t>(K) * nt + 16 + static_cast<size_t>(K) * nt;
}
__host__ __device__ constexpr size_t stream_lds_bytes(int K, int nt, size_t elem) {
    const size_t b = (stream_lds_elems(K, nt) * elem + 15) / 16 * 16;
    return b + (8 * kMaxRowWaves + 5 * kMaxRowWaves) * sizeof(double);
}

// `lds_base`: the kernel's own statically sized array, so that every LDS address is a lane
// offset plus a compile-time constant (a dynamically sized array has a link-time base that costs
// an addition per access).
template <class T>
__device__ __forceinline__ StreamLds<T> carve_stream_lds(unsigned char* lds_base, int K, int nt) {
    StreamLds<T> l;
    l.glen = K * nt + 8;
    l.grow = reinterpret_cast<RowPair<T>*>(lds_base);
    l.wrow = l.grow + 2 * l.glen;
    l.xw = reinterpret_cast<T*>(l.wrow + K * nt);
    l.delta = l.xw + 16;
    const size_t b = (stream_lds_elems(K, nt) * sizeof(T) + 15) / 16 * 16;
    l.red = reinterpret_cast<double*>(lds_base + b);
    l.wave_tot = reinterpret_cast<T*>(l.red + 5 * kMaxRowWaves);
    l.wave_tail = reinterpret_cast<T*>(l.red + 9 * kMaxRowWaves);
    return l;
}


// Register budget: with three or four columns per lane the kernel needs more registers than
// three waves per SIMD leave (170); told so, the compiler takes the 256 of two waves per SIMD
// instead of spilling.
// TG: element type of grad_output (T, or a 16-bit type when T is float: a.grad_out then points at
// elements of TG, widened to float as they are loaded).
// S > 1 (parameter sums only, rows wider than one workgroup's column slots): S workgroups share a
// band. Each owns NT*K of the row's columns q (its integral rows, its share of the five sums, a
// slot of its own for them) but places the WHOLE row pair of grad_output in LDS, since the taps
// of a column can fall anywhere in the row. The terms that belong to column w (the tails, the
// two single taps) are added by the workgroup that owns that column, over all pixel columns.
template <class T, class TG, int NT, int K, bool EXACT, bool FULL, bool PARAMS, bool SCAN, int S = 1>
__global__ void __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu((K >= 3 && PARAMS && SCAN) ? 2 : 1, (K >= 3 && PARAMS && SCAN) ? 2 : 8)))
grad_output_stream_kernel(SampleArgs<T> a) {
    static_assert(S == 1 || (S == 2 && PARAMS && !SCAN && !FULL), "column parts: parameter sums only, two parts");
    const unsigned vid = xcd_contiguous_id(a.per_xcd);
    if (vid >= a.total) return;                      // whole workgroup leaves together
    const unsigned nbands = a.nb, nfilt = a.F;
    const int part = S > 1 ? static_cast<int>(vid % S) : 0;
    const unsigned vband = S > 1 ? vid / S : vid;
    const int band = static_cast<int>(vband % nbands);
    const unsigned pf32 = vband / nbands;
    const int f = static_cast<int>(pf32 % nfilt);
    const int64_t pf = pf32, p = pf32 / nfilt;
    const int k_par = static_cast<int>(static_cast<unsigned>(a.plane0 + p) % static_cast<unsigned>(a.C)) * a.F + f;
    const int h = a.h, w = a.w, tid = threadIdx.x;
    constexpr int nt = NT;
    const unsigned row_bytes = static_cast<unsigned>(w) * sizeof(T);
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keep it scalar

    const BoxOfWorkgroup<T> bx = load_box(a.prm, k_par);
    const BoxSplit<T> s = split_grad_params(bx.xmin, bx.xmax, bx.ymin, bx.ymax);

    const int64_t pitch = w + 1;
    const int64_t mpitch = a.mpitch;
    // integral of the input; grad_output (one element early: column slot q = j + 1 is pixel j);
    // column workspace M of this (plane, filter)
    const LoadRows<T> irows(a.src + p * static_cast<int64_t>(h + 1) * pitch, pitch, w + 1, h + 1);
    const LoadRows<TG> grows(reinterpret_cast<const TG*>(a.grad_out) + pf * static_cast<int64_t>(h) * w - 1,
                             w, w + 1, h);
    T* mrows = SCAN ? a.dst + pf * static_cast<int64_t>(h + 1) * mpitch : nullptr;
    // The bands an XCD writes last (the final keep_tail bytes of its range) are stored with the
    // ordinary cache policy, everything before them non-temporally: see the store below.
    const unsigned from_end = static_cast<unsigned>(a.per_xcd) - 1u - vid % static_cast<unsigned>(a.per_xcd);
    const bool keep_in_cache =
        static_cast<uint64_t>(from_end) * a.R * mpitch * sizeof(T) < static_cast<uint64_t>(a.keep_tail);
    const Rows<T, FULL> mout(mrows, mpitch, static_cast<int>(mpitch), h + 1);
    __shared__ __align__(16) unsigned char lds_bytes[stream_lds_bytes(K, NT * S, sizeof(T))];
    const StreamLds<T> lds = carve_stream_lds<T>(lds_bytes, K, nt * S);
    const int glen = lds.glen;

    const int i0 = band * a.R;
    const int i1 = min(h, i0 + a.R);

    // The first two rows of grad_output are requested before anything else: they come from HBM
    // and need nothing but the workgroup's coordinates, so their latency runs alongside the
    // set-up below (LDS clearing, box parameters, column weights).
    // Column slots: a wave owns 64*K consecutive columns, lane l of wave v the pixel columns
    // jbase + 64*k, jbase = v*64*K + l (integral columns q = j + 1). Loads are lane-consecutive
    // dwords as with workgroup-wide slots, and the columns a lane owns in the second part of a row
    // pair (K consecutive ones, K*tid ..) belong to the same wave, so that the change of ownership
    // goes through LDS without a workgroup barrier.
    constexpr int CH = 64 * K;
    const int jbase = part * (NT * K) + wave * CH + lane;
    const int q1 = (1 + jbase) * static_cast<int>(sizeof(T));
    const int q1g = (1 + jbase) * static_cast<int>(sizeof(TG));     // the same slots in a row of TG
    // S > 1: the columns of the other part, which this workgroup only copies into LDS
    const int jother = (1 - part) * (NT * K) + wave * CH + lane;
    const int q1o = (1 + jother) * static_cast<int>(sizeof(T));
    const int q1og = (1 + jother) * static_cast<int>(sizeof(TG));
    const bool owns_w = part == S - 1;               // the part with the row's last column
    T g0[K], g1[K];
    T go0[K] = {}, go1[K] = {};
    auto load_g_at = [&](int i, int qg, T (&dst)[K]) {
        const RowRef r = grows.row(min(i, h - 1), i < i1);     // rows past the band read as zeros
#pragma unroll
        for (int k = 0; k < K; ++k) dst[k] = static_cast<T>(widen(load_slot<TG, 64, kCacheStream>(r, qg, k)));
    };
    auto load_g = [&](int i, T (&dst)[K]) { load_g_at(i, q1g, dst); };
    load_g(i0, g0);
    load_g(i0 + 1, g1);
    if (S > 1) {
        load_g_at(i0, q1og, go0);
        load_g_at(i0 + 1, q1og, go1);
    }

    // clear the grad_output rows once: pads and the columns beyond w stay zero for good; the
    // same for the W rows
    for (int e = tid; e < 2 * glen; e += nt) lds.grow[e] = RowPair<T>{T(0), T(0)};
    if (S > 1 && tid < 16) lds.xw[tid] = T(0);
    if (SCAN) {
        for (int e = tid; e < K * nt; e += nt) lds.wrow[e] = RowPair<T>{T(0), T(0)};
        if (band == 0)
            for (int c = tid; c < mpitch; c += nt) mrows[c] = T(0);            // row 0
    }
    __syncthreads();

    // tail weight of pixel column j for a box with these column offsets and border weights
    auto tail_weight = [&](int j, int ylo, int yhi, T fylo, T fyhi) {
        const T one = T(1);
        return (EXACT ? (one - fyhi) : one) * T(j > w - yhi)
             + (EXACT ? fyhi : T(0)) * T(j > w - yhi - 1)
             - (EXACT ? (one - fylo) : one) * T(j > w - ylo)
             - (EXACT ? fylo : T(0)) * T(j > w - ylo + 1);
    };
    // LDS byte offsets of the pairs (grA, gr) and (gl, glA) of column slot q
    auto tap_r = [&](int q, int yhi) {
        return static_cast<unsigned>(clampi(q - yhi - 1, -2, w) + kGPad) * static_cast<unsigned>(sizeof(RowPair<T>));
    };
    auto tap_l = [&](int q, int ylo) {
        return static_cast<unsigned>(clampi(q - ylo, -2, w) + kGPad) * static_cast<unsigned>(sizeof(RowPair<T>));
    };

    // lane-constant tap offsets; the tail weights of the lane's columns go to LDS (read back
    // once per row pair: cheaper than K live registers)
    unsigned ir[K], il[K];
    unsigned idx_ymax = 0, idx_ymin = 0;
    bool wave_has_tail = false;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const int j = jbase + 64 * k;
        ir[k] = tap_r(j + 1, s.yhi);
        il[k] = tap_l(j + 1, s.ylo);
        const T d = (FULL || j < w) ? tail_weight(j, s.ylo, s.yhi, s.fylo, s.fyhi) : T(0);
        lds.delta[j] = d;
        wave_has_tail = wave_has_tail || d != T(0);
        if (S > 1) {
            const int jo = jother + 64 * k;
            lds.delta[jo] = jo < w ? tail_weight(jo, s.ylo, s.yhi, s.fylo, s.fyhi) : T(0);
        }
    }
    if (PARAMS) {
        const int j_ymax = w - s.yhi, j_ymin = w - s.ylo + 1;
        idx_ymax = (j_ymax >= 0 && j_ymax < w) ? j_ymax + kGPad : 0;          // index 0 holds a zero
        idx_ymin = (j_ymin >= 0 && j_ymin < w) ? j_ymin + kGPad : 0;
    }
    // SCAN: the whole-pixel column offsets of the reference's mirrored split, turned back to the
    // orientation of W; they differ from s.ylo / s.yhi only when y_min - 1 rounds in T
    const BoxSplit<T> sm = split_grad_input(bx.xmin, bx.xmax, bx.ymin, bx.ymax);
    const int ylo_m = 1 - sm.yhi, yhi_m = 1 - sm.ylo;
    const bool own_w = SCAN && (ylo_m != s.ylo || yhi_m != s.yhi);               // workgroup-uniform
    wave_has_tail = __any(wave_has_tail) != 0 || own_w;                          // wave-uniform

    // The five sums are added up in T only within one row pair of one lane (2*K products each);
    // from there on in double. The products are large against the final sums (V grows along the
    // row like a running integral while the sums are differences of such terms), so longer T
    // chains would lose the low digits.
    double total[5] = {0.0, 0.0, 0.0, 0.0, 0.0};
    T colacc[K];                                      // SCAN: columns K*tid .. K*tid+K-1
#pragma unroll
    for (int k = 0; k < K; ++k) colacc[k] = T(0);

    T ta[K], bc[K], t0[K], t1[K], b1[K], b2[K];
    if (PARAMS) {
        load_row<T, 64, K>(irows.row(clampi(i0 + s.xlo - 1, 0, h)), q1, ta);
        load_row<T, 64, K>(irows.row(clampi(i0 + s.xhi, 0, h)), q1, bc);
        load_pair<T, 64, K, FULL>(irows, i0, s.xlo, s.xhi, h, q1, t0, t1, b1, b2);
    }

    // PREFETCH and the LDS buffer are compile-time tags (see forward_rows_kernel): the loop below
    // is unrolled over both buffers, so LDS addresses are lane constants plus immediates and the
    // sliding rows rotate by renaming instead of moves.
    // OWN_W: the rare box whose mirrored split differs (see above); a tag as well, so that the
    // common case carries none of its code.
    // Rows i, i+1 of grad_output (registers GA, GB) into LDS buffer FL, with the wave's share of
    // the tails and, from the owner of column w, the X[w] triples of the same pair. A macro, not
    // a lambda: arrays handed through a second closure end up in scratch memory.
#define BOXCONV_PUBLISH_PAIR(FL, GA, GB, GOA, GOB, TA, T0, T1, BC, B1, B2, TL0, TL1)                \
    {                                                                                               \
        RowPair<T>* Gp = lds.grow + ((FL) ? glen : 0);                                              \
        T* Xp0 = lds.xw + (FL) * 8;                                                                 \
        T* Xp1 = Xp0 + 4;                                                                           \
        TL0 = T(0); TL1 = T(0);                                                                     \
        _Pragma("unroll")                                                                           \
        for (int k = 0; k < K; ++k) {                                                               \
            if (slot_valid<T, 64, FULL>(q1, k, row_bytes))                                          \
                *at_bytes(Gp + kGPad - 1 + 64 * k, 2 * q1) = RowPair<T>{GA[k], GB[k]};              \
            if (S > 1 && slot_valid<T, 64, false>(q1o, k, row_bytes))                               \
                *at_bytes(Gp + kGPad - 1 + 64 * k, 2 * q1o) = RowPair<T>{GOA[k], GOB[k]};           \
            if (S == 1 || owns_w) {                                                                 \
                const T dlt = *at_bytes(lds.delta - 1 + 64 * k, q1);                                \
                TL0 += dlt * GA[k];                                                                 \
                TL1 += dlt * GB[k];                                                                 \
                if (S > 1) {                                                                        \
                    const T dlo = *at_bytes(lds.delta - 1 + 64 * k, q1o);                           \
                    TL0 += dlo * GOA[k];                                                            \
                    TL1 += dlo * GOB[k];                                                            \
                }                                                                                   \
            }                                                                                       \
            if (PARAMS && (FULL ? (k == K - 1 && tid == nt - 1) : (q1 + slot_bytes<T, 64>(k) == row_bytes))) { \
                const T dt0 = T0[k] - TA[k], db0 = B1[k] - BC[k];                                   \
                const T dt1 = T1[k] - T0[k], db1 = B2[k] - B1[k];                                   \
                T v0 = BC[k] - T0[k], v1 = B1[k] - T1[k];                                           \
                if (EXACT) {                                                                        \
                    v0 += s.fxhi * db0; v0 += s.fxlo * dt0;                                         \
                    v1 += s.fxhi * db1; v1 += s.fxlo * dt1;                                         \
                }                                                                                   \
                Xp0[0] = v0; Xp0[1] = dt0; Xp0[2] = db0;                                            \
                Xp1[0] = v1; Xp1[1] = dt1; Xp1[2] = db1;                                            \
            }                                                                                       \
        }                                                                                           \
    }

    // MERGED (workgroups of up to four waves): one workgroup barrier per row pair. The rows of the
    // NEXT pair go into the other LDS buffer before the barrier that publishes this pair's wave
    // totals, so the same barrier makes both visible. (The other buffer was last read for the
    // pair before this one, i.e. before the previous barrier.) The price: the next pair's loads
    // must have arrived by that barrier instead of by the end of the iteration; with eight waves
    // and one workgroup per CU that costs more than the barrier (1024 x 2048, 512 threads: 1.39
    // against 1.07 ms), so those keep a barrier of their own for the rows.
    // tl0, tl1: this wave's tails of the pair whose rows are in LDS.
    constexpr bool MERGED = NT <= 256;
    T tl0 = T(0), tl1 = T(0);
    if (MERGED) {
        BOXCONV_PUBLISH_PAIR(0, g0, g1, go0, go1, ta, t0, t1, bc, b1, b2, tl0, tl1)
        __syncthreads();
    }

    auto row_pair = [&](int i, auto prefetch_tag, auto flip_tag, auto own_w_tag) {
        constexpr bool PREFETCH = decltype(prefetch_tag)::value;
        constexpr int FLIP = decltype(flip_tag)::value;
        constexpr bool OWN_W = decltype(own_w_tag)::value;
        T n0[K] = {}, n1[K] = {}, n2[K] = {}, n3[K] = {}, m0[K] = {}, m1[K] = {};
        T mo0[K] = {}, mo1[K] = {};
        if (PREFETCH) {
            if (PARAMS)
                load_pair<T, 64, K, FULL>(irows, i + 2, s.xlo, s.xhi, h, q1, n0, n1, n2, n3);
            load_g(i + 2, m0);
            load_g(i + 3, m1);
            if (S > 1) {
                load_g_at(i + 2, q1og, mo0);
                load_g_at(i + 3, q1og, mo1);
            }
        }

        RowPair<T>* G = lds.grow + (FLIP ? glen : 0);
        T* X0 = lds.xw + FLIP * 8;
        T* X1 = X0 + 4;
        T* wtot = lds.wave_tot + FLIP * 2 * kMaxRowWaves;
        T* wtail = lds.wave_tail + FLIP * 2 * kMaxRowWaves;
        if (!MERGED) {
            BOXCONV_PUBLISH_PAIR(FLIP, g0, g1, go0, go1, ta, t0, t1, bc, b1, b2, tl0, tl1)
            __syncthreads();                                                 // rows are in LDS
        }
        T tail0 = tl0, tail1 = tl1;
        T tn0 = T(0), tn1 = T(0);                       // MERGED: tails of the next pair

        // W(i)[q], W(i+1)[q] of the lane's column slots
        T wq0[K], wq1[K];
        {
            T sum[5] = {T(0), T(0), T(0), T(0), T(0)};
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const RowPair<T>* R = at_bytes(G, ir[k]);
                const RowPair<T>* L = at_bytes(G, il[k]);
                const RowPair<T> grA = R[0], gr = R[1], gl = L[0], glA = L[1];
                const T dr0 = grA.r0 - gr.r0, dl0 = gl.r0 - glA.r0;
                const T dr1 = grA.r1 - gr.r1, dl1 = gl.r1 - glA.r1;
                wq0[k] = gr.r0 - gl.r0;
                wq1[k] = gr.r1 - gl.r1;
                if (EXACT) {
                    wq0[k] += s.fyhi * dr0; wq0[k] += s.fylo * dl0;
                    wq1[k] += s.fyhi * dr1; wq1[k] += s.fylo * dl1;
                }
                if (PARAMS) {
                    const T dt0 = t0[k] - ta[k], db0 = b1[k] - bc[k];
                    const T dt1 = t1[k] - t0[k], db1 = b2[k] - b1[k];
                    T v0 = bc[k] - t0[k], v1 = b1[k] - t1[k];
                    if (EXACT) {
                        v0 += s.fxhi * db0; v0 += s.fxlo * dt0;
                        v1 += s.fxhi * db1; v1 += s.fxlo * dt1;
                    }
                    sum[4] += v0 * wq0[k];
                    sum[1] += db0 * wq0[k];
                    sum[0] -= dt0 * wq0[k];
                    sum[3] += v0 * dr0;
                    sum[2] -= v0 * dl0;
                    sum[4] += v1 * wq1[k];
                    sum[1] += db1 * wq1[k];
                    sum[0] -= dt1 * wq1[k];
                    sum[3] += v1 * dr1;
                    sum[2] -= v1 * dl1;
                }
            }
            if (PARAMS) {
                const T vw0 = X0[0], dtw0 = X0[1], dbw0 = X0[2];
                const T vw1 = X1[0], dtw1 = X1[1], dbw1 = X1[2];
                sum[4] += vw0 * tail0 + vw1 * tail1;
                sum[1] += dbw0 * tail0 + dbw1 * tail1;
                sum[0] -= dtw0 * tail0 + dtw1 * tail1;
                if (tid == 0 && (S == 1 || owns_w)) {
                    const RowPair<T> gmax = G[idx_ymax], gmin = G[idx_ymin];
                    sum[3] += vw0 * gmax.r0 + vw1 * gmax.r1;
                    sum[2] -= vw0 * gmin.r0 + vw1 * gmin.r1;
                }
#pragma unroll
                for (int n = 0; n < 5; ++n) total[n] += static_cast<double>(sum[n]);
            }
        }

        if (SCAN) {
            if (OWN_W) {
                // rare: the mirrored split cuts the box at other whole pixels; weights and tails
                // of M from that split, tap offsets worked out on the spot
                tail0 = T(0); tail1 = T(0);
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    const int j = jbase + 64 * k;
                    const RowPair<T>* R = at_bytes(G, tap_r(j + 1, yhi_m));
                    const RowPair<T>* L = at_bytes(G, tap_l(j + 1, ylo_m));
                    const RowPair<T> grA = R[0], gr = R[1], gl = L[0], glA = L[1];
                    wq0[k] = gr.r0 - gl.r0;
                    wq1[k] = gr.r1 - gl.r1;
                    if (EXACT) {
                        wq0[k] += sm.fylo * (grA.r0 - gr.r0); wq0[k] += sm.fyhi * (gl.r0 - glA.r0);
                        wq1[k] += sm.fylo * (grA.r1 - gr.r1); wq1[k] += sm.fyhi * (gl.r1 - glA.r1);
                    }
                    const T dlt = (FULL || j < w) ? tail_weight(j, ylo_m, yhi_m, sm.fyhi, sm.fylo) : T(0);
                    tail0 += dlt * g0[k];
                    tail1 += dlt * g1[k];
                }
            }
            // W rows by pixel column c = q - 1, and the wave's share of the tails
#pragma unroll
            for (int k = 0; k < K; ++k)
                if (slot_valid<T, 64, FULL>(q1, k, row_bytes))
                    *at_bytes(lds.wrow - 1 + 64 * k, 2 * q1) = RowPair<T>{wq0[k], wq1[k]};
            T wt0 = T(0), wt1 = T(0);
            if (wave_has_tail) {
                wt0 = wave_sum_to_last(tail0);
                wt1 = wave_sum_to_last(tail1);
            }
            // The columns written above and the columns read below belong to this wave: LDS
            // serves a wave's accesses in order, so only the compiler has to be kept from moving
            // the reads up.
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

            // the lane's K consecutive columns K*tid .. K*tid+K-1: exclusive prefix of W inside
            // the lane, the lanes to the left by a wave scan
            T ex0[K], ex1[K];
            T base0, base1;
            {
                const RowPair<T>* r = lds.wrow + K * tid;
                T run0 = T(0), run1 = T(0);
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    const RowPair<T> wv = r[k];
                    ex0[k] = run0; run0 += wv.r0;
                    ex1[k] = run1; run1 += wv.r1;
                }
                const T inc0 = wave_inclusive_scan(run0);
                const T inc1 = wave_inclusive_scan(run1);
                base0 = run0 - inc0;                                         // -(lanes to the left)
                base1 = run1 - inc1;
                if (lane == 63) {
                    wtot[wave] = inc0; wtot[kMaxRowWaves + wave] = inc1;
                    wtail[wave] = wt0; wtail[kMaxRowWaves + wave] = wt1;
                }
            }
            if (MERGED && PREFETCH) BOXCONV_PUBLISH_PAIR(FLIP ^ 1, m0, m1, mo0, mo1, t1, n0, n1, b2, n2, n3, tn0, tn1)
            __syncthreads();                         // wave totals (and the next pair's rows) visible
            {
                // A[c] = (sum of all W + tail) - (W of the columns before c)
                //      = totals of this wave and the waves to the right + all tails - lanes to
                //        the left - columns to the left inside the lane.
                // `wave` is scalar, so the conditions below are scalar.
#pragma unroll
                for (int wv = 0; wv < NT / 64; ++wv) {
                    base0 += wtail[wv];
                    base1 += wtail[kMaxRowWaves + wv];
                    if (wv >= wave) {
                        base0 += wtot[wv];
                        base1 += wtot[kMaxRowWaves + wv];
                    }
                }
                // M rows i+1, i+2: a wave stores one contiguous run of 64*K elements per row. The
                // grad-input kernel starts with the planes written last and finds them still in
                // the memory-side cache if they were stored with the ordinary policy; the rest
                // is stored non-temporally so that it does not push the integral plane of the
                // input, which all filters of a plane re-read, out of the L2.
                const bool second = i + 1 < i1;
                const RowRef ob0 = mout.row(workspace_row(a, i + 1));
                const RowRef ob1 = mout.row(workspace_row(a, min(i + 2, h)), second);
                T out0[K];
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    out0[k] = colacc[k] + (base0 - ex0[k]);
                    colacc[k] = out0[k] + (base1 - ex1[k]);
                }
                const int first = K * tid * static_cast<int>(sizeof(T));
                const int limit = static_cast<int>(mpitch * sizeof(T));
                if (keep_in_cache) {
                    buffer_store_run<kCacheDefault, FULL>(out0, ob0, first, limit);
                    buffer_store_run<kCacheDefault, FULL>(colacc, ob1, first, limit);
                } else {
                    buffer_store_run<kCacheStream, FULL>(out0, ob0, first, limit);
                    buffer_store_run<kCacheStream, FULL>(colacc, ob1, first, limit);
                }
            }
        }

        if (!SCAN && MERGED) {
            if (PREFETCH) BOXCONV_PUBLISH_PAIR(FLIP ^ 1, m0, m1, mo0, mo1, t1, n0, n1, b2, n2, n3, tn0, tn1)
            __syncthreads();                                                 // the next pair's rows visible
        }

        if (PREFETCH) {
            if (MERGED) { tl0 = tn0; tl1 = tn1; }
#pragma unroll
            for (int k = 0; k < K; ++k) {
                if (PARAMS) {
                    ta[k] = t1[k]; bc[k] = b2[k];
                    t0[k] = n0[k]; t1[k] = n1[k]; b1[k] = n2[k]; b2[k] = n3[k];
                }
                g0[k] = m0[k]; g1[k] = m1[k];
                if (S > 1) { go0[k] = mo0[k]; go1[k] = mo1[k]; }
            }
        }
        // keep the two unrolled pairs apart: loads of the pair after next hoisted up here would
        // only add live registers
        __builtin_amdgcn_sched_barrier(0);
    };
    // (written out twice rather than through another lambda: arrays captured through two levels
    // of closures end up in scratch memory)
    // double: one loop body serves every pair of pairs, also a band's last two (the second then
    // prefetches rows that nothing uses: clamped integral rows, and rows of grad_output past the
    // band, which read as zeros). With the band's end written out as a third and a fourth copy of
    // the pair body, as for the other types, the copy for "two pairs left" returned wrong
    // parameter sums for double rows of 1537 to 2047 columns in rounded mode (the kernel spills
    // some 500 registers at that size); the loop body itself never did.
#define BOXCONV_ALL_PAIRS(OWN_W_TAG)                                         \
    if constexpr (sizeof(T) == 8) {                                          \
        int i = i0;                                                          \
        for (; i + 2 < i1; i += 4) {                                         \
            row_pair(i, std::true_type{}, Flip0{}, OWN_W_TAG{});             \
            row_pair(i + 2, std::true_type{}, Flip1{}, OWN_W_TAG{});         \
        }                                                                    \
        if (i < i1) row_pair(i, std::false_type{}, Flip0{}, OWN_W_TAG{});    \
    } else {                                                                 \
        int i = i0;                                                          \
        for (; i + 4 < i1; i += 4) {                                         \
            row_pair(i, std::true_type{}, Flip0{}, OWN_W_TAG{});             \
            row_pair(i + 2, std::true_type{}, Flip1{}, OWN_W_TAG{});         \
        }                                                                    \
        if (i + 2 < i1) {                                                    \
            row_pair(i, std::true_type{}, Flip0{}, OWN_W_TAG{});             \
            row_pair(i + 2, std::false_type{}, Flip1{}, OWN_W_TAG{});        \
        } else {                                                             \
            row_pair(i, std::false_type{}, Flip0{}, OWN_W_TAG{});            \
        }                                                                    \
    }
    if (own_w) BOXCONV_ALL_PAIRS(std::true_type)
    else BOXCONV_ALL_PAIRS(std::false_type)
#undef BOXCONV_ALL_PAIRS
#undef BOXCONV_PUBLISH_PAIR

    if (PARAMS) {
        __syncthreads();
        // slots > 0: one slot per workgroup, summed by the finalize kernel in a fixed order
        // (no clearing pass, no atomics, bit-reproducible); else atomics into the box's five sums
        if (a.acc_slots > 0)
            block_accumulate5(total, a.acc + ((static_cast<int64_t>(a.plane0 + p) * a.F + f) * a.acc_slots + band * S + part) * 5,
                              lds.red, false);
        else
            block_accumulate5(total, a.acc + static_cast<int64_t>(k_par) * 5, lds.red);
    }
}

// ---------------------------------------------------------------------------------------------
// The same pass for float rows of a multiple of four columns (w <= 4 * NT; FULL: w == 4 * NT), both
// products at once: a lane owns 4 CONSECUTIVE columns for everything, where
// grad_output_stream_kernel gives it the columns lane, lane + 64, ... of its wave and moves the
// weights W through LDS to get consecutive ones for the suffix sum. With consecutive columns
//   * the taps of a lane's 4 columns are two runs of 5 adjacent row pairs in LDS (3 instructions
//     each) instead of 16 separate pairs,
//   * W is where the suffix sum needs it: no LDS round trip, no wave barrier in the middle of a
//     row pair,
//   * the integral rows and grad_output come as one 16-byte load per lane and row (the integral
//     rows start at an odd element, so theirs are only dword-aligned, which global loads allow),
//   * wave totals and tails travel as one 16-byte word per wave.
// Same arithmetic, same order of additions inside a lane's row pair; the sums differ from the
// other kernel's only in which columns share a lane. Everything said there about the math, the
// two splits, the single barrier per row pair (MERGED) and the cache policy of the stores applies.
// !FULL: the lanes past the row's end (whole lanes, since w is a multiple of four) load from the
// row's first columns and drop what they loaded where it would be used: they put zeros into LDS
// (the row's right-hand padding), hold zero weights and a zero V, and store nothing.
typedef float f4_dword_aligned __attribute__((ext_vector_type(4), aligned(4)));
__device__ __forceinline__ void load4_dword_aligned(const float* p, float (&v)[4]) {
    const f4_dword_aligned q = *reinterpret_cast<const f4_dword_aligned*>(p);
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
}

// Two waves per SIMD on purpose, although the registers would allow three: with three, more
// workgroups are resident per XCD than share one integral plane of the input, two planes compete
// for its L2, and the kernel gets slower (226 against 217 us at 512 x 1024).
// (Workgroups of three, five and six waves may run three waves per SIMD: four or two of them then
// share a CU, where at two per SIMD two, three or two of its eight wave slots would stay empty.
// Measured at three waves: 480 x 640 170 -> 149 us; rows of 960 and 1000 columns, four waves with
// idle lanes, got slower with three per SIMD like the full rows: 230 -> 235 us.)
// SCAN = false: the parameter sums only (the input needs no gradient, as in a network's first
// layer): no suffix sums, no column workspace, half the registers; four waves per SIMD then (no
// column workspace competes for the L2).
template <class TG, int NT, bool EXACT, bool FULL, bool SCAN = true>
__global__ void __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(2, !SCAN ? 4 : (NT == 192 || NT == 320 || NT == 384) ? 3 : 2)))
grad_output_stream_consec_kernel(SampleArgs<float> a) {
    using T = float;
    constexpr int K = 4;
    constexpr int kPad = 8;                          // zero pairs in front of and behind a row in LDS
    constexpr int GLEN = K * NT + 2 * kPad;
    constexpr int WAVES = NT / 64;
    constexpr bool MERGED = NT <= 256;
    struct alignas(16) WaveSums { T tot0, tot1, tail0, tail1; };
    struct alignas(16) LastColumn { T v, dt, db, unused; };      // V, DT, DB at column w
    __shared__ __align__(16) RowPair<T> grow[2][GLEN];
    __shared__ __align__(16) T delta[K * NT];
    __shared__ WaveSums wsum[2][WAVES];
    __shared__ LastColumn xw[2][2];
    __shared__ double red[5 * WAVES];

    const unsigned vid = xcd_contiguous_id(a.per_xcd);
    if (vid >= a.total) return;                      // whole workgroup leaves together
    const unsigned nbands = a.nb, nfilt = a.F;
    const int band = static_cast<int>(vid % nbands);
    const unsigned pf32 = vid / nbands;
    const int f = static_cast<int>(pf32 % nfilt);
    const int64_t pf = pf32, p = pf32 / nfilt;
    const int k_par = static_cast<int>(static_cast<unsigned>(a.plane0 + p) % static_cast<unsigned>(a.C)) * a.F + f;
    const int h = a.h, w = a.w, tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c0 = K * tid;                          // the lane's first pixel column
    const bool lane_in = FULL || c0 < w;             // (w is a multiple of K: a lane is in or out as a whole)
    const int cl = lane_in ? c0 : 0;                 // idle lanes load the row's first columns
    const int owner = FULL ? NT - 1 : w / K - 1;     // the lane whose last column is column w

    const BoxOfWorkgroup<T> bx = load_box(a.prm, k_par);
    const BoxSplit<T> s = split_grad_params(bx.xmin, bx.xmax, bx.ymin, bx.ymax);
    const BoxSplit<T> sm = split_grad_input(bx.xmin, bx.xmax, bx.ymin, bx.ymax);
    const int ylo_m = 1 - sm.yhi, yhi_m = 1 - sm.ylo;
    const bool own_w = ylo_m != s.ylo || yhi_m != s.yhi;                        // workgroup-uniform

    const int64_t pitch = w + 1;
    const int64_t mpitch = a.mpitch;
    const T* iplane = a.src + p * static_cast<int64_t>(h + 1) * pitch;        // integral of the input
    const TG* gplane = reinterpret_cast<const TG*>(a.grad_out) + pf * static_cast<int64_t>(h) * w;
    T* mrows = a.dst + pf * static_cast<int64_t>(h + 1) * mpitch;
    const unsigned from_end = static_cast<unsigned>(a.per_xcd) - 1u - vid % static_cast<unsigned>(a.per_xcd);
    const bool keep_in_cache =
        static_cast<uint64_t>(from_end) * a.R * mpitch * sizeof(T) < static_cast<uint64_t>(a.keep_tail);
    const Rows<T, true> mout(mrows, mpitch, static_cast<int>(mpitch), h + 1);

    const int i0 = band * a.R;
    const int i1 = min(h, i0 + a.R);

    // integral row r, columns c0+1 .. c0+4; rows of grad_output, columns c0 .. c0+3 (a row past the
    // band is read from a valid address and cleared afterwards)
    // (what an idle lane loads is discarded where it would be used, not here: a select right
    // behind a load makes the lane wait for it at once)
    auto load_i = [&](int r, T (&dst)[K]) {
        load4_dword_aligned(iplane + static_cast<int64_t>(r) * pitch + 1 + cl, dst);
    };
    auto load_g = [&](int i, T (&dst)[K]) {
        load_quad(gplane + static_cast<int64_t>(min(i, h - 1)) * w + cl, dst);
    };
    auto load_window = [&](int i, T (&t0)[K], T (&t1)[K], T (&b1)[K], T (&b2)[K]) {
        load_i(clampi(i + s.xlo, 0, h), t0);
        load_i(clampi(i + 1 + s.xlo, 0, h), t1);
        load_i(clampi(i + 1 + s.xhi, 0, h), b1);
        load_i(clampi(i + 2 + s.xhi, 0, h), b2);
    };

    T g0[K], g1[K];
    load_g(i0, g0);
    load_g(i0 + 1, g1);

    // pads of both LDS rows, row 0 of the column workspace
    if (tid < 2 * kPad) {
        const int e = tid < kPad ? tid : K * NT + tid;
        grow[0][e] = RowPair<T>{T(0), T(0)};
        grow[1][e] = RowPair<T>{T(0), T(0)};
    }
    if (SCAN && band == 0)
        for (int c = tid; c < mpitch; c += NT) mrows[c] = T(0);

    auto tail_weight = [&](int j, int ylo, int yhi, T fylo, T fyhi) {
        const T one = T(1);
        return (EXACT ? (one - fyhi) : one) * T(j > w - yhi)
             + (EXACT ? fyhi : T(0)) * T(j > w - yhi - 1)
             - (EXACT ? (one - fylo) : one) * T(j > w - ylo)
             - (EXACT ? fylo : T(0)) * T(j > w - ylo + 1);
    };
    // first element (with the front pad counted in) of the runs of 5 row pairs that hold the taps
    // of the lane's columns: right run g[c0 - yhi ..], left run g[c0 + 1 - ylo ..]
    auto run_start = [&](int first) { return clampi(first, -kPad, w) + kPad; };
    const int er = run_start(c0 - s.yhi), el = run_start(c0 + 1 - s.ylo);
    const int er_m = run_start(c0 - yhi_m), el_m = run_start(c0 + 1 - ylo_m);
    bool wave_has_tail = false;
    {
        T d[K];
#pragma unroll
        for (int k = 0; k < K; ++k) {
            d[k] = lane_in ? tail_weight(c0 + k, s.ylo, s.yhi, s.fylo, s.fyhi) : T(0);
            wave_has_tail = wave_has_tail || d[k] != T(0);
        }
        *reinterpret_cast<Quad<T>*>(&delta[c0]) = Quad<T>{{d[0], d[1], d[2], d[3]}};
    }
    wave_has_tail = __any(wave_has_tail) != 0 || own_w;                          // wave-uniform
    const int j_ymax = w - s.yhi, j_ymin = w - s.ylo + 1;
    const int idx_ymax = (j_ymax >= 0 && j_ymax < w) ? j_ymax + kPad : 0;        // element 0 is a zero pad
    const int idx_ymin = (j_ymin >= 0 && j_ymin < w) ? j_ymin + kPad : 0;

    double total[5] = {0.0, 0.0, 0.0, 0.0, 0.0};
    T colacc[K];
#pragma unroll
    for (int k = 0; k < K; ++k) colacc[k] = T(0);

    T ta[K], bc[K], t0[K], t1[K], b1[K], b2[K];
    load_i(clampi(i0 + s.xlo - 1, 0, h), ta);
    load_i(clampi(i0 + s.xhi, 0, h), bc);
    load_window(i0, t0, t1, b1, b2);
    __syncthreads();                                 // pads and tail weights are in place

    // Rows i, i+1 of grad_output (GA, GB) into LDS buffer FL, the lane's share of their tails, and,
    // from the lane that owns column w, V, DT, DB of that column for both rows.
#define BOXCONV_PUBLISH_CONSEC(FL, I, GA, GB, TA, T0, T1, BC, B1, B2, TL0, TL1)                      \
    {                                                                                               \
        if ((I) + 1 >= i1) {                                                                        \
            _Pragma("unroll")                                                                       \
            for (int k = 0; k < K; ++k) GB[k] = T(0);                                               \
        }                                                                                           \
        if (!FULL && !lane_in) {                                                                    \
            _Pragma("unroll")                                                                       \
            for (int k = 0; k < K; ++k) { GA[k] = T(0); GB[k] = T(0); }                             \
        }                                                                                           \
        Quad<T>* dst = reinterpret_cast<Quad<T>*>(&grow[FL][kPad + c0]);                            \
        dst[0] = Quad<T>{{GA[0], GB[0], GA[1], GB[1]}};                                             \
        dst[1] = Quad<T>{{GA[2], GB[2], GA[3], GB[3]}};                                             \
        TL0 = T(0); TL1 = T(0);                                                                     \
        if (wave_has_tail) {                                                                        \
            const Quad<T> dq = *reinterpret_cast<const Quad<T>*>(&delta[c0]);                       \
            _Pragma("unroll")                                                                       \
            for (int k = 0; k < K; ++k) { TL0 += dq.v[k] * GA[k]; TL1 += dq.v[k] * GB[k]; }         \
        }                                                                                           \
        if (tid == owner) {                                                                         \
            const T dt0 = T0[K - 1] - TA[K - 1], db0 = B1[K - 1] - BC[K - 1];                       \
            const T dt1 = T1[K - 1] - T0[K - 1], db1 = B2[K - 1] - B1[K - 1];                       \
            T v0 = BC[K - 1] - T0[K - 1], v1 = B1[K - 1] - T1[K - 1];                               \
            if (EXACT) {                                                                            \
                v0 += s.fxhi * db0; v0 += s.fxlo * dt0;                                             \
                v1 += s.fxhi * db1; v1 += s.fxlo * dt1;                                             \
            }                                                                                       \
            xw[FL][0] = LastColumn{v0, dt0, db0, T(0)};                                             \
            xw[FL][1] = LastColumn{v1, dt1, db1, T(0)};                                             \
        }                                                                                           \
    }

    T tl0 = T(0), tl1 = T(0);
    if (MERGED) {
        BOXCONV_PUBLISH_CONSEC(0, i0, g0, g1, ta, t0, t1, bc, b1, b2, tl0, tl1)
        __syncthreads();
    }

    auto row_pair = [&](int i, auto prefetch_tag, auto flip_tag, auto own_w_tag) {
        constexpr bool PREFETCH = decltype(prefetch_tag)::value;
        constexpr int FLIP = decltype(flip_tag)::value;
        constexpr bool OWN_W = decltype(own_w_tag)::value;
        T n0[K] = {}, n1[K] = {}, n2[K] = {}, n3[K] = {}, m0[K] = {}, m1[K] = {};
        if (PREFETCH) {
            load_window(i + 2, n0, n1, n2, n3);
            load_g(i + 2, m0);
            load_g(i + 3, m1);
        }
        if (!MERGED) {
            BOXCONV_PUBLISH_CONSEC(FLIP, i, g0, g1, ta, t0, t1, bc, b1, b2, tl0, tl1)
            __syncthreads();                                                 // rows are in LDS
        }
        const RowPair<T>* G = grow[FLIP];
        T tail0 = tl0, tail1 = tl1;
        T tn0 = T(0), tn1 = T(0);

        // W(i)[q], W(i+1)[q] of the lane's columns, and the five sums
        T wq0[K], wq1[K];
        {
            RowPair<T> R[K + 1], L[K + 1];
#pragma unroll
            for (int m = 0; m <= K; ++m) { R[m] = G[er + m]; L[m] = G[el + m]; }
            T sum[5] = {T(0), T(0), T(0), T(0), T(0)};
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const RowPair<T> grA = R[k], gr = R[k + 1], gl = L[k], glA = L[k + 1];
                const T dr0 = grA.r0 - gr.r0, dl0 = gl.r0 - glA.r0;
                const T dr1 = grA.r1 - gr.r1, dl1 = gl.r1 - glA.r1;
                wq0[k] = gr.r0 - gl.r0;
                wq1[k] = gr.r1 - gl.r1;
                if (EXACT) {
                    wq0[k] += s.fyhi * dr0; wq0[k] += s.fylo * dl0;
                    wq1[k] += s.fyhi * dr1; wq1[k] += s.fylo * dl1;
                }
                if (!FULL && !lane_in) { wq0[k] = T(0); wq1[k] = T(0); }    // (no column q > w)
                const T dt0 = t0[k] - ta[k], db0 = b1[k] - bc[k];
                const T dt1 = t1[k] - t0[k], db1 = b2[k] - b1[k];
                T v0 = bc[k] - t0[k], v1 = b1[k] - t1[k];
                if (EXACT) {
                    v0 += s.fxhi * db0; v0 += s.fxlo * dt0;
                    v1 += s.fxhi * db1; v1 += s.fxlo * dt1;
                }
                // (an idle lane: its weights are zero, which takes care of the products with dt and
                // db; its V must go as well, since the taps of its columns are not zero)
                if (!FULL && !lane_in) { v0 = T(0); v1 = T(0); }
                sum[4] += v0 * wq0[k];
                sum[1] += db0 * wq0[k];
                sum[0] -= dt0 * wq0[k];
                sum[3] += v0 * dr0;
                sum[2] -= v0 * dl0;
                sum[4] += v1 * wq1[k];
                sum[1] += db1 * wq1[k];
                sum[0] -= dt1 * wq1[k];
                sum[3] += v1 * dr1;
                sum[2] -= v1 * dl1;
            }
            if (wave_has_tail || wave == 0) {
                const LastColumn x0 = xw[FLIP][0], x1 = xw[FLIP][1];
                sum[4] += x0.v * tail0 + x1.v * tail1;
                sum[1] += x0.db * tail0 + x1.db * tail1;
                sum[0] -= x0.dt * tail0 + x1.dt * tail1;
                if (tid == 0) {
                    const RowPair<T> gmax = G[idx_ymax], gmin = G[idx_ymin];
                    sum[3] += x0.v * gmax.r0 + x1.v * gmax.r1;
                    sum[2] -= x0.v * gmin.r0 + x1.v * gmin.r1;
                }
            }
#pragma unroll
            for (int n = 0; n < 5; ++n) total[n] += static_cast<double>(sum[n]);
        }

        if (SCAN && OWN_W) {
            // rare: the mirrored split cuts the box at other whole pixels; weights and tails of
            // the column workspace from that split
            RowPair<T> R[K + 1], L[K + 1];
#pragma unroll
            for (int m = 0; m <= K; ++m) { R[m] = G[er_m + m]; L[m] = G[el_m + m]; }
            tail0 = T(0); tail1 = T(0);
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const RowPair<T> grA = R[k], gr = R[k + 1], gl = L[k], glA = L[k + 1];
                wq0[k] = gr.r0 - gl.r0;
                wq1[k] = gr.r1 - gl.r1;
                if (EXACT) {
                    wq0[k] += sm.fylo * (grA.r0 - gr.r0); wq0[k] += sm.fyhi * (gl.r0 - glA.r0);
                    wq1[k] += sm.fylo * (grA.r1 - gr.r1); wq1[k] += sm.fyhi * (gl.r1 - glA.r1);
                }
                if (!FULL && !lane_in) { wq0[k] = T(0); wq1[k] = T(0); }
                const T dlt = lane_in ? tail_weight(c0 + k, ylo_m, yhi_m, sm.fyhi, sm.fylo) : T(0);
                const RowPair<T> own = G[kPad + c0 + k];
                tail0 += dlt * own.r0;
                tail1 += dlt * own.r1;
            }
        }

        // A[c] = (sum of all W + tail) - (W of the columns before c): exclusive prefix inside the
        // lane, the lanes to the left by a wave scan, the other waves through LDS
        T ex0[K] = {}, ex1[K] = {};
        T base0 = T(0), base1 = T(0);
        if (SCAN) {
            T run0 = T(0), run1 = T(0);
#pragma unroll
            for (int k = 0; k < K; ++k) {
                ex0[k] = run0; run0 += wq0[k];
                ex1[k] = run1; run1 += wq1[k];
            }
            const T inc0 = wave_inclusive_scan(run0);
            const T inc1 = wave_inclusive_scan(run1);
            base0 = run0 - inc0;                                             // -(lanes to the left)
            base1 = run1 - inc1;
            T wt0 = T(0), wt1 = T(0);
            if (wave_has_tail) {
                wt0 = wave_sum_to_last(tail0);
                wt1 = wave_sum_to_last(tail1);
            }
            if (lane == 63) wsum[FLIP][wave] = WaveSums{inc0, inc1, wt0, wt1};
        }
        if (MERGED && PREFETCH) BOXCONV_PUBLISH_CONSEC(FLIP ^ 1, i + 2, m0, m1, t1, n0, n1, b2, n2, n3, tn0, tn1)
        __syncthreads();                             // wave totals (and the next pair's rows) visible
        if (SCAN) {
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) {
                const WaveSums ws = wsum[FLIP][wv];
                base0 += ws.tail0;
                base1 += ws.tail1;
                if (wv >= wave) {                    // `wave` is scalar
                    base0 += ws.tot0;
                    base1 += ws.tot1;
                }
            }
            const bool second = i + 1 < i1;
            const RowRef ob0 = mout.row(workspace_row(a, i + 1));
            const RowRef ob1 = mout.row(workspace_row(a, min(i + 2, h)), second);
            T out0[K];
#pragma unroll
            for (int k = 0; k < K; ++k) {
                out0[k] = colacc[k] + (base0 - ex0[k]);
                colacc[k] = out0[k] + (base1 - ex1[k]);
            }
            const int first = c0 * static_cast<int>(sizeof(T));
            const int limit = static_cast<int>(mpitch * sizeof(T));
            // (the rows are addressed by offset into one descriptor for the plane: a lane past the
            // row's end must not store at all)
            if (FULL || lane_in) {
                if (keep_in_cache) {
                    buffer_store_run<kCacheDefault, true>(out0, ob0, first, limit);
                    buffer_store_run<kCacheDefault, true>(colacc, ob1, first, limit);
                } else {
                    buffer_store_run<kCacheStream, true>(out0, ob0, first, limit);
                    buffer_store_run<kCacheStream, true>(colacc, ob1, first, limit);
                }
            }
        }
        if (PREFETCH) {
            if (MERGED) { tl0 = tn0; tl1 = tn1; }
#pragma unroll
            for (int k = 0; k < K; ++k) {
                ta[k] = t1[k]; bc[k] = b2[k];
                t0[k] = n0[k]; t1[k] = n1[k]; b1[k] = n2[k]; b2[k] = n3[k];
                g0[k] = m0[k]; g1[k] = m1[k];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };
#define BOXCONV_ALL_PAIRS(OWN_W_TAG)                                         \
    {                                                                        \
        int i = i0;                                                          \
        for (; i + 4 < i1; i += 4) {                                         \
            row_pair(i, std::true_type{}, Flip0{}, OWN_W_TAG{});             \
            row_pair(i + 2, std::true_type{}, Flip1{}, OWN_W_TAG{});         \
        }                                                                    \
        if (i + 2 < i1) {                                                    \
            row_pair(i, std::true_type{}, Flip0{}, OWN_W_TAG{});             \
            row_pair(i + 2, std::false_type{}, Flip1{}, OWN_W_TAG{});        \
        } else {                                                             \
            row_pair(i, std::false_type{}, Flip0{}, OWN_W_TAG{});            \
        }                                                                    \
    }
    if (SCAN && own_w) BOXCONV_ALL_PAIRS(std::true_type)
    else BOXCONV_ALL_PAIRS(std::false_type)
#undef BOXCONV_ALL_PAIRS
#undef BOXCONV_PUBLISH_CONSEC

    __syncthreads();
    block_accumulate5(total, a.acc + ((static_cast<int64_t>(a.plane0 + p) * a.F + f) * a.acc_slots + band) * 5,
                      red, false);
}

// ---------------------------------------------------------------------------------------------
// Gather kernels (helpers in box_sampling_common.hpp): one thread per output pixel.

template <class T, bool EXACT>
__global__ void __launch_bounds__(256) grad_input_gather_kernel(SampleArgs<T> a) {
    const int64_t hw = static_cast<int64_t>(a.h) * a.w;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= a.total) return;
    const int64_t p = idx / hw;
    const int pix = static_cast<int>(idx % hw);
    const int i = pix / a.w, j = pix % a.w;
    const int c_in = static_cast<int>(static_cast<unsigned>(a.plane0 + p) % static_cast<unsigned>(a.C));
    const int64_t ipl = static_cast<int64_t>(a.h + 1) * (a.w + 1);
    T acc = T(0);
    for (int f = 0; f < a.F; ++f) {
        const BoxOfWorkgroup<T> bx = load_box(a.prm, c_in * a.F + f);
        const BoxSplit<T> s = split_grad_input(bx.xmin, bx.xmax, bx.ymin, bx.ymax);
        const T scale = a.normalize
            ? inverse_extent(bx.xmin, bx.xmax, bx.ymin, bx.ymax, EXACT, true, true) : T(1);
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
    const int k_par = static_cast<int>(static_cast<unsigned>(a.plane0 + p) % static_cast<unsigned>(a.C)) * a.F + static_cast<int>(pf % a.F);
    double v[5] = {0, 0, 0, 0, 0};
    if (pix < h * w) {
        const int i = pix / w, j = pix % w;
        const BoxOfWorkgroup<T> bx = load_box(a.prm, k_par);
        const BoxSplit<T> s = split_grad_params(bx.xmin, bx.xmax, bx.ymin, bx.ymax);
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



}  // namespace


template <class T>
FinalizeArgs<T> finalize_args(const ParamFinish<T>& f) {
    FinalizeArgs<T> fa{};
    fa.acc = f.acc; fa.batch = f.batch; fa.slots = f.acc_slots;
    for (int i = 0; i < 4; ++i) fa.g[i] = f.grad[i];
    fa.n = f.n_boxes; fa.reparam_h = f.reparam_h; fa.reparam_w = f.reparam_w;
    fa.normalize = f.normalize ? 1 : 0; fa.exact = f.exact ? 1 : 0;
    fa.integ = f.integ; fa.grad_out = f.grad_out; fa.grad_dtype = f.grad_dtype; fa.h = f.h; fa.w = f.w;
    fa.F = f.num_filters;
    return fa;
}

// BOXCONV_GI_SPLIT_FILTERS=0: every workgroup of the grad-input kernel walks through all
// filters itself (for comparison).
inline bool split_filters_enabled() { return switches().gi_split_filters; }

// Shape of the grad-input launch for an image of h x w with F filters per plane: 2^lq lanes
// (4 columns each) side by side, rb output rows per lane, fs sets of threads sharing the filters.
struct ColsConfig { int lq, rb, fs; };
inline ColsConfig cols_config(int64_t planes, int F, int h, int w, bool allow_split) {
    ColsConfig c;
    const int quads = (w + 3) / 4;
    c.lq = 3;
    while (c.lq < 8 && (1 << c.lq) < quads) ++c.lq;          // 8 .. 256 lanes per row group
    // Rows wider than one strip: the strip width (one, two or four waves) that leaves the fewest
    // lanes idle; the kernel is local to a column, so narrower strips cost nothing else
    // (720 x 1280, 16 x 8 planes: two strips of 1024 columns 144 us, five of 256 columns 112 us).
    if (quads > 256) {
        auto lanes_launched = [&](int lq) { return ((quads + (1 << lq) - 1) >> lq) << lq; };
        for (int lq = 7; lq >= 6; --lq)
            if (lanes_launched(lq) < lanes_launched(c.lq)) c.lq = lq;
    }
    c.rb = 8;
    c.fs = 1;
    // Small problems: more, shorter-lived waves (2 rows per lane), and the filters of a plane
    // spread over several sets of threads. "Small": fewer waves than the chip holds at once.
    auto waves = [&](int rb) {
        const int ntx = std::max(64, 1 << c.lq), rg = ntx >> c.lq;
        const int64_t strips = (w + (4 << c.lq) - 1) / (4 << c.lq);
        return planes * ((h + rb * rg - 1) / (rb * rg)) * strips * (ntx / 64);
    };
    if (waves(8) < 2048) c.rb = 2;
    if (allow_split && F >= 4 && c.rb == 2 && waves(c.rb) <= 4096 && c.lq <= 6) {
        c.fs = F >= 16 ? 8 : 4;
        while (c.fs > 1 && waves(c.rb) * c.fs > 16384) c.fs /= 2;
        if (c.fs == 2) c.fs = 1;
    }
    return c;
}

template <class T, class TO>
hipError_t grad_input_launch(const T* gint, int band_rows, BoxParams<T> prm, TO* grad_in, Dims d,
                             bool normalize, bool exact, hipStream_t stream,
                             const ParamFinish<T>* finish, bool* finish_done) {
    if (finish_done != nullptr) *finish_done = false;
    if (d.planes == 0 || d.hw() == 0) return hipSuccess;
    SampleArgs<T> a = base_args(prm, d);
    a.src = gint; a.dst = reinterpret_cast<T*>(grad_in); a.normalize = normalize ? 1 : 0;
    a.off_R = band_rows;

    if (band_rows == 0) {
        if (!std::is_same<T, TO>::value) return hipErrorInvalidValue;   // gather kernel: T only
        // true integral images: one thread per pixel (any width)
        finish_args(a, d.planes * d.hw());
        const dim3 grid(static_cast<unsigned>((a.total + 255) / 256));
        if (exact) BOXCONV_LAUNCH("grad_input_gather", (grad_input_gather_kernel<T, true>), grid, dim3(256), 0, stream, a);
        else       BOXCONV_LAUNCH("grad_input_gather", (grad_input_gather_kernel<T, false>), grid, dim3(256), 0, stream, a);
        return hipGetLastError();
    }

    a.reverse = reverse_grad_input() ? 1 : 0;
    a.mpitch = column_workspace_pitch(d.w);
    set_workspace_layout(a, d.h, band_rows);
    a.vec_out = (d.w % 4 == 0 && reinterpret_cast<uintptr_t>(grad_in) % (4 * sizeof(TO)) == 0) ? 1 : 0;
    const ColsConfig cc = cols_config(d.planes, d.F, d.h, d.w, split_filters_enabled());
    const int ntx = std::max(64, 1 << cc.lq), rg = ntx >> cc.lq;
    const int64_t strips = (d.w + (4 << cc.lq) - 1) / (4 << cc.lq);
    a.nb = (d.h + cc.rb * rg - 1) / (cc.rb * rg);
    a.R = cc.rb;
    if (band_rows < cc.rb + 1 && band_rows < d.h) return hipErrorInvalidValue;   // a run may cross one band edge only
    finish_args(a, d.planes * a.nb * strips);
    const dim3 grid(static_cast<unsigned>(a.per_xcd * kXcds));
    const size_t lds = cc.fs > 1 ? static_cast<size_t>(cc.fs - 1) * cc.rb * 4 * ntx * sizeof(T) : 0;
    FinalizeArgs<T> fin{};
    if (finish != nullptr && finish->acc != nullptr && grid.x >= static_cast<unsigned>(finish->n_boxes)) {
        fin = finalize_args(*finish);
        if (finish_done != nullptr) *finish_done = true;
    }
#define LAUNCH_GC(LQ, RB, FS)                                                                          \
    do {                                                                                               \
        constexpr int NTX_ = (LQ) > 6 ? (1 << (LQ)) : 64;                                              \
        if (exact) BOXCONV_LAUNCH("grad_input_cols", (grad_input_cols_kernel<T, TO, LQ, RB, true, FS>), grid, dim3(NTX_, FS), lds, stream, a, fin); \
        else       BOXCONV_LAUNCH("grad_input_cols", (grad_input_cols_kernel<T, TO, LQ, RB, false, FS>), grid, dim3(NTX_, FS), lds, stream, a, fin); \
    } while (0)
#define LAUNCH_GC_FS(LQ, RB)                                                                           \
    do {                                                                                               \
        if (cc.fs == 8) LAUNCH_GC(LQ, RB, 8);                                                          \
        else if (cc.fs == 4) LAUNCH_GC(LQ, RB, 4);                                                     \
        else LAUNCH_GC(LQ, RB, 1);                                                                     \
    } while (0)
#define LAUNCH_GC_RB(LQ)                                                                               \
    do {                                                                                               \
        if (cc.rb == 2) LAUNCH_GC_FS(LQ, 2);                                                           \
        else LAUNCH_GC(LQ, 8, 1);                                                                      \
    } while (0)
    switch (cc.lq) {
        case 3: LAUNCH_GC_RB(3); break;
        case 4: LAUNCH_GC_RB(4); break;
        case 5: LAUNCH_GC_RB(5); break;
        case 6: LAUNCH_GC_RB(6); break;
        case 7: if (cc.rb == 2) LAUNCH_GC(7, 2, 1); else LAUNCH_GC(7, 8, 1); break;
        default: if (cc.rb == 2) LAUNCH_GC(8, 2, 1); else LAUNCH_GC(8, 8, 1); break;
    }
#undef LAUNCH_GC_RB
#undef LAUNCH_GC_FS
#undef LAUNCH_GC
    return hipGetLastError();
}

// How much of the band-local integral, counted from its end, is written with the ordinary cache
// policy (the memory-side cache holds 256 MB; the grad-input kernel reads that part first).
inline int64_t cached_tail_bytes() { return switches().keep_tail_bytes; }

// The launches of grad_output_stream_consec_kernel (`lanes` busy lanes of a workgroup of `cnt`;
// SCAN = false: parameter sums only). Its instantiations are translation units of their own
// (BOXCONV_INST_PART 3 and 4): some hundred kernels that would otherwise double the compile time
// of the unit with the other variant.
template <class TG, bool SCAN>
hipError_t grad_output_stream_consec_launch(const SampleArgs<float>& a, int lanes, int cnt, bool exact,
                                            dim3 grid, hipStream_t stream);
#if defined(BOXCONV_INST_PART) && (BOXCONV_INST_PART == 3 || BOXCONV_INST_PART == 4)
template <class TG, bool SCAN>
hipError_t grad_output_stream_consec_launch(const SampleArgs<float>& a, int lanes, int cnt, bool exact,
                                            dim3 grid, hipStream_t stream) {
    const size_t lds = 0;                              // the kernel's LDS is statically sized
#define LAUNCH_GC(NT) \
    if (lanes == NT) { \
        if (exact) BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_consec_kernel<TG, NT, true, true, SCAN>), grid, dim3(NT), lds, stream, a); \
        else       BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_consec_kernel<TG, NT, false, true, SCAN>), grid, dim3(NT), lds, stream, a); \
    } else { \
        if (exact) BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_consec_kernel<TG, NT, true, false, SCAN>), grid, dim3(NT), lds, stream, a); \
        else       BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_consec_kernel<TG, NT, false, false, SCAN>), grid, dim3(NT), lds, stream, a); \
    }
    switch (cnt) {
        case 64: LAUNCH_GC(64) break;
        case 128: LAUNCH_GC(128) break;
        case 192: LAUNCH_GC(192) break;
        case 256: LAUNCH_GC(256) break;
        case 320: LAUNCH_GC(320) break;
        case 384: LAUNCH_GC(384) break;
        case 448: LAUNCH_GC(448) break;
        default: LAUNCH_GC(512) break;
    }
#undef LAUNCH_GC
    return hipGetLastError();
}
#endif

template <class T, class TG>
hipError_t grad_output_stream_launch(const T* integ, const TG* grad_out, BoxParams<T> prm,
                                     double* acc, int acc_slots, T* column_workspace,
                                     const StreamPlan& sp, Dims d, bool exact, hipStream_t stream) {
    const int64_t planes_f = d.planes * d.F;
    if (planes_f == 0 || d.hw() == 0) return hipSuccess;
    const bool params = acc != nullptr, scan = column_workspace != nullptr;
    if (!sp.usable || (!params && !scan)) return hipErrorInvalidValue;
    SampleArgs<T> a = base_args(prm, d);
    a.src = integ; a.grad_out = reinterpret_cast<const T*>(grad_out); a.acc = acc; a.acc_slots = acc_slots;
    a.dst = column_workspace;
    a.mpitch = column_workspace_pitch(d.w);
    if (acc_slots != 0 && acc_slots != sp.nb * sp.parts) return hipErrorInvalidValue;
    a.nb = sp.nb; a.R = sp.R;
    set_workspace_layout(a, d.h, sp.R);
    a.keep_tail = scan ? cached_tail_bytes() / kXcds : 0;
    finish_args(a, planes_f * a.nb);
    const RowConfig rc = stream_row_config(d.w, sizeof(T));
    // The workspace layout was fixed by plan_grad_output_stream for a gfx950 CU's LDS; a device
    // that grants a workgroup less cannot run this kernel (and has no fallback at this point).
    if (stream_lds_bytes(rc.K, rc.nt, sizeof(T)) > device_lds_limit()) return hipErrorInvalidConfiguration;
    const dim3 grid(static_cast<unsigned>(a.per_xcd * kXcds));
    const size_t lds = 0;                              // the kernel's LDS is statically sized
    if (rc.nt == 1024) {
        // Rows of 2049 to 4096 columns: 16 waves per workgroup leave a lane 128 registers, which
        // the kernel that does both jobs at once does not fit; the two jobs run one after the
        // other (grad_output is then read twice).
        if constexpr (sizeof(T) <= 4) {
            // parameter sums: two workgroups of 512 threads per band, each owning half the columns
            // (a lane of the 1024-thread shape would spill half of that kernel's state)
            SampleArgs<T> ap = a;
            if (params && acc_slots == 0) return hipErrorInvalidValue;   // (the atomic mode has no slot per part)
            finish_args(ap, planes_f * a.nb * 2);
            const dim3 grid_p(static_cast<unsigned>(ap.per_xcd * kXcds));
#define LAUNCH_GW(NT, KK, EX, FU) \
            if (params) BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_kernel<T, TG, 512, KK, EX, false, true, false, 2>), grid_p, dim3(512), lds, stream, ap); \
            if (scan)   BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_kernel<T, TG, NT, KK, EX, FU, false, true>), grid, dim3(NT), lds, stream, a)
#define LAUNCH_GW_K(EX, FU) if (rc.K == 3) { LAUNCH_GW(1024, 3, EX, FU); } else { LAUNCH_GW(1024, 4, EX, FU); }
            if (exact) { if (rc.full) { LAUNCH_GW_K(true, true) } else { LAUNCH_GW_K(true, false) } }
            else       { if (rc.full) { LAUNCH_GW_K(false, true) } else { LAUNCH_GW_K(false, false) } }
#undef LAUNCH_GW_K
#undef LAUNCH_GW
            return hipGetLastError();
        } else {
            return hipErrorInvalidValue;
        }
    }
    if constexpr (sizeof(T) == 8) {
        if (stream_double_wide_split(d.w, sizeof(T))) {
            SampleArgs<T> ap = a;
            if (params && acc_slots == 0) return hipErrorInvalidValue;   // (the atomic mode has no slot per part)
            finish_args(ap, planes_f * a.nb * 2);
            const dim3 grid_p(static_cast<unsigned>(ap.per_xcd * kXcds));
#define LAUNCH_GD(KK, EX, FU) \
            if (params) BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_kernel<T, TG, 512, 2, EX, false, true, false, 2>), grid_p, dim3(512), lds, stream, ap); \
            if (scan)   BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_kernel<T, TG, 512, KK, EX, FU, false, true>), grid, dim3(512), lds, stream, a)
#define LAUNCH_GD_K(EX, FU) if (rc.K == 3) { LAUNCH_GD(3, EX, FU); } else { LAUNCH_GD(4, EX, FU); }
            if (rc.nt != 512 || rc.K < 3) return hipErrorInvalidValue;
            if (exact) { if (rc.full) { LAUNCH_GD_K(true, true) } else { LAUNCH_GD_K(true, false) } }
            else       { if (rc.full) { LAUNCH_GD_K(false, true) } else { LAUNCH_GD_K(false, false) } }
#undef LAUNCH_GD_K
#undef LAUNCH_GD
            return hipGetLastError();
        }
    }
    // float rows of a multiple of four columns, the parameter sums wanted (with or without the column
    // workspace), a slot per workgroup for the sums: the kernel with four consecutive columns per lane
    if constexpr (std::is_same<T, float>::value) {
        const bool aligned = reinterpret_cast<uintptr_t>(grad_out) % (4 * sizeof(TG)) == 0 && d.w % 4 == 0;
        // the smallest workgroup (whole waves) whose lanes, four columns each, cover the row. Only
        // a single wave can be left mostly idle (from two waves on, more than half of the lanes
        // are busy): rows that fill less than three eighths of it stay with the other kernel
        // (measured, 16 x 4 planes of 256 rows: 100 columns 97 -> 86 us, 128: 91 -> 91, 144:
        // 110 -> 90, 260: 138 -> 118, 300: 142 -> 121; but 64 columns 72 -> 83). Rows of exactly
        // 128 columns also stay there: they fill that kernel's two waves at one column per lane
        // with no bounds to check (10 to 38 x 64 planes of 64 to 256 rows: 70 against 80 us).
        const int lanes = d.w / 4;
        const int cnt = (lanes + 63) / 64 * 64;
        const bool exact_fit = lanes == cnt && (cnt == 64 || cnt == 128 || cnt == 256 || cnt == 512);
        const bool covers = d.w <= 2048 && lanes >= 1 &&
                            (exact_fit || (switches().stream_consecutive_partial && lanes * 8 >= cnt * 3 &&
                                           !(rc.full && rc.K == 1)));
        if (switches().stream_consecutive && covers && params && acc_slots > 0 && aligned) {
            if (scan) return grad_output_stream_consec_launch<TG, true>(a, lanes, cnt, exact, grid, stream);
            return grad_output_stream_consec_launch<TG, false>(a, lanes, cnt, exact, grid, stream);
        }
    }
    // doubles, two columns per lane on four or eight waves: the kernel that does both jobs needs
    // more registers than a lane has there (512 threads: 50 to 120 of them in scratch memory);
    // either job alone fits. Measured, 16 x 8 planes of 256 rows: 512 columns 212 -> 186 us,
    // 1024 columns 468 -> 362 us; on two waves (256 columns) the one kernel is as fast.
    const bool split_jobs = sizeof(T) == 8 && rc.K == 2 && rc.nt >= 256 && switches().stream_narrow_double;
#pragma push_macro("BOXCONV_DISPATCH_WIDE")
#pragma push_macro("BOXCONV_DISPATCH_K2")
#undef BOXCONV_DISPATCH_WIDE
#undef BOXCONV_DISPATCH_K2
#define BOXCONV_DISPATCH_WIDE(KERNEL, K, ...) { return hipErrorInvalidValue; }
#define BOXCONV_DISPATCH_K2(KERNEL, NT, ...)                                         \
    if constexpr (sizeof(T) == 8) { KERNEL(NT, 2, __VA_ARGS__); }                    \
    else { return hipErrorInvalidValue; }
#define LAUNCH_GS(NT, KK, EX, FU) \
    if (params && scan && split_jobs) { \
        BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_kernel<T, TG, NT, KK, EX, FU, true, false>), grid, dim3(NT), lds, stream, a); \
        BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_kernel<T, TG, NT, KK, EX, FU, false, true>), grid, dim3(NT), lds, stream, a); \
    } else \
    if (params && scan) BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_kernel<T, TG, NT, KK, EX, FU, true, true>), grid, dim3(NT), lds, stream, a); \
    else if (params)    BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_kernel<T, TG, NT, KK, EX, FU, true, false>), grid, dim3(NT), lds, stream, a); \
    else                BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_kernel<T, TG, NT, KK, EX, FU, false, true>), grid, dim3(NT), lds, stream, a)
    BOXCONV_DISPATCH_SHAPE_EXACT_FULL(LAUNCH_GS, rc, exact)
#undef LAUNCH_GS
#pragma pop_macro("BOXCONV_DISPATCH_K2")
#pragma pop_macro("BOXCONV_DISPATCH_WIDE")
    return hipGetLastError();
}

// Parameter-gradient sums from a true integral image with the gather kernel (any width).
template <class T>
hipError_t grad_params_gather_launch(const T* integ, const T* grad_out, BoxParams<T> prm,
                                     double* acc, Dims d, bool exact, hipStream_t stream) {
    const int64_t planes_f = d.planes * d.F;
    if (planes_f == 0 || d.hw() == 0) return hipSuccess;
    SampleArgs<T> a = base_args(prm, d);
    a.src = integ; a.grad_out = grad_out; a.acc = acc;
    const int bpp = static_cast<int>((d.hw() + 255) / 256);
    finish_args(a, planes_f * bpp);
    const dim3 grid(static_cast<unsigned>(a.total));
    if (exact) BOXCONV_LAUNCH("grad_params_gather", (grad_params_gather_kernel<T, true>), grid, dim3(256), 0, stream, a, bpp);
    else       BOXCONV_LAUNCH("grad_params_gather", (grad_params_gather_kernel<T, false>), grid, dim3(256), 0, stream, a, bpp);
    return hipGetLastError();
}

template <class T>
hipError_t grad_params_finish(const ParamFinish<T>& f, BoxParams<T> prm, hipStream_t stream) {
    if (f.n_boxes == 0) return hipSuccess;
    BOXCONV_LAUNCH("param_grad_finalize", (param_grad_finalize_kernel<T>), dim3(f.n_boxes), dim3(64), 0,
                   stream, finalize_args(f), prm);
    return hipGetLastError();
}

}  // namespace boxconv
