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

#include "box_sampling_common.hpp"

namespace boxconv {

bool force_gather_kernels() {
    const char* e = std::getenv("BOXCONV_FORCE_GATHER");
    return e != nullptr && e[0] == '1';
}

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
};

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
    if (lane != 63) return;
    const T xmin = prm.xmin[k], xmax = prm.xmax[k], ymin = prm.ymin[k], ymax = prm.ymax[k];
    const bool ex = fa.exact != 0;
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
// Gradient w.r.t. the input. Work item = (plane p = (b,c), band of RB rows); the F mirrored boxes
// are visited in order and summed in registers, so no [B,C,F,h,w] temporary exists.
//
// OFFS: `src` holds BAND-LOCAL integral images (see grad_output_stream_kernel). A box sum only
// involves differences between rows, so a row is corrected relative to a reference band (that of
// the first row this workgroup touches for the filter): the bulk of the integral cancels before
// it is ever added.
//
// Registers: the float shapes that need about 128 registers per lane are held to 128 (four waves per
// SIMD, i.e. two 512-thread workgroups per CU; one register more would halve that); the wider
// shapes need far more and are left to the compiler.
//
// FS > 1 (narrow images, one column per lane): the workgroup holds FS sets of NT threads
// (threadIdx.y), set g visits filters g, g + FS, ..., and the FS partial sums are added in that
// order at the end. A small workgroup that walks through all F filters is one long chain of
// memory round trips; on small problems, which cannot fill the chip with workgroups, that chain
// is the whole run time of the launch.
template <class T, int NT, int K, int RB, bool EXACT, bool FULL, bool OFFS, int FS = 1>
__global__ void __launch_bounds__(NT * FS, (FS == 1 && sizeof(T) == 4 && (K <= 2 || (K == 3 && !FULL)) ? 4 : 1))
grad_input_rows_kernel(SampleArgs<T> a, FinalizeArgs<T> fin) {
    static_assert(RB % 4 == 0, "rows are handled in pairs, and pairs alternate between two LDS buffers");
    // Rides along: the first fin.n workgroups each finish the parameter gradients of one box from
    // the sums the preceding launch left (one wave's work; saves a launch of its own).
    if (fin.acc != nullptr && blockIdx.x < static_cast<unsigned>(fin.n) && threadIdx.x < 64 &&
        (FS == 1 || threadIdx.y == 0))
        finalize_box(fin, a.prm, static_cast<int>(blockIdx.x), static_cast<int>(threadIdx.x));
    unsigned vid = xcd_contiguous_id(a.per_xcd);
    if (vid >= a.total) return;
    if (a.reverse) vid = static_cast<unsigned>(a.total) - 1u - vid;
    const unsigned nbands = a.nb;
    const int band = static_cast<int>(vid % nbands);
    const int64_t p = vid / nbands;
    const int c_in = static_cast<int>(static_cast<unsigned>(a.plane0 + p) % static_cast<unsigned>(a.C));
    const int h = a.h, w = a.w;
    const unsigned row_bytes = static_cast<unsigned>(w) * sizeof(T);
    const int64_t pitch = w + 1;
    const int64_t ipl = static_cast<int64_t>(h + 1) * pitch;
    const int vlen = w + 3;
    // which share of the filters (one value per wave: kept scalar)
    const int fgroup = FS > 1 ? __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.y)) : 0;
    RowPair<T>* vbuf = reinterpret_cast<RowPair<T>*>(smem_raw) + fgroup * 2 * vlen;
    clear_row_pads(vbuf, vlen);
    const int i0 = band * RB;

    const int q1 = lane_q1<T>();

    T acc[RB][K];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int k = 0; k < K; ++k) acc[r][k] = T(0);

    // The box of the next filter is fetched while the current one is worked on (scalar loads
    // whose latency would otherwise sit in front of every filter's first row loads).
    // (FS > 1: every wave makes the same number of turns, as the barriers below are the
    // workgroup's; a wave whose turn has no filter left repeats the last one and adds nothing.)
    BoxOfWorkgroup<T> bx_next = load_box(a.prm, c_in * a.F + min(fgroup, a.F - 1));
    for (int f0 = 0; f0 < a.F; f0 += FS) {
        const int f = min(f0 + fgroup, a.F - 1);
        const bool counts = f0 + fgroup < a.F;
        const BoxOfWorkgroup<T> bx = bx_next;
        bx_next = load_box(a.prm, c_in * a.F + min(f + FS, a.F - 1));
        const BoxSplit<T> s = split_grad_input(bx.xmin, bx.xmax, bx.ymin, bx.ymax);
        const T scale = a.normalize
            ? inverse_extent(bx.xmin, bx.xmax, bx.ymin, bx.ymax, EXACT, true, true) : T(1);
        const LoadRows<T> irows(a.src + (p * a.F + f) * ipl, pitch, w + 1, h + 1);

        unsigned lo[K], hi[K];
        column_taps<T, NT, K>(lo, hi, s.ylo, s.yhi, w);

        // OFFS: the plane holds a band-local integral (bands of off_R rows, each restarting at
        // zero). Integral row r (1..h) belongs to band (r-1)/off_R; row 0 counts as band 0. The
        // true integral I[r] is the stored row L[r] plus base(band(r)), the sum of the bottom rows
        // of all bands above. V only contains differences of rows, so only differences of base()
        // matter. The RB+2 rows of a side (top: i+xlo-1 .., bottom: i+xhi ..) span fewer rows than
        // a band, so each side starts in one band (band_t, band_b) and may cross into the next
        // once. Relative to band_t:
        //   I_t = L_t + c * E_t,             c = 1 for top rows beyond band_t, E_t = its bottom row
        //   I_b = L_b + off_b + d * E_b,     d = 1 for bottom rows beyond band_b, E_b likewise,
        //                                    off_b = base(band_b) - base(band_t), summed in double
        // and V picks these up with the weights of its rows: off_b once, E_t and E_b with scalar
        // weights that are 0 or -+1 except in the one row pair where the crossing happens.
        const int first_t = clampi(i0 + s.xlo - 1, 0, h), final_t = clampi(i0 + RB - 1 + s.xlo, 0, h);
        const int first_b = clampi(i0 + s.xhi, 0, h), final_b = clampi(i0 + RB + s.xhi, 0, h);
        auto bottoms_between = [&](int from_band, int to_band, T (&dst)[K]) {
            double sum[K];
#pragma unroll
            for (int k = 0; k < K; ++k) sum[k] = 0.0;
            for (int b = from_band; b < to_band; ++b) {
                T bottom[K];
                load_row<T, NT, K>(irows.row(min(h, (b + 1) * a.off_R)), q1, bottom);
#pragma unroll
                for (int k = 0; k < K; ++k) sum[k] += static_cast<double>(bottom[k]);
            }
#pragma unroll
            for (int k = 0; k < K; ++k) dst[k] = static_cast<T>(sum[k]);
        };
        // The first six rows are requested before anything else that reads memory for this
        // filter (the band offsets below wait for their own rows band by band): their latency
        // then overlaps with those waits instead of following them.
        // (Only with one or two columns per lane: with more, keeping six more rows in registers
        // across the offset code lowers the occupancy, which costs more than the overlap gains.)
        constexpr bool EARLY_ROWS = K <= 2;
        T ta[K], bc[K], t0[K], t1[K], b1[K], b2[K];
        auto first_rows = [&]() {
            load_row<T, NT, K>(irows.row(first_t), q1, ta);
            load_row<T, NT, K>(irows.row(first_b), q1, bc);
            load_pair<T, NT, K, FULL>(irows, i0, s.xlo, s.xhi, h, q1, t0, t1, b1, b2);
        };
        if (EARLY_ROWS) first_rows();

        int last_t = h, last_b = h;                 // last row of the band each side starts in
        bool crossing = false;
        T off_b[K], e_t[K], e_b[K];
#pragma unroll
        for (int k = 0; k < K; ++k) { off_b[k] = T(0); e_t[k] = T(0); e_b[k] = T(0); }
        if (OFFS) {
            const int band_t = max(first_t - 1, 0) / a.off_R, band_b = max(first_b - 1, 0) / a.off_R;
            last_t = (band_t + 1) * a.off_R;
            last_b = (band_b + 1) * a.off_R;
            if (band_b > band_t) bottoms_between(band_t, band_b, off_b);
            if (band_b < band_t) {                  // a box given with min > max
                bottoms_between(band_b, band_t, off_b);
#pragma unroll
                for (int k = 0; k < K; ++k) off_b[k] = -off_b[k];
            }
            const bool cross_t = final_t > last_t, cross_b = final_b > last_b;
            crossing = cross_t || cross_b;
            if (cross_t) load_row<T, NT, K>(irows.row(min(h, last_t)), q1, e_t);
            if (cross_b) load_row<T, NT, K>(irows.row(min(h, last_b)), q1, e_b);
        }
        if (!EARLY_ROWS) first_rows();

        // All RB rows are always computed (rows past the image read clamped, valid rows and
        // are not stored) and the prefetch of the next pair is decided at compile time:
        // straight-line code, so loads stay in flight across the barrier.
#pragma unroll
        for (int r = 0; r < RB; r += 2) {
            const int i = i0 + r;
            T n0[K] = {}, n1[K] = {}, n2[K] = {}, n3[K] = {};
            const bool more = r + 2 < RB;                            // known after unrolling
            if (more)
                load_pair<T, NT, K, FULL>(irows, i + 2, s.xlo, s.xhi, h, q1, n0, n1, n2, n3);
            RowPair<T>* V = vbuf + (((r >> 1) & 1) ? vlen : 0);
            T v0[K], v1[K];
#pragma unroll
            for (int k = 0; k < K; ++k) {
                v0[k] = blend<T, EXACT>(ta[k], t0[k], bc[k], b1[k], s.fxlo, s.fxhi);
                v1[k] = blend<T, EXACT>(t0[k], t1[k], b1[k], b2[k], s.fxlo, s.fxhi);
                if (OFFS) { v0[k] += off_b[k]; v1[k] += off_b[k]; }
            }
            if (OFFS && crossing) {                                  // uniform; one batch in four
                // which of the pair's rows lie beyond their side's first band (scalars)
                const T cA = T(clampi(i + s.xlo - 1, 0, h) > last_t), c0 = T(clampi(i + s.xlo, 0, h) > last_t),
                        c1 = T(clampi(i + 1 + s.xlo, 0, h) > last_t);
                const T dC = T(clampi(i + s.xhi, 0, h) > last_b), d1 = T(clampi(i + 1 + s.xhi, 0, h) > last_b),
                        d2 = T(clampi(i + 2 + s.xhi, 0, h) > last_b);
                // weights of E_b and E_t in blend(lo_adv, lo, hi, hi_adv)
                const T fhi = EXACT ? s.fxhi : T(0), flo = EXACT ? s.fxlo : T(0);
                const T wb0 = dC + fhi * (d1 - dC), wt0 = flo * (c0 - cA) - c0;
                const T wb1 = d1 + fhi * (d2 - d1), wt1 = flo * (c1 - c0) - c1;
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    v0[k] += wb0 * e_b[k] + wt0 * e_t[k];
                    v1[k] += wb1 * e_b[k] + wt1 * e_t[k];
                }
            }
            publish_rows<T, NT, K, FULL>(V, v0, v1, w, row_bytes, q1);
            __syncthreads();
#pragma unroll
            for (int k = 0; k < K; ++k) {
                if (slot_valid<T, NT, FULL>(q1, k, row_bytes) && (FS == 1 || counts)) {
                    const RowPair<T> o = sample_columns<T, EXACT>(V, lo[k], hi[k], s.fylo, s.fyhi);
                    acc[r][k] += scale * o.r0;
                    acc[r + 1][k] += scale * o.r1;
                }
            }
            if (more) {
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    ta[k] = t1[k]; bc[k] = b2[k];
                    t0[k] = n0[k]; t1[k] = n1[k]; b1[k] = n2[k]; b2[k] = n3[k];
                }
            }
        }
    }

    if constexpr (FS > 1) {
        // partial sums of waves 1..FS-1 go through LDS (the row buffers are done with) and are
        // added by wave 0 in wave order
        T* part = reinterpret_cast<T*>(smem_raw);
        __syncthreads();
        if (fgroup > 0) {
#pragma unroll
            for (int r = 0; r < RB; ++r)
#pragma unroll
                for (int k = 0; k < K; ++k)
                    part[(((fgroup - 1) * RB + r) * K + k) * NT + threadIdx.x] = acc[r][k];
        }
        __syncthreads();
        if (fgroup > 0) return;
        for (int g = 1; g < FS; ++g)
#pragma unroll
            for (int r = 0; r < RB; ++r)
#pragma unroll
                for (int k = 0; k < K; ++k)
                    acc[r][k] += part[(((g - 1) * RB + r) * K + k) * NT + threadIdx.x];
    }

    // column slot q = j + 1 lands on pixel j; rows past the image get size 0
    const Rows<T, FULL> orows(a.dst + p * static_cast<int64_t>(h) * w - 1, w, w + 1, h);
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        const int i = i0 + r;
        const RowRef ob = orows.row(min(i, h - 1), i < h);
#pragma unroll
        for (int k = 0; k < K; ++k) store_slot<T, NT, kCacheDefault>(acc[r][k], ob, q1, k);
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
// (SCAN) the BAND-LOCAL integral image of grad_output: L[i+1][c+1] = sum of grad_output over rows
// band_start..i and columns 0..c. Bands do not depend on each other, so nothing has to be known
// about the rows above: the true integral is L plus the bottom rows of the bands above, which
// the grad-input kernel adds when it loads a row. Lanes own K consecutive columns for this part
// (read back from the LDS row) and store them as one run, so a wave writes 64*K contiguous
// elements per row.
//
// LDS: [2 buffers][K*nt + 8] RowPair grad_output rows (4 zero pairs in front, >= 4 behind),
//      [2][2][4] X[w] triples, [K*nt] tail weights, [8*5] doubles, [2][8] wave totals.
constexpr int kGPad = 4;

template <class T>
struct StreamLds {
    RowPair<T>* grow;   // [2][glen]
    T* xw;              // [2][2][4]
    T* delta;           // [K*nt] tail weight of pixel column j
    double* red;        // [5 * kMaxRowWaves]
    T* wave_tot;        // [2][kMaxRowWaves]
    int glen;
};

__host__ __device__ inline size_t stream_lds_bytes(int K, int nt, size_t elem) {
    const size_t glen = static_cast<size_t>(K) * nt + 8;
    size_t b = (4 * glen + 16 + static_cast<size_t>(K) * nt) * elem;
    b = (b + 15) / 16 * 16;
    return b + (2 * kMaxRowWaves + 5 * kMaxRowWaves) * sizeof(double);
}

template <class T>
__device__ __forceinline__ StreamLds<T> carve_stream_lds(int K, int nt) {
    StreamLds<T> l;
    l.glen = K * nt + 8;
    l.grow = reinterpret_cast<RowPair<T>*>(smem_raw);
    l.xw = reinterpret_cast<T*>(l.grow + 2 * l.glen);
    l.delta = l.xw + 16;
    size_t b = (4 * static_cast<size_t>(l.glen) + 16 + static_cast<size_t>(K) * nt) * sizeof(T);
    b = (b + 15) / 16 * 16;
    l.red = reinterpret_cast<double*>(smem_raw + b);
    l.wave_tot = reinterpret_cast<T*>(l.red + 5 * kMaxRowWaves);
    return l;
}

template <class T, int WV>
__device__ __forceinline__ void add_waves_left(const T* wave_tot, int wave, T& carry0, T& carry1) {
    if constexpr (WV < kMaxRowWaves - 1) {
        if (wave > WV) {
            carry0 += wave_tot[WV];
            carry1 += wave_tot[kMaxRowWaves + WV];
            add_waves_left<T, WV + 1>(wave_tot, wave, carry0, carry1);
        }
    }
}

template <class T, int NT, int K, bool EXACT, bool FULL, bool PARAMS, bool SCAN>
__global__ void __launch_bounds__(NT) grad_output_stream_kernel(SampleArgs<T> a) {
    const unsigned vid = xcd_contiguous_id(a.per_xcd);
    if (vid >= a.total) return;                      // whole workgroup leaves together
    const unsigned nbands = a.nb, nfilt = a.F;
    const int band = static_cast<int>(vid % nbands);
    const unsigned pf32 = vid / nbands;
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
    // integral of the input; grad_output (one element early: column slot q = j + 1 is pixel j);
    // band-local integral of grad_output
    const LoadRows<T> irows(a.src + p * static_cast<int64_t>(h + 1) * pitch, pitch, w + 1, h + 1);
    const LoadRows<T> grows(a.grad_out + pf * static_cast<int64_t>(h) * w - 1, w, w + 1, h);
    T* lrows = SCAN ? a.dst + pf * static_cast<int64_t>(h + 1) * pitch : nullptr;
    // The bands an XCD writes last (the final keep_tail bytes of its range) are stored with the
    // ordinary cache policy, everything before them non-temporally: see the store below.
    const unsigned from_end = static_cast<unsigned>(a.per_xcd) - 1u - vid % static_cast<unsigned>(a.per_xcd);
    const bool keep_in_cache =
        static_cast<uint64_t>(from_end) * a.R * pitch * sizeof(T) < static_cast<uint64_t>(a.keep_tail);
    const Rows<T, FULL> lout(lrows, pitch, w + 1, h + 1);
    const StreamLds<T> lds = carve_stream_lds<T>(K, nt);
    const int glen = lds.glen;

    const int i0 = band * a.R;
    const int i1 = min(h, i0 + a.R);

    // The first two rows of grad_output are requested before anything else: they come from HBM
    // and need nothing but the workgroup's coordinates, so their latency runs alongside the
    // set-up below (LDS clearing, box parameters, column weights).
    const int q1 = lane_q1<T>();
    T g0[K], g1[K];
    auto load_g = [&](int i, T (&dst)[K]) {
        const RowRef r = grows.row(min(i, h - 1), i < i1);     // rows past the band read as zeros
#pragma unroll
        for (int k = 0; k < K; ++k) dst[k] = load_slot<T, NT, kCacheStream>(r, q1, k);
    };
    load_g(i0, g0);
    load_g(i0 + 1, g1);

    // clear the grad_output rows once: pads and the columns beyond w stay zero for good
    for (int e = tid; e < 2 * glen; e += nt) lds.grow[e] = RowPair<T>{T(0), T(0)};
    if (SCAN && band == 0)
        for (int c = tid; c <= w; c += nt) lrows[c] = T(0);                    // integral row 0
    __syncthreads();

    // lane-constant LDS byte offsets of the pairs (grA, gr) and (gl, glA); the tail weights of the
    // lane's columns go to LDS (read back once per row pair: cheaper than K live registers)
    unsigned ir[K], il[K];
    unsigned idx_ymax = 0, idx_ymin = 0;
    if (PARAMS) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int j = tid + nt * k;
            const int q = j + 1;
            ir[k] = static_cast<unsigned>(clampi(q - s.yhi - 1, -2, w) + kGPad) * static_cast<unsigned>(sizeof(RowPair<T>));
            il[k] = static_cast<unsigned>(clampi(q - s.ylo, -2, w) + kGPad) * static_cast<unsigned>(sizeof(RowPair<T>));
            T d = T(0);
            if (FULL || j < w) {
                const T one = T(1);
                d = (EXACT ? (one - s.fyhi) : one) * T(j > w - s.yhi)
                  + (EXACT ? s.fyhi : T(0)) * T(j > w - s.yhi - 1)
                  - (EXACT ? (one - s.fylo) : one) * T(j > w - s.ylo)
                  - (EXACT ? s.fylo : T(0)) * T(j > w - s.ylo + 1);
            }
            lds.delta[j] = d;
        }
        const int j_ymax = w - s.yhi, j_ymin = w - s.ylo + 1;
        idx_ymax = (j_ymax >= 0 && j_ymax < w) ? j_ymax + kGPad : 0;          // index 0 holds a zero
        idx_ymin = (j_ymin >= 0 && j_ymin < w) ? j_ymin + kGPad : 0;
    }

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
        load_row<T, NT, K>(irows.row(clampi(i0 + s.xlo - 1, 0, h)), q1, ta);
        load_row<T, NT, K>(irows.row(clampi(i0 + s.xhi, 0, h)), q1, bc);
        load_pair<T, NT, K, FULL>(irows, i0, s.xlo, s.xhi, h, q1, t0, t1, b1, b2);
    }

    int flip = 0;
    auto row_pair = [&](int i, auto prefetch_tag) {
        constexpr bool PREFETCH = decltype(prefetch_tag)::value;   // see forward_rows_kernel
        // (the LDS buffer alternates at run time here: unrolling this loop over both buffers, as
        // the forward kernel does, costs more registers than the kernel can afford)
        const int FLIP = flip;
        flip ^= 1;
        T n0[K] = {}, n1[K] = {}, n2[K] = {}, n3[K] = {}, m0[K] = {}, m1[K] = {};
        if (PREFETCH) {
            if (PARAMS)
                load_pair<T, NT, K, FULL>(irows, i + 2, s.xlo, s.xhi, h, q1, n0, n1, n2, n3);
            load_g(i + 2, m0);
            load_g(i + 3, m1);
        }

        RowPair<T>* G = lds.grow + (FLIP ? glen : 0);
        T* X0 = lds.xw + FLIP * 8;
        T* X1 = X0 + 4;

        T tail0 = T(0), tail1 = T(0);
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (slot_valid<T, NT, FULL>(q1, k, row_bytes))
                *at_bytes(G + kGPad - 1 + NT * k, 2 * q1) = RowPair<T>{g0[k], g1[k]};
            if (PARAMS) {
                const T dlt = *at_bytes(lds.delta - 1 + NT * k, q1);
                tail0 += dlt * g0[k];
                tail1 += dlt * g1[k];
            }
            if (PARAMS && (FULL ? (k == K - 1 && tid == nt - 1) : (q1 + slot_bytes<T, NT>(k) == row_bytes))) {   // owner of column q = w
                const T dt0 = t0[k] - ta[k], db0 = b1[k] - bc[k];
                const T dt1 = t1[k] - t0[k], db1 = b2[k] - b1[k];
                T v0 = bc[k] - t0[k], v1 = b1[k] - t1[k];
                if (EXACT) {
                    v0 += s.fxhi * db0; v0 += s.fxlo * dt0;
                    v1 += s.fxhi * db1; v1 += s.fxlo * dt1;
                }
                X0[0] = v0; X0[1] = dt0; X0[2] = db0;
                X1[0] = v1; X1[1] = dt1; X1[2] = db1;
            }
        }
        __syncthreads();                                                     // rows are in LDS

        if (PARAMS) {
            T sum[5] = {T(0), T(0), T(0), T(0), T(0)};
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const T dt0 = t0[k] - ta[k], db0 = b1[k] - bc[k];
                const T dt1 = t1[k] - t0[k], db1 = b2[k] - b1[k];
                T v0 = bc[k] - t0[k], v1 = b1[k] - t1[k];
                if (EXACT) {
                    v0 += s.fxhi * db0; v0 += s.fxlo * dt0;
                    v1 += s.fxhi * db1; v1 += s.fxlo * dt1;
                }
                const RowPair<T>* R = at_bytes(G, ir[k]);
                const RowPair<T>* L = at_bytes(G, il[k]);
                const RowPair<T> grA = R[0], gr = R[1], gl = L[0], glA = L[1];
                {
                    const T dr = grA.r0 - gr.r0, dl = gl.r0 - glA.r0;
                    T wq = gr.r0 - gl.r0;
                    if (EXACT) { wq += s.fyhi * dr; wq += s.fylo * dl; }
                    sum[4] += v0 * wq;
                    sum[1] += db0 * wq;
                    sum[0] -= dt0 * wq;
                    sum[3] += v0 * dr;
                    sum[2] -= v0 * dl;
                }
                {
                    const T dr = grA.r1 - gr.r1, dl = gl.r1 - glA.r1;
                    T wq = gr.r1 - gl.r1;
                    if (EXACT) { wq += s.fyhi * dr; wq += s.fylo * dl; }
                    sum[4] += v1 * wq;
                    sum[1] += db1 * wq;
                    sum[0] -= dt1 * wq;
                    sum[3] += v1 * dr;
                    sum[2] -= v1 * dl;
                }
            }
            const T vw0 = X0[0], dtw0 = X0[1], dbw0 = X0[2];
            const T vw1 = X1[0], dtw1 = X1[1], dbw1 = X1[2];
            sum[4] += vw0 * tail0 + vw1 * tail1;
            sum[1] += dbw0 * tail0 + dbw1 * tail1;
            sum[0] -= dtw0 * tail0 + dtw1 * tail1;
            if (tid == 0) {
                const RowPair<T> gmax = G[idx_ymax], gmin = G[idx_ymin];
                sum[3] += vw0 * gmax.r0 + vw1 * gmax.r1;
                sum[2] -= vw0 * gmin.r0 + vw1 * gmin.r1;
            }
#pragma unroll
            for (int n = 0; n < 5; ++n) total[n] += static_cast<double>(sum[n]);
        }

        if (SCAN) {
            // lane owns columns K*tid .. K*tid+K-1; two rows of the band-local integral. A band
            // restarts at zero and the row prefix is a tree (inside the lane, across the wave,
            // across waves), so plain T arithmetic loses a few ulps of the band-local value only.
            T loc0[K], loc1[K];
            T carry0, carry1;
            {
                const RowPair<T>* r = G + kGPad + K * tid;
                T run0 = T(0), run1 = T(0);
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    const RowPair<T> g = r[k];
                    colacc[k] += g.r0;
                    run0 += colacc[k];
                    loc0[k] = run0;
                    colacc[k] += g.r1;
                    run1 += colacc[k];
                    loc1[k] = run1;
                }
                const T inc0 = wave_inclusive_scan(run0);
                const T inc1 = wave_inclusive_scan(run1);
                carry0 = inc0 - run0;
                carry1 = inc1 - run1;
                if (lane == 63) { lds.wave_tot[wave] = inc0; lds.wave_tot[kMaxRowWaves + wave] = inc1; }
            }
            __syncthreads();                                                 // wave totals visible
            {
                // totals of the waves to the left; `wave` is scalar, so these are scalar branches
                // and wave n takes n + 1 of them
                add_waves_left<T, 0>(lds.wave_tot, wave, carry0, carry1);
                // the lane's K consecutive columns K*tid+1 .. K*tid+K of integral rows i+1, i+2:
                // a wave stores one contiguous run of 64*K elements per row. The grad-input
                // kernel starts with the planes written last and finds them still in the
                // memory-side cache if they were stored with the ordinary policy; the rest is
                // stored non-temporally so that it does not push the integral plane of the
                // input, which all filters of a plane re-read, out of the L2.
                T* o0 = lrows + static_cast<int64_t>(i + 1) * pitch;
                const bool second = i + 1 < i1;
                const RowRef ob0 = lout.row(i + 1);
                const RowRef ob1 = lout.row(min(i + 2, h), second);
                T out0[K], out1[K];
#pragma unroll
                for (int k = 0; k < K; ++k) { out0[k] = carry0 + loc0[k]; out1[k] = carry1 + loc1[k]; }
                const int first = (1 + K * tid) * static_cast<int>(sizeof(T));
                if (keep_in_cache) {
                    buffer_store_run<kCacheDefault, FULL>(out0, ob0, first, static_cast<int>(row_bytes + sizeof(T)));
                    buffer_store_run<kCacheDefault, FULL>(out1, ob1, first, static_cast<int>(row_bytes + sizeof(T)));
                } else {
                    buffer_store_run<kCacheStream, FULL>(out0, ob0, first, static_cast<int>(row_bytes + sizeof(T)));
                    buffer_store_run<kCacheStream, FULL>(out1, ob1, first, static_cast<int>(row_bytes + sizeof(T)));
                }
                if (tid == 0) {
                    o0[0] = T(0);
                    if (second) o0[pitch] = T(0);
                }
            }
        }

        if (PREFETCH) {
#pragma unroll
            for (int k = 0; k < K; ++k) {
                if (PARAMS) {
                    ta[k] = t1[k]; bc[k] = b2[k];
                    t0[k] = n0[k]; t1[k] = n1[k]; b1[k] = n2[k]; b2[k] = n3[k];
                }
                g0[k] = m0[k]; g1[k] = m1[k];
            }
        }
        // keep the two unrolled pairs apart: loads of the pair after next hoisted up here would
        // only add live registers
        __builtin_amdgcn_sched_barrier(0);
    };
    int i = i0;
    for (; i + 2 < i1; i += 2) row_pair(i, std::true_type{});
    row_pair(i, std::false_type{});

    if (PARAMS) {
        __syncthreads();
        // slots > 0: one slot per workgroup, summed by the finalize kernel in a fixed order
        // (no clearing pass, no atomics, bit-reproducible); else atomics into the box's five sums
        if (a.acc_slots > 0)
            block_accumulate5(total, a.acc + ((static_cast<int64_t>(a.plane0 + p) * a.F + f) * a.acc_slots + band) * 5,
                              lds.red, false);
        else
            block_accumulate5(total, a.acc + static_cast<int64_t>(k_par) * 5, lds.red);
    }
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

// ---------------------------------------------------------------------------------------------
__global__ void fill_zero_kernel(double* __restrict__ p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.0;
}


}  // namespace


template <class T>
FinalizeArgs<T> finalize_args(const ParamFinish<T>& f) {
    FinalizeArgs<T> fa{};
    fa.acc = f.acc; fa.batch = f.batch; fa.slots = f.acc_slots;
    for (int i = 0; i < 4; ++i) fa.g[i] = f.grad[i];
    fa.n = f.n_boxes; fa.reparam_h = f.reparam_h; fa.reparam_w = f.reparam_w;
    fa.normalize = f.normalize ? 1 : 0; fa.exact = f.exact ? 1 : 0;
    return fa;
}

// BOXCONV_GI_SPLIT_FILTERS=0 keeps the workgroups of narrow images at one row's width (for
// comparison; read at every call, so that a test can switch it within one process).
inline bool split_filters_enabled() {
    const char* e = std::getenv("BOXCONV_GI_SPLIT_FILTERS");
    return e == nullptr || std::atoi(e) != 0;
}

template <class T>
hipError_t grad_input_launch(const T* gint, int band_rows, BoxParams<T> prm, T* grad_in, Dims d,
                             bool normalize, bool exact, hipStream_t stream,
                             const ParamFinish<T>* finish, bool* finish_done) {
    if (finish_done != nullptr) *finish_done = false;
    if (d.planes == 0 || d.hw() == 0) return hipSuccess;
    SampleArgs<T> a = base_args(prm, d);
    a.src = gint; a.dst = grad_in; a.normalize = normalize ? 1 : 0;
    a.off_R = band_rows;
    a.reverse = (band_rows > 0 && reverse_grad_input()) ? 1 : 0;

    if (!row_kernels_apply(d.h, d.w, sizeof(T))) {
        if (band_rows > 0) return hipErrorInvalidValue;         // the gather kernel needs a true integral
        finish_args(a, d.planes * d.hw());
        const dim3 grid(static_cast<unsigned>((a.total + 255) / 256));
        if (exact) BOXCONV_LAUNCH("grad_input_gather", (grad_input_gather_kernel<T, true>), grid, dim3(256), 0, stream, a);
        else       BOXCONV_LAUNCH("grad_input_gather", (grad_input_gather_kernel<T, false>), grid, dim3(256), 0, stream, a);
        return hipGetLastError();
    }

    constexpr int RB = 8;
    static const int gi_threads = preferred_row_threads("BOXCONV_GI_THREADS", 512);
    const RowConfig rc = row_config(d.w, gi_threads);
    a.nb = (d.h + RB - 1) / RB;
    a.R = RB;
    finish_args(a, d.planes * a.nb);
    const dim3 grid(static_cast<unsigned>(a.per_xcd * kXcds));
    const size_t lds = 4 * static_cast<size_t>(d.w + 3) * sizeof(T);
    // One column per lane on a problem too small to fill the chip: the workgroup is widened to
    // 512 (one or two waves per row) or 1024 threads (four waves per row) and its waves share the
    // filters (see the kernel).
    const int waves_per_row = rc.nt / 64;
    const bool split_filters = rc.K == 1 && rc.nt <= 256 && d.F >= 4 &&
                               a.total * waves_per_row <= 4096 && split_filters_enabled();
    const int fs = rc.nt == 64 ? 8 : 4;
    const size_t lds_split = std::max(lds * fs, static_cast<size_t>(fs - 1) * RB * rc.nt * sizeof(T));
    FinalizeArgs<T> fin{};
    if (finish != nullptr && finish->acc != nullptr && grid.x >= static_cast<unsigned>(finish->n_boxes)) {
        fin = finalize_args(*finish);
        if (finish_done != nullptr) *finish_done = true;
    }
#define LAUNCH_GI(NT, KK, EX, FU) \
    if (band_rows > 0) BOXCONV_LAUNCH("grad_input_rows", (grad_input_rows_kernel<T, NT, KK, RB, EX, FU, true>), grid, dim3(NT), lds, stream, a, fin); \
    else BOXCONV_LAUNCH("grad_input_rows", (grad_input_rows_kernel<T, NT, KK, RB, EX, FU, false>), grid, dim3(NT), lds, stream, a, fin)
#define LAUNCH_GI_SPLIT(NT, FS, EX, FU) \
    if (band_rows > 0) BOXCONV_LAUNCH("grad_input_rows", (grad_input_rows_kernel<T, NT, 1, RB, EX, FU, true, FS>), grid, dim3(NT, FS), lds_split, stream, a, fin); \
    else BOXCONV_LAUNCH("grad_input_rows", (grad_input_rows_kernel<T, NT, 1, RB, EX, FU, false, FS>), grid, dim3(NT, FS), lds_split, stream, a, fin)
#define LAUNCH_GI_SPLIT_SHAPE(EX, FU) \
    if (rc.nt == 64) { LAUNCH_GI_SPLIT(64, 8, EX, FU); } \
    else if (rc.nt == 128) { LAUNCH_GI_SPLIT(128, 4, EX, FU); } \
    else { LAUNCH_GI_SPLIT(256, 4, EX, FU); }
    if (split_filters) {
        if (exact) { if (rc.full) { LAUNCH_GI_SPLIT_SHAPE(true, true) } else { LAUNCH_GI_SPLIT_SHAPE(true, false) } }
        else       { if (rc.full) { LAUNCH_GI_SPLIT_SHAPE(false, true) } else { LAUNCH_GI_SPLIT_SHAPE(false, false) } }
    } else {
        BOXCONV_DISPATCH_SHAPE_EXACT_FULL(LAUNCH_GI, rc, exact)
    }
#undef LAUNCH_GI_SPLIT_SHAPE
#undef LAUNCH_GI_SPLIT
#undef LAUNCH_GI
    return hipGetLastError();
}

hipError_t grad_params_begin(double* acc, int n_boxes, hipStream_t stream) {
    if (n_boxes == 0) return hipSuccess;
    BOXCONV_LAUNCH("fill_zero", fill_zero_kernel, dim3((n_boxes * 5 + 255) / 256), dim3(256), 0,
                   stream, acc, n_boxes * 5);
    return hipGetLastError();
}

StreamPlan plan_grad_output_stream(int64_t planes_f, int h, int w, size_t elem_size) {
    StreamPlan sp{};
    const RowConfig rc = stream_row_config(std::max(w, 1));
    sp.usable = row_kernels_apply(h, w, elem_size) &&
                stream_lds_bytes(rc.K, rc.nt, elem_size) <= kMaxDynamicLds;
    int nb = bands_for(std::max<int64_t>(planes_f, 1), h, 32, 2048);
    int R = (h + nb - 1) / nb;
    R += R & 1;                                        // rows are handled in pairs
    sp.R = std::max(R, 2);
    sp.nb = (h + sp.R - 1) / sp.R;
    return sp;
}

// How much of the band-local integral, counted from its end, is written with the ordinary cache
// policy (the memory-side cache holds 256 MB; the grad-input kernel reads that part first).
inline int64_t cached_tail_bytes() {
    static const int64_t v = [] {
        const char* e = std::getenv("BOXCONV_L_KEEP_MB");
        return static_cast<int64_t>(e != nullptr ? std::max(0, std::atoi(e)) : 192) << 20;
    }();
    return v;
}

template <class T>
hipError_t grad_output_stream_launch(const T* integ, const T* grad_out, BoxParams<T> prm,
                                     double* acc, int acc_slots, T* local_integral,
                                     const StreamPlan& sp, Dims d, bool exact, hipStream_t stream) {
    const int64_t planes_f = d.planes * d.F;
    if (planes_f == 0 || d.hw() == 0) return hipSuccess;
    const bool params = acc != nullptr, scan = local_integral != nullptr;
    if (!sp.usable || (!params && !scan)) return hipErrorInvalidValue;
    SampleArgs<T> a = base_args(prm, d);
    a.src = integ; a.grad_out = grad_out; a.acc = acc; a.acc_slots = acc_slots; a.dst = local_integral;
    if (acc_slots != 0 && acc_slots != sp.nb) return hipErrorInvalidValue;
    a.nb = sp.nb; a.R = sp.R;
    a.keep_tail = scan ? cached_tail_bytes() / kXcds : 0;
    finish_args(a, planes_f * a.nb);
    const RowConfig rc = stream_row_config(d.w);
    const dim3 grid(static_cast<unsigned>(a.per_xcd * kXcds));
    const size_t lds = stream_lds_bytes(rc.K, rc.nt, sizeof(T));
#define LAUNCH_GS(NT, KK, EX, FU) \
    if (params && scan) BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_kernel<T, NT, KK, EX, FU, true, true>), grid, dim3(NT), lds, stream, a); \
    else if (params)    BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_kernel<T, NT, KK, EX, FU, true, false>), grid, dim3(NT), lds, stream, a); \
    else                BOXCONV_LAUNCH("grad_output_stream", (grad_output_stream_kernel<T, NT, KK, EX, FU, false, true>), grid, dim3(NT), lds, stream, a)
    BOXCONV_DISPATCH_SHAPE_EXACT_FULL(LAUNCH_GS, rc, exact)
#undef LAUNCH_GS
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

#define BOXCONV_INSTANTIATE(T)                                                                     \
    template hipError_t grad_input_launch<T>(const T*, int, BoxParams<T>, T*, Dims, bool, bool,    \
                                             hipStream_t, const ParamFinish<T>*, bool*);           \
    template hipError_t grad_output_stream_launch<T>(const T*, const T*, BoxParams<T>, double*, int, \
                                                     T*, const StreamPlan&, Dims, bool,            \
                                                     hipStream_t);                                 \
    template hipError_t grad_params_gather_launch<T>(const T*, const T*, BoxParams<T>, double*,    \
                                                     Dims, bool, hipStream_t);                     \
    template hipError_t grad_params_finish<T>(const ParamFinish<T>&, BoxParams<T>, hipStream_t);

BOXCONV_INSTANTIATE(float)
BOXCONV_INSTANTIATE(double)

}  // namespace boxconv
