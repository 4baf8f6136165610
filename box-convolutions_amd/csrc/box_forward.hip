// Forward box sampling for gfx950: output[p][f] = box sums of integral plane p for box (c, f).
// Replaces cpu::boxConvUpdateOutput, src/box_convolution.cpp:100-261 (CUDA:
// box_convolution_cuda_forward.cu:28-251). The math and the row-streaming scheme are described at
// the top of box_sampling.hip.

#include "box_sampling_common.hpp"

namespace boxconv {

namespace {

// ---------------------------------------------------------------------------------------------
// Forward. Work item = (plane p, filter f, band). blockDim = NT, K >= ceil(w / NT).
// LDS: [2 buffers][w+3] RowPair<T>.
template <class T, int NT, int K, bool EXACT, bool FULL>
__global__ void __launch_bounds__(NT) forward_rows_kernel(SampleArgs<T> a) {
    const unsigned vid = xcd_contiguous_id(a.per_xcd);
    if (vid >= a.total) return;
    const unsigned nbands = a.nb, nfilt = a.F;
    const int band = static_cast<int>(vid % nbands);
    const unsigned pf32 = vid / nbands;
    const int f = static_cast<int>(pf32 % nfilt);
    const int64_t pf = pf32, p = pf32 / nfilt;
    const int k_par = static_cast<int>(static_cast<unsigned>(a.plane0 + p) % static_cast<unsigned>(a.C)) * a.F + f;
    const int h = a.h, w = a.w;
    const unsigned row_bytes = static_cast<unsigned>(w) * sizeof(T);

    const BoxOfWorkgroup<T> bx = load_box(a.prm, k_par);
    const BoxSplit<T> s = split_forward(bx.xmin, bx.xmax, bx.ymin, bx.ymax);
    const T scale = a.normalize
        ? inverse_extent(bx.xmin, bx.xmax, bx.ymin, bx.ymax, EXACT, true, true) : T(1);

    const int64_t pitch = w + 1;
    const T* plane = a.src + p * static_cast<int64_t>(h + 1) * pitch;
    // output rows start one element early so that column slot q = j + 1 lands on pixel j
    const LoadRows<T> irows(plane, pitch, w + 1, h + 1);
    const Rows<T, FULL> orows(a.dst + pf * static_cast<int64_t>(h) * w - 1, w, w + 1, h);
    RowPair<T>* vbuf = reinterpret_cast<RowPair<T>*>(smem_raw);
    const int vlen = w + 3;
    clear_row_pads(vbuf, vlen);

    const int i0 = band * a.R;
    const int i1 = min(h, i0 + a.R);

    const int q1 = lane_q1<T>();
    unsigned lo[K], hi[K];
    column_taps<T, NT, K>(lo, hi, s.ylo, s.yhi, w);

    T ta[K], bc[K];                       // I[t(i-1)], I[b(i)]
    T t0[K], t1[K], b1[K], b2[K];         // I[t(i)], I[t(i+1)], I[b(i+1)], I[b(i+2)]
    load_row<T, NT, K>(irows.row(clampi(i0 + s.xlo - 1, 0, h)), q1, ta);
    load_row<T, NT, K>(irows.row(clampi(i0 + s.xhi, 0, h)), q1, bc);
    load_pair<T, NT, K, FULL>(irows, i0, s.xlo, s.xhi, h, q1, t0, t1, b1, b2);

    // One row pair. PREFETCH and the LDS buffer are compile-time tags: the loop body always
    // issues the next pair's loads and the last pair is peeled, so no branch joins a path with
    // loads in flight to one without (the wait-count insertion would have to drain the prefetch
    // at such a join); the loop is unrolled over both buffers so that LDS addresses are lane
    // constants plus immediates and the sliding rows rotate by renaming instead of moves.
    auto row_pair = [&](int i, auto prefetch_tag, auto flip_tag) {
        constexpr bool PREFETCH = decltype(prefetch_tag)::value;
        constexpr int FLIP = decltype(flip_tag)::value;
        T n0[K] = {}, n1[K] = {}, n2[K] = {}, n3[K] = {};
        if (PREFETCH)
            load_pair<T, NT, K, FULL>(irows, i + 2, s.xlo, s.xhi, h, q1, n0, n1, n2, n3);

        RowPair<T>* V = vbuf + (FLIP ? vlen : 0);
        T v0[K], v1[K];
#pragma unroll
        for (int k = 0; k < K; ++k) {
            v0[k] = blend<T, EXACT>(ta[k], t0[k], bc[k], b1[k], s.fxlo, s.fxhi);
            v1[k] = blend<T, EXACT>(t0[k], t1[k], b1[k], b2[k], s.fxlo, s.fxhi);
        }
        publish_rows<T, NT, K, FULL>(V, v0, v1, w, row_bytes, q1);
        __syncthreads();

        const RowRef ob0 = orows.row(i);
        const RowRef ob1 = orows.row(min(i + 1, h - 1), i + 1 < i1);   // may lie past the band
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (slot_valid<T, NT, FULL>(q1, k, row_bytes)) {
                const RowPair<T> o = sample_columns<T, EXACT>(V, lo[k], hi[k], s.fylo, s.fyhi);
                store_slot<T, NT, kCacheStream>(o.r0 * scale, ob0, q1, k);
                store_slot<T, NT, kCacheStream>(o.r1 * scale, ob1, q1, k);
            }
        }
        if (PREFETCH) {
#pragma unroll
            for (int k = 0; k < K; ++k) {
                ta[k] = t1[k]; bc[k] = b2[k];
                t0[k] = n0[k]; t1[k] = n1[k]; b1[k] = n2[k]; b2[k] = n3[k];
            }
        }
    };
    int i = i0;
    for (; i + 4 < i1; i += 4) {
        row_pair(i, std::true_type{}, Flip0{});
        row_pair(i + 2, std::true_type{}, Flip1{});
    }
    if (i + 2 < i1) {
        row_pair(i, std::true_type{}, Flip0{});
        row_pair(i + 2, std::false_type{}, Flip1{});
    } else {
        row_pair(i, std::false_type{}, Flip0{});
    }
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
    const int k_par = static_cast<int>(static_cast<unsigned>(a.plane0 + p) % static_cast<unsigned>(a.C)) * a.F + static_cast<int>(pf % a.F);
    const BoxOfWorkgroup<T> bx = load_box(a.prm, k_par);
    const BoxSplit<T> s = split_forward(bx.xmin, bx.xmax, bx.ymin, bx.ymax);
    const T scale = a.normalize
        ? inverse_extent(bx.xmin, bx.xmax, bx.ymin, bx.ymax, EXACT, true, true) : T(1);
    const T* plane = a.src + p * static_cast<int64_t>(a.h + 1) * (a.w + 1);
    a.dst[idx] = gather_box<T, EXACT>(plane, s, i, j, a.h, a.w) * scale;
}

}  // namespace

template <class T>
hipError_t forward_launch(const T* integ, BoxParams<T> prm, T* out, Dims d, bool normalize,
                          bool exact, hipStream_t stream) {
    const int64_t planes_f = d.planes * d.F;
    if (planes_f == 0 || d.hw() == 0) return hipSuccess;
    SampleArgs<T> a = base_args(prm, d);
    a.src = integ; a.dst = out; a.normalize = normalize ? 1 : 0;

    if (!row_kernels_apply(d.h, d.w, sizeof(T))) {
        finish_args(a, planes_f * d.hw());
        const dim3 grid(static_cast<unsigned>((a.total + 255) / 256));
        if (exact) BOXCONV_LAUNCH("forward_gather", (forward_gather_kernel<T, true>), grid, dim3(256), 0, stream, a);
        else       BOXCONV_LAUNCH("forward_gather", (forward_gather_kernel<T, false>), grid, dim3(256), 0, stream, a);
        return hipGetLastError();
    }

    static const int fwd_threads = preferred_row_threads("BOXCONV_FWD_THREADS", 512);
    const RowConfig rc = row_config(d.w, fwd_threads);
    a.nb = bands_for(planes_f, d.h, 16, 4096);
    a.R = (d.h + a.nb - 1) / a.nb;
    a.R += a.R & 1;                                   // rows are handled in pairs
    a.nb = (d.h + a.R - 1) / a.R;
    finish_args(a, planes_f * a.nb);
    const dim3 grid(static_cast<unsigned>(a.per_xcd * kXcds));
    const size_t lds = 4 * static_cast<size_t>(d.w + 3) * sizeof(T);
#define LAUNCH_FWD(NT, KK, EX, FU) \
    BOXCONV_LAUNCH("forward_rows", (forward_rows_kernel<T, NT, KK, EX, FU>), grid, dim3(NT), lds, stream, a)
    BOXCONV_DISPATCH_SHAPE_EXACT_FULL(LAUNCH_FWD, rc, exact)
#undef LAUNCH_FWD
    return hipGetLastError();
}

template hipError_t forward_launch<float>(const float*, BoxParams<float>, float*, Dims, bool, bool, hipStream_t);
template hipError_t forward_launch<double>(const double*, BoxParams<double>, double*, Dims, bool, bool, hipStream_t);

}  // namespace boxconv
