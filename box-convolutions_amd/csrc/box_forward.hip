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
//
// TO: element type of the output (T, or a 16-bit type when T is float). TAIL: what happens to a
// box sum S on its way out, fused into the store (inference only, there is no backward for it):
//   y = S * channel_scale[c*F+f] + channel_shift[c*F+f]  (+ residual[same pixel])  (max(y, 0))
// which is the tail of a block such as BoxConv -> BatchNorm (eval) -> residual add -> ReLU.
// Absent pieces are neutral: a null scale/shift reads as 1/0, a null residual as zeros (its row
// descriptors get size 0, so the loads return 0 without a branch).
template <class TO>
struct ForwardTail {
    TO* dst;
    const TO* residual;
    const float* channel_scale;
    const float* channel_shift;
    int relu;
};

template <class T, class TO, int NT, int K, bool EXACT, bool FULL, bool TAIL>
__global__ void __launch_bounds__(NT) forward_rows_kernel(SampleArgs<T> a, ForwardTail<TO> tl) {
    const unsigned vid = xcd_contiguous_id(a.per_xcd);
    if (vid >= a.total) return;
    const unsigned nbands = a.nb, nfilt = a.F;
    // (plane, filter, band) order, or (plane, band, filter): see forward_launch_any
    const unsigned inner = a.band_major ? nfilt : nbands, outer = a.band_major ? nbands : nfilt;
    const unsigned v_in = vid % inner, v_rest = vid / inner;
    const unsigned v_out = v_rest % outer, p32 = v_rest / outer;
    const int band = static_cast<int>(a.band_major ? v_out : v_in);
    const int f = static_cast<int>(a.band_major ? v_in : v_out);
    const int64_t p = p32, pf = p * nfilt + f;
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
    const Rows<TO, FULL> orows(tl.dst + pf * static_cast<int64_t>(h) * w - 1, w, w + 1, h);
    const Rows<const TO, false> rrows((tl.residual != nullptr ? tl.residual : tl.dst) +
                                          pf * static_cast<int64_t>(h) * w - 1,
                                      w, tl.residual != nullptr ? w + 1 : 0, h);
    T ch_scale = T(1), ch_shift = T(0);
    if (TAIL) {
        if (tl.channel_scale != nullptr) ch_scale = static_cast<T>(tl.channel_scale[k_par]);
        if (tl.channel_shift != nullptr) ch_shift = static_cast<T>(tl.channel_shift[k_par]);
    }
    const bool relu = TAIL && tl.relu != 0;
    RowPair<T>* vbuf = reinterpret_cast<RowPair<T>*>(smem_raw);
    const int vlen = w + 3;
    clear_row_pads(vbuf, vlen);

    const int i0 = band * a.R;
    const int i1 = min(h, i0 + a.R);

    const int q1 = lane_q1<T>();
    const int qo = lane_q1<TO>();         // the same column slots in a row of TO
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

        // residual of the two output rows: issued with the row loads, used after the barrier
        TO res0[K] = {}, res1[K] = {};
        if (TAIL) {
            const RowRef rb0 = rrows.row(i);
            const RowRef rb1 = rrows.row(min(i + 1, h - 1), i + 1 < i1);
#pragma unroll
            for (int k = 0; k < K; ++k) {
                res0[k] = load_slot<TO, NT, kCacheStream>(rb0, qo, k);
                res1[k] = load_slot<TO, NT, kCacheStream>(rb1, qo, k);
            }
        }

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
                T y0 = o.r0 * scale, y1 = o.r1 * scale;
                if (TAIL) {
                    y0 = y0 * ch_scale + ch_shift + static_cast<T>(widen(res0[k]));
                    y1 = y1 * ch_scale + ch_shift + static_cast<T>(widen(res1[k]));
                    if (relu) { y0 = y0 < T(0) ? T(0) : y0; y1 = y1 < T(0) ? T(0) : y1; }
                }
                TO z0, z1;
                narrow(y0, z0);
                narrow(y1, z1);
                if (a.stream_out) {                      // (workgroup-uniform)
                    store_slot<TO, NT, kCacheStream>(z0, ob0, qo, k);
                    store_slot<TO, NT, kCacheStream>(z1, ob1, qo, k);
                } else {
                    store_slot<TO, NT, kCacheDefault>(z0, ob0, qo, k);
                    store_slot<TO, NT, kCacheDefault>(z1, ob1, qo, k);
                }
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

template <class T, class TO, bool EXACT, bool TAIL>
__global__ void __launch_bounds__(256) forward_gather_kernel(SampleArgs<T> a, ForwardTail<TO> tl) {
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
    T y = gather_box<T, EXACT>(plane, s, i, j, a.h, a.w) * scale;
    if (TAIL) {
        const T ch_scale = tl.channel_scale != nullptr ? static_cast<T>(tl.channel_scale[k_par]) : T(1);
        const T ch_shift = tl.channel_shift != nullptr ? static_cast<T>(tl.channel_shift[k_par]) : T(0);
        const T res = tl.residual != nullptr ? static_cast<T>(widen(tl.residual[idx])) : T(0);
        y = y * ch_scale + ch_shift + res;
        if (tl.relu != 0 && y < T(0)) y = T(0);
    }
    narrow(y, tl.dst[idx]);
}

}  // namespace

// TAIL selects the kernels with the fused tail; without it only tail.dst is used.
template <class T, class TO, bool TAIL>
hipError_t forward_launch_any(const T* integ, BoxParams<T> prm, ForwardTail<TO> tail, Dims d,
                              bool normalize, bool exact, hipStream_t stream) {
    const int64_t planes_f = d.planes * d.F;
    if (planes_f == 0 || d.hw() == 0) return hipSuccess;
    SampleArgs<T> a = base_args(prm, d);
    a.src = integ; a.normalize = normalize ? 1 : 0;

    // (the row kernel keeps two row pairs of w + 3 columns in LDS, up to 64 KiB + 48 bytes for the
    // widest rows it takes; a device that grants a workgroup less goes to the gather kernel)
    if (!row_kernels_apply(d.h, d.w, sizeof(T)) ||
        4 * static_cast<size_t>(d.w + 3) * sizeof(T) > std::min(kMaxDynamicLds, device_lds_limit())) {
        finish_args(a, planes_f * d.hw());
        const dim3 grid(static_cast<unsigned>((a.total + 255) / 256));
        if (exact) BOXCONV_LAUNCH("forward_gather", (forward_gather_kernel<T, TO, true, TAIL>), grid, dim3(256), 0, stream, a, tail);
        else       BOXCONV_LAUNCH("forward_gather", (forward_gather_kernel<T, TO, false, TAIL>), grid, dim3(256), 0, stream, a, tail);
        return hipGetLastError();
    }

    const RowConfig rc = row_config(d.w, switches().fwd_threads);
    // Many short-lived workgroups (bands of 8 rows at the headline size): the kernel then ends
    // with a short tail. Measured per step: 16 workgroup-waves' worth of bands 0.501 ms, 8 0.508 ms,
    // 4 0.517 ms, 32 (bands of 4 rows, too much halo) 0.523 ms.
    a.nb = bands_for(planes_f, d.h, 8, 16384);
    a.R = (d.h + a.nb - 1) / a.nb;
    a.R += a.R & 1;                                   // rows are handled in pairs
    a.nb = (d.h + a.R - 1) / a.R;
    finish_args(a, planes_f * a.nb);
    // An integral plane that does not fit an XCD's 4 MB L2 is streamed from memory once per filter
    // when the bands of one filter run one after the other; with the filters of a band side by
    // side their rows (a box height apart at most) are fetched together (1024 x 2048 with two
    // filters: 737 -> 703 us). Planes that fit are faster in filter order (512 x 1024: 97 vs 100 us).
    a.band_major = (static_cast<uint64_t>(d.h + 1) * (d.w + 1) * sizeof(T) > (4u << 20)) ? 1 : 0;
    // The output is written once and not read again by this pass: non-temporal stores keep it out
    // of the way of the integral rows in the caches (512 x 1024, 16 x 8 planes: 97 against 130 us,
    // and the grad-input pass that follows 121 against 132). A lane stores one element per
    // instruction, though, and where rows do not start on 64-byte boundaries such stores reach
    // memory as partly covered 32-byte sectors that nothing merges any more: 256 x 132, 16 x 64
    // planes, 61 against 37 us; 256 x 300 51 against 38. Such rows keep the ordinary policy while
    // the output fits the memory-side cache; beyond that the streaming policy wins even so
    // (500 x 1000, 512 MB: 128 against 142 us, and the next pass 122 against 138).
    const uint64_t out_bytes = static_cast<uint64_t>(planes_f) * d.hw() * sizeof(TO);
    a.stream_out = ((static_cast<uint64_t>(d.w) * sizeof(TO)) % 64 == 0 || out_bytes > (256ull << 20)) ? 1 : 0;
    const dim3 grid(static_cast<unsigned>(a.per_xcd * kXcds));
    const size_t lds = 4 * static_cast<size_t>(d.w + 3) * sizeof(T);
#define LAUNCH_FWD(NT, KK, EX, FU) \
    BOXCONV_LAUNCH("forward_rows", (forward_rows_kernel<T, TO, NT, KK, EX, FU, TAIL>), grid, dim3(NT), lds, stream, a, tail)
    BOXCONV_DISPATCH_SHAPE_EXACT_FULL(LAUNCH_FWD, rc, exact)
#undef LAUNCH_FWD
    return hipGetLastError();
}

template <class T>
hipError_t forward_launch(const T* integ, BoxParams<T> prm, T* out, Dims d, bool normalize,
                          bool exact, hipStream_t stream) {
    return forward_launch_any<T, T, false>(integ, prm, ForwardTail<T>{out, nullptr, nullptr, nullptr, 0},
                                           d, normalize, exact, stream);
}

template <class TO>
hipError_t forward_fused_launch(const float* integ, BoxParams<float> prm, TO* out, const TO* residual,
                                const float* channel_scale, const float* channel_shift, bool relu,
                                Dims d, bool normalize, bool exact, hipStream_t stream) {
    const ForwardTail<TO> tail{out, residual, channel_scale, channel_shift, relu ? 1 : 0};
    if (residual == nullptr && channel_scale == nullptr && channel_shift == nullptr && !relu)
        return forward_launch_any<float, TO, false>(integ, prm, tail, d, normalize, exact, stream);
    return forward_launch_any<float, TO, true>(integ, prm, tail, d, normalize, exact, stream);
}

template hipError_t forward_launch<float>(const float*, BoxParams<float>, float*, Dims, bool, bool, hipStream_t);
template hipError_t forward_launch<double>(const double*, BoxParams<double>, double*, Dims, bool, bool, hipStream_t);
#define BOXCONV_INSTANTIATE_FUSED(TO)                                                              \
    template hipError_t forward_fused_launch<TO>(const float*, BoxParams<float>, TO*, const TO*,   \
                                                 const float*, const float*, bool, Dims, bool,     \
                                                 bool, hipStream_t);
BOXCONV_INSTANTIATE_FUSED(float)
BOXCONV_INSTANTIATE_FUSED(f16_t)
BOXCONV_INSTANTIATE_FUSED(bf16_t)

}  // namespace boxconv
