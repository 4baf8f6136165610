// Integral image (2-D inclusive prefix sum with a zero first row and column) for gfx950.
//
// Replaces reference src/integral_image.cpp:8-39 (CPU) / src/integral_image_cuda.cu:67-173.
// out[p][r+1][c+1] = sum_{i<=r, j<=c} in[p][i][j], out[p][0][*] = out[p][*][0] = 0.
//
// Decomposition. A plane is cut into horizontal bands of R rows; one workgroup owns one band at
// full width, so the only dependency between workgroups is "everything above my band", a vector
// of w column sums. That dependency is resolved without any inter-workgroup waiting by three
// stream-ordered launches:
//   1. band_colsum_kernel  : column sums of every band but the last  -> aux[p][band][c]
//   2. band_prefix_kernel  : running sum of aux over bands (in place) -> sum of all bands above
//   3. band_scan_kernel    : per band, rows top to bottom: column accumulators (registers) +=
//                            input row, then a row-direction prefix of the accumulators.
// With a single band (tall enough grid without cutting) only launch 3 runs. Rows of at most 4096
// columns use band_scan_rows_kernel for launch 3, which adds up the bands above itself (no launch
// 2). For float rows that fill a workgroup exactly and planes of at most 16 bands of 32 rows, one
// kernel does everything in a single pass over the input (band_scan_lookback_kernel): workgroups
// hand their column sums to the ones below them, with a bounded wait. Planes of at most 192 rows
// and 256 columns take plane_scan_kernel: the bands of a plane are the waves of one workgroup,
// which hand their sums over through LDS.
//
// Arithmetic. All sums are carried in double and rounded once on store, so every stored value
// is the correctly rounded exact sum (the CPU reference carries row sums in double as well but
// rounds the column carry every row; this is at least as accurate).
//
// Memory. Loads are 4 consecutive elements per lane (16 B for float, coalesced across the wave).
// The output pitch w+1 is odd, so results are staged through LDS and written as consecutive
// dwords per lane (256 B contiguous per wave instruction).

#include <cstdlib>
#include <type_traits>

#include "boxconv_device.hpp"
#include "boxconv_host.hpp"

namespace boxconv {

namespace {

template <class T>
struct alignas(4 * sizeof(T)) Vec4 { T v[4]; };

// ---- pass 1 -----------------------------------------------------------------------------------
// One workgroup per (plane, band, strip of 1024 columns); lane `tid` owns 4 consecutive columns
// and keeps 8 row loads in flight. VEC: rows are 16-byte aligned and w is a multiple of 4.
// TI: element type of the input (T, or a 16-bit type widened to T = float on load).
template <class T, class TI, bool VEC>
__global__ void __launch_bounds__(256)
band_colsum_kernel(const TI* __restrict__ in, double* __restrict__ aux, int h, int w, int nb,
                   int R, int strips) {
    constexpr int U = 8;
    unsigned blk = blockIdx.x;                      // (p * (nb-1) + band) * strips + strip
    const int strip = static_cast<int>(blk % static_cast<unsigned>(strips));
    blk /= static_cast<unsigned>(strips);
    const int band = static_cast<int>(blk % static_cast<unsigned>(nb - 1));
    const int64_t p = blk / static_cast<unsigned>(nb - 1);
    const int r0 = band * R;
    const int r1 = min(h, r0 + R);
    const int c0 = strip * 1024 + 4 * static_cast<int>(threadIdx.x);
    const TI* src = in + p * static_cast<int64_t>(h) * w;
    const Rows<const TI, false> irows(src, w, w, h);
    const int off = c0 * static_cast<int>(sizeof(TI));

    double acc[4] = {0.0, 0.0, 0.0, 0.0};
    for (int r = r0; r < r1; r += U) {
        T x[U][4];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (VEC) {
#pragma unroll
                for (int v = 0; v < 4; ++v) x[u][v] = T(0);
                if (r + u < r1 && c0 < w) load_quad(src + static_cast<int64_t>(r + u) * w + c0, x[u]);
            } else {
                buffer_load_run_as<kCacheDefault, TI>(x[u], irows.row(min(r + u, h - 1), r + u < r1), off);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[v] += static_cast<double>(x[u][v]);
    }
    double* dst = aux + static_cast<int64_t>(blk) * w;
#pragma unroll
    for (int v = 0; v < 4; ++v)
        if (c0 + v < w) dst[c0 + v] = acc[v];
}

// ---- pass 2 -----------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
band_prefix_kernel(double* __restrict__ aux, int64_t planes, int w, int nb) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= planes * w) return;
    const int64_t p = idx / w;
    const int c = static_cast<int>(idx % w);
    double* col = aux + p * static_cast<int64_t>(nb - 1) * w + c;
    double run = col[0];
    for (int k = 1; k < nb - 1; ++k) {
        run += col[static_cast<int64_t>(k) * w];
        col[static_cast<int64_t>(k) * w] = run;
    }
}

// ---- pass 3 -----------------------------------------------------------------------------------
// WAVES*64 threads; a "chunk" is WAVES*256 consecutive columns (4 per lane); M chunks cover the
// tile of columns this launch handles per row; RB rows are in flight together.
template <class T, int WAVES, int M, int RB, bool VEC>
__global__ void __launch_bounds__(WAVES * 64)
band_scan_kernel(const T* __restrict__ in, T* __restrict__ out, const double* __restrict__ aux,
                 int h, int w, int nb, int R, int64_t total, int64_t per_xcd, int reverse) {
    constexpr int NT = WAVES * 64;
    constexpr int CW = NT * 4;          // columns per chunk
    constexpr int TW = CW * M;          // columns per tile

    __shared__ double wave_tot[RB][M][WAVES];
    __shared__ __align__(32) T stage[RB][TW];
    __shared__ double row_carry[256];   // prefix of each band row up to the current tile; R <= 256

    unsigned blk = xcd_contiguous_id(per_xcd);    // p * nb + band
    if (blk >= total) return;
    if (reverse) blk = static_cast<unsigned>(total) - 1u - blk;
    const int band = static_cast<int>(blk % static_cast<unsigned>(nb));
    const int64_t p = blk / static_cast<unsigned>(nb);
    const int r0 = band * R;
    const int r1 = min(h, r0 + R);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keep it scalar
    const int64_t W1 = static_cast<int64_t>(w) + 1;

    const T* src = in + p * static_cast<int64_t>(h) * w;
    T* dst = out + p * static_cast<int64_t>(h + 1) * W1;
    const double* above = (band > 0)
        ? aux + (p * static_cast<int64_t>(nb - 1) + (band - 1)) * static_cast<int64_t>(w)
        : nullptr;

    if (band == 0)
        for (int c = tid; c <= w; c += NT) dst[c] = T(0);
    for (int r = tid; r < r1 - r0; r += NT) row_carry[r] = 0.0;
    __syncthreads();

    for (int c0 = 0; c0 < w; c0 += TW) {
        // column accumulators for this tile start at the sum of all bands above
        double colacc[M][4];
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int c = c0 + m * CW + 4 * tid + v;
                colacc[m][v] = (above != nullptr && c < w) ? above[c] : 0.0;
            }

        for (int rbase = r0; rbase < r1; rbase += RB) {
            // -- issue all loads of the batch
            T x[RB][M][4];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const int row = rbase + rb;
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    const int c = c0 + m * CW + 4 * tid;
                    if (VEC) {
                        Vec4<T> q = {{T(0), T(0), T(0), T(0)}};
                        if (row < r1 && c < w)
                            q = *reinterpret_cast<const Vec4<T>*>(src + static_cast<int64_t>(row) * w + c);
#pragma unroll
                        for (int v = 0; v < 4; ++v) x[rb][m][v] = q.v[v];
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            x[rb][m][v] = (row < r1 && c + v < w)
                                ? src[static_cast<int64_t>(row) * w + c + v] : T(0);
                    }
                }
            }

            // -- accumulate down the rows, prefix inside the lane, scan across the wave
            double pre[RB][M][4];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    double run = 0.0;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        colacc[m][v] += static_cast<double>(x[rb][m][v]);
                        run += colacc[m][v];
                        pre[rb][m][v] = run;            // inclusive within the lane
                    }
                    const double incl = wave_inclusive_scan(run);
                    const double excl = incl - run;     // lanes to the left, this wave
#pragma unroll
                    for (int v = 0; v < 4; ++v) pre[rb][m][v] += excl;
                    if (lane == 63) wave_tot[rb][m][wave] = incl;
                }
            __syncthreads();

            // -- add waves/chunks to the left and the tiles to the left; stage as T
            double tile_end[RB];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const int row = rbase + rb;
                double left = (row < r1) ? row_carry[row - r0] : 0.0;
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    double mine = left;
#pragma unroll
                    for (int wv = 0; wv < WAVES; ++wv) {
                        const double t = wave_tot[rb][m][wv];
                        if (wv < wave) mine += t;
                        left += t;
                    }
                    Vec4<T> q;
#pragma unroll
                    for (int v = 0; v < 4; ++v) q.v[v] = static_cast<T>(mine + pre[rb][m][v]);
                    *reinterpret_cast<Vec4<T>*>(&stage[rb][m * CW + 4 * tid]) = q;
                }
                tile_end[rb] = left;        // row prefix through the end of this tile
            }
            __syncthreads();
            if (tid == 0 && c0 + TW < w) {
#pragma unroll
                for (int rb = 0; rb < RB; ++rb)
                    if (rbase + rb < r1) row_carry[rbase + rb - r0] = tile_end[rb];
            }

            // -- coalesced stores: lane-consecutive dwords into the (w+1)-pitched output
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const int row = rbase + rb;
                if (row < r1) {
                    T* orow = dst + static_cast<int64_t>(row + 1) * W1;
                    const int lim = min(TW, w - c0);
                    for (int i = tid; i < lim; i += NT) orow[c0 + i + 1] = stage[rb][i];
                    if (c0 == 0 && tid == 0) orow[0] = T(0);
                }
            }
            __syncthreads();
        }
    }
}

// ---- pass 3, rows no wider than one tile --------------------------------------------------------
// WAVES*64 threads, lane `tid` owns the 4 consecutive columns 4*tid .. 4*tid+3, so a row of up to
// WAVES*256 columns is one tile. Differences to band_scan_kernel: `aux` holds the plain per-band
// column sums (the sum over the bands above is formed here, no band_prefix pass); the loads of the
// next RB rows are in flight while the current ones are scanned; there is one barrier per RB rows
// (wave totals, double-buffered) and results are stored straight from registers, 4 consecutive
// elements per lane. VEC: rows are 16-byte aligned and w is a multiple of 4. FULL: w == 4 * threads.
template <class T, class TI, int WAVES, int RB, bool VEC, bool FULL>
__global__ void __launch_bounds__(WAVES * 64)
band_scan_rows_kernel(const TI* __restrict__ in, T* __restrict__ out, const double* __restrict__ aux,
                      int h, int w, int nb, int R, int64_t total, int64_t per_xcd, int reverse) {
    constexpr int NT = WAVES * 64;
    __shared__ double wave_tot[2][RB][WAVES];

    unsigned blk = xcd_contiguous_id(per_xcd);    // p * nb + band
    if (blk >= total) return;
    if (reverse) blk = static_cast<unsigned>(total) - 1u - blk;
    const int band = static_cast<int>(blk % static_cast<unsigned>(nb));
    const int64_t p = blk / static_cast<unsigned>(nb);
    const int r0 = band * R;
    const int r1 = min(h, r0 + R);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keep it scalar
    const int64_t W1 = static_cast<int64_t>(w) + 1;
    const int c0 = 4 * tid;                       // first of the lane's columns

    const TI* src = in + p * static_cast<int64_t>(h) * w;
    const Rows<const TI, false> irows(src, w, w, h);
    T* dst = out + p * static_cast<int64_t>(h + 1) * W1;
    const Rows<T, FULL> orows(dst, W1, w + 1, h + 1);
    const int in_off = c0 * static_cast<int>(sizeof(TI));
    const int out_off = (c0 + 1) * static_cast<int>(sizeof(T));

    if (band == 0)
        for (int c = tid; c <= w; c += NT) dst[c] = T(0);

    // column accumulators start at the sum of all bands above
    double colacc[4] = {0.0, 0.0, 0.0, 0.0};
    {
        const Rows<const double, false> arows(aux + p * static_cast<int64_t>(nb - 1) * w, w, w, max(nb - 1, 1));
        for (int b = 0; b < band; ++b) {
            double part[4];
            buffer_load_run<kCacheDefault>(part, arows.row(b), c0 * 8);
#pragma unroll
            for (int v = 0; v < 4; ++v) colacc[v] += part[v];
        }
    }

    auto load_batch = [&](int rbase, T (&x)[RB][4]) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const int row = rbase + rb;
            if (VEC) {
#pragma unroll
                for (int v = 0; v < 4; ++v) x[rb][v] = T(0);
                if (row < r1 && c0 < w) load_quad(src + static_cast<int64_t>(row) * w + c0, x[rb]);
            } else {
                buffer_load_run_as<kCacheStream, TI>(x[rb], irows.row(min(row, h - 1), row < r1), in_off);
            }
        }
    };

    T x[RB][4];
    load_batch(r0, x);
    int buf = 0;
    for (int rbase = r0; rbase < r1; rbase += RB) {
        T nx[RB][4];
        load_batch(rbase + RB, nx);               // rows past the band come back as zeros, unread

        double pre[RB][4], excl[RB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            double run = 0.0;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                colacc[v] += static_cast<double>(x[rb][v]);
                run += colacc[v];
                pre[rb][v] = run;                 // inclusive within the lane
            }
            const double incl = wave_inclusive_scan(run);
            excl[rb] = incl - run;                // lanes to the left, this wave
            if (lane == 63) wave_tot[buf][rb][wave] = incl;
        }
        __syncthreads();
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const int row = rbase + rb;
            double left = excl[rb];
#pragma unroll
            for (int wv = 0; wv < WAVES - 1; ++wv)
                if (wv < wave) left += wave_tot[buf][rb][wv];      // scalar condition
            T res[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) res[v] = static_cast<T>(left + pre[rb][v]);
            const RowRef orow = orows.row(min(row + 1, h), row < r1);
            buffer_store_run<kCacheDefault, FULL>(res, orow, out_off, (w + 1) * static_cast<int>(sizeof(T)));
            if (tid == 0 && row < r1) dst[static_cast<int64_t>(row + 1) * W1] = T(0);
        }
        buf ^= 1;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int v = 0; v < 4; ++v) x[rb][v] = nx[rb][v];
    }
}

// ---- single pass, rows no wider than one tile and bands of at most 32 rows ----------------------
// Same tiling as band_scan_rows_kernel, but the input is read exactly once: a workgroup first
// loads its whole band into registers and publishes the band's column sums in `aux`, then collects
// the column sums of the bands above it in the same plane and scans its rows out of the registers.
//
// Hand-over. `aux` is filled with a marker value before the launch (fill_marker_kernel); every
// column sum is published with one 64-bit device-scope atomic store and collected with 64-bit
// device-scope atomic loads that are repeated while they return the marker. Data and "ready" are
// the same memory word, so no ordering between different locations (no fence, no cache
// write-back or invalidation) is needed. The marker is a NaN whose low mantissa bits are set: a sum
// of floats converted to double can be a NaN only with a payload that came from a float, whose
// low 29 bits are zero, so no published value equals the marker.
//
// Progress. A workgroup publishes before it collects and publishing depends on nothing, so a
// collecting workgroup only needs the workgroups of the bands above to have been started. Those
// have lower workgroup ids on the same XCD (per_xcd is a multiple of nb, so a plane never
// straddles two XCDs) and workgroups of one XCD are started in id order. The wait is nevertheless
// bounded: after `spin_limit` rounds of loads a lane sums the band's input rows for its own
// columns instead, which gives the same value bit for bit (same rows, same order, double
// accumulation). A launch therefore terminates and is correct whatever the start order;
// spin_limit = 0 takes that path for every band (used by the tests).
constexpr int kLookbackRows = 32;     // band height limit: 32 rows x 4 columns per lane in registers
constexpr int kLookbackBands = 64;
constexpr unsigned long long kNotPublished = 0x7ff8deadbeef0001ull;
// Scopes of the hand-over. All bands of a plane run on one XCD (see Progress below), so the
// words only have to meet in that XCD's L2. The stores have workgroup scope: plain writes into the
// L2 (the vector L1 is write-through); at agent scope every 8-byte store went through to memory
// as a 32-byte write (measured: 16 MB of extra HBM writes per 4 MB of sums). The loads keep agent
// scope, which is what makes them bypass the vector L1 (a workgroup-scope load may hit there and
// would poll a stale line until its wait runs out). Should a publisher ever run on another XCD,
// its words reach the poller late or never; the bounded wait then ends in the local
// re-summation: slower, never wrong.
// Hand-over words per band of a plane: four for every lane of the workgroup, whole waves of 256 columns.
inline int64_t lookback_row_words(int w) { return static_cast<int64_t>((w + 255) / 256) * 256; }
constexpr int kPublishScope = __HIP_MEMORY_SCOPE_WORKGROUP;
constexpr int kCollectScope = __HIP_MEMORY_SCOPE_AGENT;

__global__ void __launch_bounds__(256) fill_marker_kernel(unsigned long long* dst, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) dst[i] = kNotPublished;
}

// The same fill with a clip job on the side (its first clip_blocks workgroups): what a
// training-mode forward does before the integral image, in one launch.
template <class T>
__global__ void __launch_bounds__(256)
clip_and_fill_marker_kernel(ClipArgs<T> clip, int clip_blocks, unsigned long long* dst, int64_t n) {
    if (static_cast<int>(blockIdx.x) < clip_blocks) {
        const int i = blockIdx.x * 256 + threadIdx.x;
        if (i < clip.n) clip_box(clip, i);
        return;
    }
    const int64_t i = static_cast<int64_t>(blockIdx.x - clip_blocks) * 256 + threadIdx.x;
    if (i < n) dst[i] = kNotPublished;
}

template <class TI, int WAVES, int RB, bool VEC, bool FULL>
__global__ void __launch_bounds__(WAVES * 64)
band_scan_lookback_kernel(const TI* __restrict__ in, float* __restrict__ out, double* aux,
                          int h, int w, int nb, int R, int64_t planes, int64_t per_xcd,
                          int reverse, int spin_limit) {
    using T = float;
    constexpr int NT = WAVES * 64;
    constexpr int RMAX = kLookbackRows;
    __shared__ double wave_tot[2][RB][WAVES];

    const unsigned blk = xcd_contiguous_id(per_xcd);    // p * nb + band, bands of a plane in order
    const int band = static_cast<int>(blk % static_cast<unsigned>(nb));
    int64_t p = blk / static_cast<unsigned>(nb);
    if (p >= planes) return;
    if (reverse) p = planes - 1 - p;
    const int r0 = band * R;
    const int r1 = min(h, r0 + R);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t W1 = static_cast<int64_t>(w) + 1;
    const int c0 = 4 * tid;

    const TI* src = in + p * static_cast<int64_t>(h) * w;
    const Rows<const TI, false> irows(src, w, w, h);
    T* dst = out + p * static_cast<int64_t>(h + 1) * W1;
    const Rows<T, FULL> orows(dst, W1, w + 1, h + 1);
    // [nb-1][4][NT]: word v of lane t at v * NT + t, so that a wave's load or store of one word
    // per lane covers 512 consecutive bytes (with the four words of a lane side by side every such
    // instruction touched 16 cache lines for 512 bytes, and the look-back's requests outnumbered
    // those of the band itself)
    unsigned long long* sums = reinterpret_cast<unsigned long long*>(aux) +
                               p * static_cast<int64_t>(nb - 1) * (4 * NT) + tid;
    const int in_off = c0 * static_cast<int>(sizeof(TI));
    const int out_off = (c0 + 1) * static_cast<int>(sizeof(T));

    // Loads are unconditional (a clamped address, the value dropped afterwards) so that all rows
    // of the band are in flight together; the row address is wave-uniform, the lane part 32 bits.
    const bool lane_in = c0 < w;
    const unsigned lane_col = lane_in ? static_cast<unsigned>(c0) : 0u;
    auto load_row = [&](int row, bool exists, T (&x)[4]) {
        if (VEC) {
            const TI* rowp = src + static_cast<int64_t>(min(row, h - 1)) * w;
            load_quad(rowp + lane_col, x);
            if (!(exists && lane_in)) {
#pragma unroll
                for (int v = 0; v < 4; ++v) x[v] = T(0);
            }
        } else {
            buffer_load_run_as<kCacheStream, TI>(x, irows.row(min(row, h - 1), exists), in_off);
        }
    };

    // -- the whole band into registers, its column sums published
    T x[RMAX][4];
#pragma unroll
    for (int r = 0; r < RMAX; ++r) load_row(r0 + r, r < R && r0 + r < r1, x[r]);

    if (band == 0)
        for (int c = tid; c <= w; c += NT) dst[c] = T(0);

    if (band < nb - 1) {
        double own[4] = {0.0, 0.0, 0.0, 0.0};
#pragma unroll
        for (int r = 0; r < RMAX; ++r)
#pragma unroll
            for (int v = 0; v < 4; ++v) own[v] += static_cast<double>(x[r][v]);
        unsigned long long* mine = sums + static_cast<int64_t>(band) * (4 * NT);
#pragma unroll
        for (int v = 0; v < 4; ++v)      // (lanes past the row's end publish the zeros they hold)
            __hip_atomic_store(mine + v * NT, static_cast<unsigned long long>(__double_as_longlong(own[v])),
                               __ATOMIC_RELAXED, kPublishScope);
    }

    // -- column sums of the bands above, four bands per round trip: the first loads of a group
    // are all in flight together; a band that was not published yet is then waited for on its own.
    // (Measured no faster: groups of eight bands, and two groups in flight with the next one's
    // loads issued before the current one is waited for, whose registers also cost the workgroups
    // of four waves a wave per SIMD. What the hand-over costs is the wait for the bands above to
    // have read their rows, not the round trips: with the collection left out the kernel takes
    // 0.77 to 0.85 of its time.)
    double colacc[4] = {0.0, 0.0, 0.0, 0.0};
    constexpr int GROUP = 4;
    for (int b0 = 0; b0 < band; b0 += GROUP) {
        unsigned long long bits[GROUP][4];
        bool have[GROUP];
#pragma unroll
        for (int u = 0; u < GROUP; ++u) {
            have[u] = false;
#pragma unroll
            for (int v = 0; v < 4; ++v) bits[u][v] = 0ull;
            if (b0 + u < band && spin_limit > 0) {
                const unsigned long long* theirs = sums + static_cast<int64_t>(b0 + u) * (4 * NT);
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    bits[u][v] = __hip_atomic_load(theirs + v * NT, __ATOMIC_RELAXED, kCollectScope);
            }
        }
#pragma unroll
        for (int u = 0; u < GROUP; ++u) {
            const int b = b0 + u;
            if (b >= band) break;
            if (spin_limit > 0) {
                have[u] = true;
#pragma unroll
                for (int v = 0; v < 4; ++v) have[u] = have[u] && bits[u][v] != kNotPublished;
            }
            const unsigned long long* theirs = sums + static_cast<int64_t>(b) * (4 * NT);
            for (int it = 1; it < spin_limit && !have[u]; ++it) {
                __builtin_amdgcn_s_sleep(8);
                have[u] = true;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    bits[u][v] = __hip_atomic_load(theirs + v * NT, __ATOMIC_RELAXED, kCollectScope);
                    have[u] = have[u] && bits[u][v] != kNotPublished;
                }
            }
            if (have[u]) {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    colacc[v] += __longlong_as_double(static_cast<long long>(bits[u][v]));
            } else {
                double part[4] = {0.0, 0.0, 0.0, 0.0};
                for (int r = b * R; r < (b + 1) * R; ++r) {      // bands above are complete bands
                    T t[4];
                    load_row(r, true, t);
#pragma unroll
                    for (int v = 0; v < 4; ++v) part[v] += static_cast<double>(t[v]);
                }
#pragma unroll
                for (int v = 0; v < 4; ++v) colacc[v] += part[v];
            }
        }
    }

    // -- scan the rows out of the registers, RB at a time (one barrier per batch)
#pragma unroll
    for (int bi = 0; bi < RMAX / RB; ++bi) {
        if (bi * RB >= R) break;
        const int buf = bi & 1;
        double pre[RB][4], excl[RB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            double run = 0.0;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                colacc[v] += static_cast<double>(x[bi * RB + rb][v]);
                run += colacc[v];
                pre[rb][v] = run;
            }
            const double incl = wave_inclusive_scan(run);
            excl[rb] = incl - run;
            if (lane == 63) wave_tot[buf][rb][wave] = incl;
        }
        __syncthreads();
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const int row = r0 + bi * RB + rb;
            double left = excl[rb];
#pragma unroll
            for (int wv = 0; wv < WAVES - 1; ++wv)
                if (wv < wave) left += wave_tot[buf][rb][wv];
            T res[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) res[v] = static_cast<T>(left + pre[rb][v]);
            const RowRef orow = orows.row(min(row + 1, h), row < r1);
            // (FULL: the rows are addressed by offset into one descriptor for the plane, without a
            // bounds check of their own, so a lane past the row's end must not store)
            if (!FULL || lane_in)
                buffer_store_run<kCacheDefault, FULL>(res, orow, out_off, (w + 1) * static_cast<int>(sizeof(T)));
            if (tid == 0 && row < r1) dst[static_cast<int64_t>(row + 1) * W1] = T(0);
        }
    }
}

// ---- single pass, a whole plane per workgroup ---------------------------------------------------
// Planes of at most 256 columns and 192 rows: wave b of the workgroup owns band b of the plane at
// full width (a row is one wave, four columns per lane), so the bands of a plane meet in one
// workgroup and hand their column sums over through LDS with one barrier: one launch, the input
// read once, nothing in global memory besides input and output, no waiting between workgroups.
// The arithmetic is that of band_scan_lookback_kernel with one wave per row: the band's rows in
// registers, double column sums added in band order, rows scanned out of the registers.
constexpr int kPlaneWaves = 8;        // bands per plane at most
constexpr int kPlaneRows = 24;        // rows per band at most (registers: 4 x 24 floats per lane without spilling)
constexpr int kPlaneMaxRows = kPlaneWaves * kPlaneRows, kPlaneMaxCols = 256;

template <class TI, int RMAX, bool VEC>
__global__ void __launch_bounds__(kPlaneWaves * 64)
plane_scan_kernel(const TI* __restrict__ in, float* __restrict__ out, int h, int w, int R, int64_t planes,
                  int reverse, ClipArgs<float> clip, int clip_blocks) {
    using T = float;
    constexpr int RB = 4;
    __shared__ double sums[kPlaneWaves][4][64];

    // a clip job on the side (its first clip_blocks workgroups): what a training-mode forward does
    // before the integral image, in the same launch
    if (static_cast<int>(blockIdx.x) < clip_blocks) {
        const int i = blockIdx.x * blockDim.x + threadIdx.x;
        if (i < clip.n) clip_box(clip, i);
        return;
    }
    int64_t p = blockIdx.x - clip_blocks;
    if (reverse) p = planes - 1 - p;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int band = __builtin_amdgcn_readfirstlane(tid >> 6);     // one wave per band
    const int r0 = band * R;
    const int r1 = min(h, r0 + R);                                  // (every wave of the launch has rows)
    const int64_t W1 = static_cast<int64_t>(w) + 1;
    const int c0 = 4 * lane;

    const TI* src = in + p * static_cast<int64_t>(h) * w;
    const Rows<const TI, false> irows(src, w, w, h);
    T* dst = out + p * static_cast<int64_t>(h + 1) * W1;
    const Rows<T, VEC> orows(dst, W1, w + 1, h + 1);
    const int in_off = c0 * static_cast<int>(sizeof(TI));
    const int out_off = (c0 + 1) * static_cast<int>(sizeof(T));
    const bool lane_in = c0 < w;
    const unsigned lane_col = lane_in ? static_cast<unsigned>(c0) : 0u;

    // the whole band into registers, all loads in flight together (clamped addresses, values of
    // rows and lanes that do not exist dropped afterwards)
    T x[RMAX][4];
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
        const int row = r0 + r;
        const bool exists = r < R && row < r1;
        if (VEC) {
            load_quad(src + static_cast<int64_t>(min(row, h - 1)) * w + lane_col, x[r]);
            if (!(exists && lane_in)) {
#pragma unroll
                for (int v = 0; v < 4; ++v) x[r][v] = T(0);
            }
        } else {
            buffer_load_run_as<kCacheStream, TI>(x[r], irows.row(min(row, h - 1), exists), in_off);
        }
    }

    if (band == 0)
        for (int c = lane; c <= w; c += 64) dst[c] = T(0);

    {
        double own[4] = {0.0, 0.0, 0.0, 0.0};
#pragma unroll
        for (int r = 0; r < RMAX; ++r)
#pragma unroll
            for (int v = 0; v < 4; ++v) own[v] += static_cast<double>(x[r][v]);
#pragma unroll
        for (int v = 0; v < 4; ++v) sums[band][v][lane] = own[v];
    }
    __syncthreads();
    double colacc[4] = {0.0, 0.0, 0.0, 0.0};
    for (int b = 0; b < band; ++b)
#pragma unroll
        for (int v = 0; v < 4; ++v) colacc[v] += sums[b][v][lane];

#pragma unroll
    for (int bi = 0; bi < RMAX / RB; ++bi) {
        if (bi * RB >= R) break;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const int row = r0 + bi * RB + rb;
            double run = 0.0, pre[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                colacc[v] += static_cast<double>(x[bi * RB + rb][v]);
                run += colacc[v];
                pre[v] = run;
            }
            const double left = wave_inclusive_scan(run) - run;
            T res[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) res[v] = static_cast<T>(left + pre[v]);
            const RowRef orow = orows.row(min(row + 1, h), row < r1);
            // (VEC: the rows are addressed by offset into one descriptor for the plane, without a
            // bounds check of their own, so a lane past the row's end must not store)
            if (!VEC || lane_in)
                buffer_store_run<kCacheDefault, VEC>(res, orow, out_off, (w + 1) * static_cast<int>(sizeof(T)));
            if (lane == 0 && row < r1) dst[static_cast<int64_t>(row + 1) * W1] = T(0);
        }
    }
}

// Inclusive prefix sum within segments of L consecutive lanes (L = 16 or 32): the first steps of
// wave_inclusive_scan. All lanes must be active.
template <int L>
__device__ __forceinline__ double segment_inclusive_scan(double x) {
    static_assert(L == 16 || L == 32, "segments of one or two DPP rows");
    x += dpp_move<0x111, 0xf>(x, x);
    x += dpp_move<0x112, 0xf>(x, x);
    x += dpp_move<0x114, 0xf>(x, x);
    x += dpp_move<0x118, 0xf>(x, x);
    if (L == 32) x += dpp_move<0x142, 0xa>(0.0, x);   // lane 15 of rows 0,2 into rows 1,3
    return x;
}

// The same for planes of at most 128 (L = 32) or 64 (L = 16) columns, which would leave half or
// three quarters of every wave idle: a wave takes 64 / L bands side by side, L lanes each (band
// v of the plane: wave v / (64/L), lanes (v % (64/L)) * L ..), every lane walking down its own
// band's rows. Rows of a multiple of four columns from a 16-byte aligned address only.
template <class TI, int RMAX, int L>
__global__ void __launch_bounds__(kPlaneWaves * 64)
plane_scan_packed_kernel(const TI* __restrict__ in, float* __restrict__ out, int h, int w, int R, int64_t planes,
                         int reverse, ClipArgs<float> clip, int clip_blocks) {
    using T = float;
    constexpr int RB = 4, S = 64 / L;
    __shared__ double sums[kPlaneWaves * S * 4 * L];      // [band][4][L]

    if (static_cast<int>(blockIdx.x) < clip_blocks) {
        const int i = blockIdx.x * blockDim.x + threadIdx.x;
        if (i < clip.n) clip_box(clip, i);
        return;
    }
    int64_t p = blockIdx.x - clip_blocks;
    if (reverse) p = planes - 1 - p;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int l = lane & (L - 1);
    const int band = (tid >> 6) * S + lane / L;             // per lane; bands past the plane hold no rows
    const int r0 = band * R;
    const int r1 = min(h, r0 + R);
    const int64_t W1 = static_cast<int64_t>(w) + 1;
    const int c0 = 4 * l;
    const bool lane_in = c0 < w;

    const TI* src = in + p * static_cast<int64_t>(h) * w;
    T* dst = out + p * static_cast<int64_t>(h + 1) * W1;
    const Rows<T, true> orows(dst, W1, w + 1, h + 1);
    const RowRef oplane = orows.row(0);                      // the plane as one buffer; rows by offset
    const unsigned lane_col = lane_in ? static_cast<unsigned>(c0) : 0u;

    T x[RMAX][4];
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
        const int row = r0 + r;
        const bool exists = r < R && row < r1 && lane_in;
        load_quad(src + static_cast<int64_t>(min(row, h - 1)) * w + lane_col, x[r]);
        if (!exists) {
#pragma unroll
            for (int v = 0; v < 4; ++v) x[r][v] = T(0);
        }
    }

    if (tid < 64)
        for (int c = tid; c <= w; c += 64) dst[c] = T(0);

    {
        double own[4] = {0.0, 0.0, 0.0, 0.0};
#pragma unroll
        for (int r = 0; r < RMAX; ++r)
#pragma unroll
            for (int v = 0; v < 4; ++v) own[v] += static_cast<double>(x[r][v]);
#pragma unroll
        for (int v = 0; v < 4; ++v) sums[(band * 4 + v) * L + l] = own[v];
    }
    __syncthreads();
    double colacc[4] = {0.0, 0.0, 0.0, 0.0};
    const int wave_last = ((tid >> 6) + 1) * S - 1;         // the wave's last band (wave-uniform)
    for (int b = 0; b < wave_last; ++b)
        if (b < band) {
#pragma unroll
            for (int v = 0; v < 4; ++v) colacc[v] += sums[(b * 4 + v) * L + l];
        }

#pragma unroll
    for (int bi = 0; bi < RMAX / RB; ++bi) {
        if (bi * RB >= R) break;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const int row = r0 + bi * RB + rb;
            double run = 0.0, pre[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                colacc[v] += static_cast<double>(x[bi * RB + rb][v]);
                run += colacc[v];
                pre[v] = run;
            }
            const double left = segment_inclusive_scan<L>(run) - run;
            T res[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) res[v] = static_cast<T>(left + pre[v]);
            if (row < r1) {
                const int off = static_cast<int>((static_cast<int64_t>(row + 1) * W1 + c0 + 1) * sizeof(T));
                if (lane_in) buffer_store_run<kCacheDefault, true>(res, oplane, off, 0);
                if (l == 0) dst[static_cast<int64_t>(row + 1) * W1] = T(0);
            }
        }
    }
}

template <class T>
bool aligned_for_vec4(const T* p, int w) {
    return (w % 4 == 0) && (reinterpret_cast<uintptr_t>(p) % (4 * sizeof(T)) == 0);
}

template <class T, int WAVES, int M, int RB>
hipError_t launch_scan(const T* in, T* out, const double* aux, int64_t planes, int h, int w,
                       int nb, int R, bool reverse, hipStream_t stream) {
    const int64_t total = planes * nb;
    const int64_t per_xcd = (total + kXcds - 1) / kXcds;
    const int rev = reverse ? 1 : 0;
    const dim3 grid(static_cast<unsigned>(per_xcd * kXcds));
    const dim3 block(WAVES * 64);
    if (aligned_for_vec4(in, w))
        BOXCONV_LAUNCH("band_scan", (band_scan_kernel<T, WAVES, M, RB, true>), grid, block, 0, stream,
                       in, out, aux, h, w, nb, R, total, per_xcd, rev);
    else
        BOXCONV_LAUNCH("band_scan", (band_scan_kernel<T, WAVES, M, RB, false>), grid, block, 0, stream,
                       in, out, aux, h, w, nb, R, total, per_xcd, rev);
    return hipGetLastError();
}

template <class T, class TI, int WAVES, int RB>
hipError_t launch_scan_rows(const TI* in, T* out, const double* aux, int64_t planes, int h, int w,
                            int nb, int R, bool reverse, hipStream_t stream) {
    const int64_t total = planes * nb;
    const int64_t per_xcd = (total + kXcds - 1) / kXcds;
    const int rev = reverse ? 1 : 0;
    const dim3 grid(static_cast<unsigned>(per_xcd * kXcds));
    const dim3 block(WAVES * 64);
    const bool vec = aligned_for_vec4(in, w), full = (w == WAVES * 256);
#define LAUNCH_ROWS(VEC, FULL)                                                                     \
    BOXCONV_LAUNCH("band_scan", (band_scan_rows_kernel<T, TI, WAVES, RB, VEC, FULL>), grid, block, 0,  \
                   stream, in, out, aux, h, w, nb, R, total, per_xcd, rev)
    if (vec && full) LAUNCH_ROWS(true, true);
    else if (vec)    LAUNCH_ROWS(true, false);
    else             LAUNCH_ROWS(false, false);
#undef LAUNCH_ROWS
    return hipGetLastError();
}

// Polls of a band's hand-over words before the band is summed directly instead. A poll is a
// load round trip plus a short sleep, 1 to 2 us; the sums of a band above normally arrive within
// a few polls, and re-summing 32 rows costs a few microseconds, so 64 polls (about 100 us at
// worst) bound the damage should workgroups ever be started out of order.
int lookback_spin_limit() { return switches().spin_limit; }
// BOXCONV_INTEGRAL_LOOKBACK=2: single-pass kernel for every shape it covers, not only those where
// it was measured to be faster (used by the tests to reach its partial-row and partial-band code).
bool lookback_any_shape() { return switches().lookback_any_shape; }
bool lookback_enabled() { return switches().lookback; }

template <class TI, int WAVES>
hipError_t launch_lookback(const TI* in, float* out, double* aux, int64_t planes, int h, int w,
                           int nb, int R, bool reverse, bool prepared, hipStream_t stream) {
    if (!prepared) {
        const int64_t nsums = planes * static_cast<int64_t>(nb - 1) * lookback_row_words(w);
        BOXCONV_LAUNCH("fill_marker", fill_marker_kernel, dim3(static_cast<unsigned>((nsums + 255) / 256)),
                       dim3(256), 0, stream, reinterpret_cast<unsigned long long*>(aux), nsums);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    const int64_t per_xcd = ((planes + kXcds - 1) / kXcds) * nb;     // whole planes per XCD
    const int rev = reverse ? 1 : 0;
    const int spin = lookback_spin_limit();
    const dim3 grid(static_cast<unsigned>(per_xcd * kXcds));
    const dim3 block(WAVES * 64);
    // full: every lane holds four columns of the row or none (rows of a multiple of four columns)
    const bool vec = aligned_for_vec4(in, w), full = vec;
#define LAUNCH_LOOKBACK(VEC, FULL)                                                                 \
    BOXCONV_LAUNCH("band_scan", (band_scan_lookback_kernel<TI, WAVES, 4, VEC, FULL>), grid, block, 0,  \
                   stream, in, out, aux, h, w, nb, R, planes, per_xcd, rev, spin)
    if (vec && full) LAUNCH_LOOKBACK(true, true);
    else if (vec)    LAUNCH_LOOKBACK(true, false);
    else             LAUNCH_LOOKBACK(false, false);
#undef LAUNCH_LOOKBACK
    return hipGetLastError();
}
template <class T, class TI>
struct LookbackByWidth {
    static hipError_t run(const TI*, T*, double*, int64_t, int, int, int, int, bool, bool, hipStream_t) {
        return hipErrorInvalidValue;       // float output only
    }
};
template <class TI>
struct LookbackByWidth<float, TI> {
    static hipError_t run(const TI* in, float* out, double* aux, int64_t planes, int h, int w, int nb,
                          int R, bool reverse, bool prepared, hipStream_t stream) {
        // as many waves as the row needs at 256 columns each
        switch ((w + 255) / 256) {
            case 1: return launch_lookback<TI, 1>(in, out, aux, planes, h, w, nb, R, reverse, prepared, stream);
            case 2: return launch_lookback<TI, 2>(in, out, aux, planes, h, w, nb, R, reverse, prepared, stream);
            case 3: return launch_lookback<TI, 3>(in, out, aux, planes, h, w, nb, R, reverse, prepared, stream);
            case 4: return launch_lookback<TI, 4>(in, out, aux, planes, h, w, nb, R, reverse, prepared, stream);
            case 5: return launch_lookback<TI, 5>(in, out, aux, planes, h, w, nb, R, reverse, prepared, stream);
            case 6: return launch_lookback<TI, 6>(in, out, aux, planes, h, w, nb, R, reverse, prepared, stream);
            case 7: return launch_lookback<TI, 7>(in, out, aux, planes, h, w, nb, R, reverse, prepared, stream);
            default: return launch_lookback<TI, 8>(in, out, aux, planes, h, w, nb, R, reverse, prepared, stream);
        }
    }
};

// Bands of the plane-per-workgroup kernels: `slots` bands fit a workgroup (eight waves, times the
// bands a wave takes side by side); rows per band: whole row batches, at least 8, so that all
// rows fit those bands.
inline int plane_band_rows(int h, int slots) {
    return std::max(((h + slots - 1) / slots + 3) / 4 * 4, 8);
}

template <class TI>
hipError_t launch_plane_scan(const TI* in, float* out, int64_t planes, int h, int w, bool reverse,
                             hipStream_t stream, const ClipArgs<float>* clip_job = nullptr) {
    const ClipArgs<float> clip = clip_job != nullptr ? *clip_job : ClipArgs<float>{};
    const int rev = reverse ? 1 : 0;
    const bool vec = aligned_for_vec4(in, w);
    // lanes per row: rows of at most 128 / 64 columns share a wave with one / three more bands
    const int L = (vec && w <= 64) ? 16 : (vec && w <= 128) ? 32 : 64;
    const int S = 64 / L;
    const int R = plane_band_rows(h, kPlaneWaves * S);
    const int nb = (h + R - 1) / R;
    const int waves = (nb + S - 1) / S;
    const int clip_blocks = (clip.n + waves * 64 - 1) / (waves * 64);
    const dim3 grid(static_cast<unsigned>(planes + clip_blocks)), block(waves * 64);
#define LAUNCH_PLANE(RMAX)                                                                                \
    if (L == 16)  BOXCONV_LAUNCH("band_scan", (plane_scan_packed_kernel<TI, RMAX, 16>), grid, block, 0, stream, \
                                 in, out, h, w, R, planes, rev, clip, clip_blocks);                       \
    else if (L == 32) BOXCONV_LAUNCH("band_scan", (plane_scan_packed_kernel<TI, RMAX, 32>), grid, block, 0, stream, \
                                 in, out, h, w, R, planes, rev, clip, clip_blocks);                       \
    else if (vec) BOXCONV_LAUNCH("band_scan", (plane_scan_kernel<TI, RMAX, true>), grid, block, 0, stream, in, out, \
                            h, w, R, planes, rev, clip, clip_blocks);                                     \
    else     BOXCONV_LAUNCH("band_scan", (plane_scan_kernel<TI, RMAX, false>), grid, block, 0, stream, in, out, \
                            h, w, R, planes, rev, clip, clip_blocks)
    if (R <= 8)       { LAUNCH_PLANE(8); }
    else if (R <= 16) { LAUNCH_PLANE(16); }
    else              { LAUNCH_PLANE(kPlaneRows); }
#undef LAUNCH_PLANE
    return hipGetLastError();
}
template <class T, class TI>
struct PlaneScan {
    static hipError_t run(const TI*, T*, int64_t, int, int, bool, hipStream_t) {
        return hipErrorInvalidValue;       // float output only
    }
};
template <class TI>
struct PlaneScan<float, TI> {
    static hipError_t run(const TI* in, float* out, int64_t planes, int h, int w, bool reverse,
                          hipStream_t stream) {
        return launch_plane_scan<TI>(in, out, planes, h, w, reverse, stream);
    }
};

template <class T>
bool plane_pass_applies(const IntegralPlan& pl) {
    return pl.plane_per_workgroup && std::is_same<T, float>::value;
}
template <class T>
bool single_pass_applies(const IntegralPlan& pl) {
    return pl.lookback && std::is_same<T, float>::value && lookback_enabled() && !plane_pass_applies<T>(pl);
}

// Rows this narrow are scanned by band_scan_rows_kernel, which sums the band column sums itself;
// the bands above a workgroup are few (nb <= h/32), so re-reading them is cheaper than a pass.
inline bool scan_by_rows(int h, int w, size_t elem) {
    const uint64_t plane_bytes = (static_cast<uint64_t>(h) + 1) * (static_cast<uint64_t>(w) + 1) * elem;
    return w <= kMaxScanRowsWidth && plane_bytes < (1ull << 31);
}

}  // namespace

IntegralPlan plan_integral(int64_t planes, int h, int w, int64_t want) {
    IntegralPlan pl;
    // Small planes (float output): a workgroup per plane, a wave per band, bands of 8 to 24 rows
    // (whole row batches) so that up to eight waves share the plane. The rest of the plan is what
    // the types that kernel is not built for take, and what the workspace is sized for.
    // (BOXCONV_INTEGRAL_LOOKBACK=2 asks for the look-back kernel wherever it applies, here too)
    pl.plane_per_workgroup = switches().plane_integral && !lookback_any_shape() && h <= kPlaneMaxRows &&
                             w <= kPlaneMaxCols && planes < (1ll << 31);
    // Enough workgroups to cover 256 CUs several times over, but bands no shorter than 32 rows
    // (the per-band column-sum vector is 8 B per column, i.e. 2/R of the input bytes) and no
    // taller than 256 (size of the per-row carry array in LDS).
    // Problems that give few workgroups are bound by the length of a workgroup's chain of row
    // batches, not by bytes: images of 64 to 256 rows are then cut into bands of 16 rows
    // (measured 0.74-0.89 of the time with bands of 32 rows; shorter images would go from one
    // launch to two, taller ones would spend the gain on adding up the many bands above).
    int min_rows = 32;
    if (h >= 64 && h <= 256 && planes * (h / 32) < 2048) { min_rows = 16; want = std::max<int64_t>(want, 4096); }
    const int64_t wanted = (want + planes - 1) / std::max<int64_t>(planes, 1);
    int nb = static_cast<int>(std::min<int64_t>(wanted, std::max(1, h / min_rows)));
    // Where planes get cut anyway and the single-pass kernel covers the width, cut them into
    // bands of at most 32 rows, which that kernel holds in registers.
    // Measured against the three launches: 0.6-0.95 of their time when all workgroups are on the
    // chip at once (they then read, hand over and write in step, so the bands above are never
    // late) or when there are several times more than fit (they fall out of step and reads overlap
    // writes); 1.05-1.3 in between, for rows that do not fill the workgroup exactly, and for
    // planes of more than 32 bands in the first case.
    const int bands32 = (h + kLookbackRows - 1) / kLookbackRows;
    const int64_t groups = planes * bands32;                          // workgroups of the launch
    // workgroups that are on the chip at once: eight wave slots per CU at two waves per SIMD;
    // workgroups of five waves and more, of which only one would fit, get three per SIMD
    const int waves = std::max(1, (w + 255) / 256);
    const int64_t resident = 256 * (waves <= 4 ? 8 / waves : 12 / waves);
    // (rows of a multiple of four columns: every lane holds four columns or none. Measured on
    // 16 x 8 or 32 x 8 planes, single pass against two: 720 x 1280 43 against 59 us, 512 x 768 27
    // against 44, 256 x 1536 26 against 37, 512 x 1000 40 against 50, 480 x 640 35 against 41;
    // but 540 x 960, one workgroup in sixteen too many to be resident, 63 against 51, and
    // 1080 x 1920, 34 bands per plane, 117 against 80.)
    // Narrower rows leave most of a wave idle in either kernel; the two passes are faster there
    // (64 x 128: 20 against 24 us, 135 x 240: 21 against 25).
    const bool measured_faster = w % 4 == 0 && w >= 256 && ((groups <= resident && bands32 <= 32) || groups >= 4096);
    const bool single_pass = wanted >= 2 && h > kLookbackRows && w <= 2048 && scan_by_rows(h, w, sizeof(float)) &&
                             bands32 <= kLookbackBands && (lookback_any_shape() || measured_faster);
    if (single_pass) nb = (h + kLookbackRows - 1) / kLookbackRows;
    nb = std::max(nb, (h + 255) / 256);
    nb = std::max(nb, 1);
    int R = (h + nb - 1) / nb;
    R = ((R + 3) / 4) * 4;                 // whole row batches
    R = std::min(R, 256);
    nb = (h + R - 1) / R;
    pl.nb = nb;
    pl.R = R;
    pl.lookback = single_pass && nb > 1 && nb <= kLookbackBands && R <= kLookbackRows &&
                  planes * nb < (1ll << 31);
    pl.aux_doubles = (nb > 1) ? planes * static_cast<int64_t>(nb - 1) * (pl.lookback ? lookback_row_words(w) : w) : 0;
    return pl;
}

bool clip_rides_on_integral(const IntegralPlan& pl, int64_t planes) {
    return pl.plane_per_workgroup && planes > 0 && planes + (1 << 20) < (1ll << 31);
}

template <class TI>
hipError_t clip_and_plane_integral_launch(const ClipArgs<float>& clip, const TI* in, float* out,
                                          int64_t planes, int h, int w, const IntegralPlan& pl,
                                          hipStream_t stream) {
    if (!clip_rides_on_integral(pl, planes)) return hipErrorInvalidValue;
    return launch_plane_scan<TI>(in, out, planes, h, w, false, stream, &clip);
}
template hipError_t clip_and_plane_integral_launch<float>(const ClipArgs<float>&, const float*, float*, int64_t,
                                                          int, int, const IntegralPlan&, hipStream_t);
template hipError_t clip_and_plane_integral_launch<f16_t>(const ClipArgs<float>&, const f16_t*, float*, int64_t,
                                                          int, int, const IntegralPlan&, hipStream_t);
template hipError_t clip_and_plane_integral_launch<bf16_t>(const ClipArgs<float>&, const bf16_t*, float*, int64_t,
                                                           int, int, const IntegralPlan&, hipStream_t);

template <class T>
hipError_t clip_and_prepare_integral_launch(const ClipArgs<T>& clip, int64_t planes, int w,
                                            double* aux, const IntegralPlan& pl, bool* prepared,
                                            hipStream_t stream) {
    const bool fill = single_pass_applies<T>(pl);
    *prepared = fill;
    const int clip_blocks = (clip.n + 255) / 256;
    const int64_t nsums = fill ? planes * static_cast<int64_t>(pl.nb - 1) * lookback_row_words(w) : 0;
    const int64_t blocks = clip_blocks + (nsums + 255) / 256;
    if (blocks == 0) return hipSuccess;
    BOXCONV_LAUNCH("clip", (clip_and_fill_marker_kernel<T>), dim3(static_cast<unsigned>(blocks)), dim3(256),
                   0, stream, clip, clip_blocks, reinterpret_cast<unsigned long long*>(aux), nsums);
    return hipGetLastError();
}

// The tiled kernels for widths above 4096 read T only.
template <class T, class TI>
struct TiledScan {
    static hipError_t run(const TI*, T*, double*, int64_t, int, int, int, int, bool, hipStream_t) {
        return hipErrorInvalidValue;
    }
};
template <class T>
struct TiledScan<T, T> {
    static hipError_t run(const T* in, T* out, double* aux, int64_t planes, int h, int w, int nb, int R,
                          bool reverse_order, hipStream_t stream) {
        // Tile width: one wave covers 256 columns per chunk, four waves 1024.
        if (w <= 256)        return launch_scan<T, 1, 1, 4>(in, out, aux, planes, h, w, nb, R, reverse_order, stream);
        else if (w <= 512)   return launch_scan<T, 2, 1, 4>(in, out, aux, planes, h, w, nb, R, reverse_order, stream);
        else if (w <= 1024)  return launch_scan<T, 4, 1, 4>(in, out, aux, planes, h, w, nb, R, reverse_order, stream);
        else if (w <= 2048)  return launch_scan<T, 4, 2, 2>(in, out, aux, planes, h, w, nb, R, reverse_order, stream);
        else                 return launch_scan<T, 4, 4, 1>(in, out, aux, planes, h, w, nb, R, reverse_order, stream);
    }
};

template <class T, class TI>
hipError_t integral_image_any(const TI* in, T* out, int64_t planes, int h, int w, double* aux,
                              const IntegralPlan& pl, bool workspace_prepared, bool reverse_order,
                              hipStream_t stream) {
    if (planes == 0) return hipSuccess;
    const int nb = pl.nb, R = pl.R;
    const bool by_rows = scan_by_rows(h, w, sizeof(T));
    if (!by_rows && !std::is_same<T, TI>::value) return hipErrorInvalidValue;
    if (plane_pass_applies<T>(pl))
        return PlaneScan<T, TI>::run(in, out, planes, h, w, reverse_order, stream);
    if (single_pass_applies<T>(pl))
        return LookbackByWidth<T, TI>::run(in, out, aux, planes, h, w, nb, R, reverse_order,
                                           workspace_prepared, stream);
    if (nb > 1) {
        const int strips = (w + 1023) / 1024;
        const dim3 grid(static_cast<unsigned>(planes * (nb - 1) * strips));
        if (aligned_for_vec4(in, w))
            BOXCONV_LAUNCH("band_colsum", (band_colsum_kernel<T, TI, true>), grid, dim3(256), 0, stream,
                           in, aux, h, w, nb, R, strips);
        else
            BOXCONV_LAUNCH("band_colsum", (band_colsum_kernel<T, TI, false>), grid, dim3(256), 0, stream,
                           in, aux, h, w, nb, R, strips);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (nb > 2 && !by_rows) {
        const int64_t n = planes * w;
        BOXCONV_LAUNCH("band_prefix", band_prefix_kernel,
                       dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, stream, aux,
                       planes, w, nb);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (by_rows) {
        if (w <= 256)       return launch_scan_rows<T, TI, 1, 4>(in, out, aux, planes, h, w, nb, R, reverse_order, stream);
        else if (w <= 512)  return launch_scan_rows<T, TI, 2, 4>(in, out, aux, planes, h, w, nb, R, reverse_order, stream);
        else if (w <= 1024) return launch_scan_rows<T, TI, 4, 4>(in, out, aux, planes, h, w, nb, R, reverse_order, stream);
        else if (w <= 2048) return launch_scan_rows<T, TI, 8, 4>(in, out, aux, planes, h, w, nb, R, reverse_order, stream);
        else                return launch_scan_rows<T, TI, 16, 4>(in, out, aux, planes, h, w, nb, R, reverse_order, stream);
    }
    return TiledScan<T, TI>::run(in, out, aux, planes, h, w, nb, R, reverse_order, stream);
}

template <class T>
hipError_t integral_image_launch(const T* in, T* out, int64_t planes, int h, int w,
                                 double* aux, const IntegralPlan& pl, bool workspace_prepared,
                                 bool reverse_order, hipStream_t stream) {
    return integral_image_any<T, T>(in, out, planes, h, w, aux, pl, workspace_prepared, reverse_order,
                                    stream);
}

template <class TI>
hipError_t integral_image_widening_launch(const TI* in, float* out, int64_t planes, int h, int w,
                                          double* aux, const IntegralPlan& pl, hipStream_t stream,
                                          bool workspace_prepared) {
    return integral_image_any<float, TI>(in, out, planes, h, w, aux, pl, workspace_prepared, false, stream);
}

bool integral_image_widening_applies(int h, int w) {
    return w <= kMaxWideningWidth && scan_by_rows(h, w, sizeof(float));
}

template hipError_t integral_image_widening_launch<f16_t>(const f16_t*, float*, int64_t, int, int,
                                                          double*, const IntegralPlan&, hipStream_t, bool);
template hipError_t integral_image_widening_launch<bf16_t>(const bf16_t*, float*, int64_t, int, int,
                                                           double*, const IntegralPlan&, hipStream_t, bool);
template hipError_t integral_image_launch<float>(const float*, float*, int64_t, int, int,
                                                 double*, const IntegralPlan&, bool, bool, hipStream_t);
template hipError_t integral_image_launch<double>(const double*, double*, int64_t, int, int,
                                                  double*, const IntegralPlan&, bool, bool, hipStream_t);
template hipError_t clip_and_prepare_integral_launch<float>(const ClipArgs<float>&, int64_t, int, double*,
                                                            const IntegralPlan&, bool*, hipStream_t);
template hipError_t clip_and_prepare_integral_launch<double>(const ClipArgs<double>&, int64_t, int, double*,
                                                             const IntegralPlan&, bool*, hipStream_t);

}  // namespace boxconv
