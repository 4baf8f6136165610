// TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// Plain C++ (no torch, no HIP) restatement of the CPU path of shrubb/box-convolutions:
//   * src/integral_image.cpp:8-39                 -> integral_image<T>
//   * src/box_convolution.cpp:14-40,43-69,72-98   -> split_forward / split_grad_input / split_grad_params
//   * src/box_convolution.cpp:100-261             -> box_forward<T>
//   * src/box_convolution.cpp:286-456             -> box_grad_input_planes<T>
//   * src/box_convolution.cpp:480-715             -> box_grad_param_pixel<T>
//   * src/box_convolution.cpp:729-763             -> clip_pair<T>
//   * src/box_convolution.cpp:765-793             -> inverse_extent<T>
//   * src/box_convolution_interface.cpp:141-395   -> box_backward<T> (orchestration)
//   * src/box_convolution_interface.cpp:397-415   -> clip entry (min sizes 1.001f / 2.001f)
//
// Every floating-point expression keeps the reference's operand order and working type
// (scalar_t), so that the forward output and the per-filter grad-input planes agree with a
// compiled reference bit for bit. Two places deliberately differ, both in the direction of
// *more* accuracy, because the reference delegates them to ATen's `sum` whose blocked
// summation order is an implementation detail of the installed torch:
//   (1) the reduction over (batch, h*w) of tmp*grad_output and grad_output*output
//       (src/box_convolution_interface.cpp:343-346,357-358) accumulates in double here;
//   (2) nothing else.
// Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this file's
// library; the product (the HIP library) never does.
//
// Pinning status of each function is recorded in tests/test_oracle_pins.py.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

namespace {

inline int clampi(int v, int lo, int hi) { return std::max(lo, std::min(v, hi)); }

// ---------------------------------------------------------------------------------------------
// Integral image, src/integral_image.cpp:20-37. The running row sum lives in the accumulate type
// (double for float and for double, at::acc_type<scalar_t,false>); the previous output row is
// read back in scalar_t and the store rounds to scalar_t.
// Integer tensors (AT_DISPATCH_ALL_TYPES, src/integral_image.cpp:14) accumulate in int64
// (at::acc_type<integer, false>) and store back in their own type, i.e. modulo 2^bits.
template <class T> struct AccumulateType { using type = double; };
template <> struct AccumulateType<uint8_t> { using type = int64_t; };
template <> struct AccumulateType<int8_t> { using type = int64_t; };
template <> struct AccumulateType<int16_t> { using type = int64_t; };
template <> struct AccumulateType<int32_t> { using type = int64_t; };
template <> struct AccumulateType<int64_t> { using type = int64_t; };

template <class T>
void integral_image(const T* in, T* out, int64_t planes, int h, int w) {
    using Acc = typename AccumulateType<T>::type;
    const int64_t W1 = w + 1;
    for (int64_t p = 0; p < planes; ++p) {
        const T* src = in + p * (int64_t)h * w;
        T* dst = out + p * (int64_t)(h + 1) * W1;
        std::memset(dst, 0, sizeof(T) * W1);
        for (int row = 0; row < h; ++row) {
            T* cur = dst + (int64_t)(row + 1) * W1;
            const T* prev = dst + (int64_t)row * W1;
            cur[0] = T(0);
            Acc run = 0;
            for (int col = 0; col < w; ++col) {
                run += src[(int64_t)row * w + col];
                cur[col + 1] = static_cast<T>(run + prev[col + 1]);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Integer / fractional split of one box; three variants.
template <class T>
struct Split {
    int xlo, xhi, ylo, yhi;      // xMinInt, xMaxInt, yMinInt, yMaxInt
    T fxlo, fxhi, fylo, fyhi;    // xMinFrac, xMaxFrac, yMinFrac, yMaxFrac
};

// src/box_convolution.cpp:22-38
template <class T>
Split<T> split_forward(T xmin, T xmax, T ymin, T ymax) {
    Split<T> s;
    T v;
    v = std::ceil(xmin);  s.fxlo = v - xmin; s.xlo = static_cast<int>(v);
    v = std::ceil(ymin);  s.fylo = v - ymin; s.ylo = static_cast<int>(v);
    v = std::floor(xmax); s.fxhi = xmax - v; s.xhi = static_cast<int>(v) + 1;
    v = std::floor(ymax); s.fyhi = ymax - v; s.yhi = static_cast<int>(v) + 1;
    return s;
}

// src/box_convolution.cpp:51-67 (box mirrored through the origin)
template <class T>
Split<T> split_grad_input(T xmin, T xmax, T ymin, T ymax) {
    Split<T> s;
    T v;
    v = std::ceil(-xmax);       s.fxlo = v + xmax;        s.xlo = static_cast<int>(v);
    v = std::ceil(-ymax);       s.fylo = v + ymax;        s.ylo = static_cast<int>(v);
    v = std::floor(-xmin) + 1;  s.fxhi = -xmin + 1 - v;   s.xhi = static_cast<int>(v);
    v = std::floor(-ymin) + 1;  s.fyhi = -ymin + 1 - v;   s.yhi = static_cast<int>(v);
    return s;
}

// src/box_convolution.cpp:80-96 (used with 1-based pixel coordinates)
template <class T>
Split<T> split_grad_params(T xmin, T xmax, T ymin, T ymax) {
    Split<T> s;
    T v;
    v = std::ceil(xmin - 1); s.fxlo = v - xmin + 1; s.xlo = static_cast<int>(v);
    v = std::ceil(ymin - 1); s.fylo = v - ymin + 1; s.ylo = static_cast<int>(v);
    v = std::floor(xmax);    s.fxhi = xmax - v;     s.xhi = static_cast<int>(v);
    v = std::floor(ymax);    s.fyhi = ymax - v;     s.yhi = static_cast<int>(v);
    return s;
}

// src/box_convolution.cpp:765-793: reciprocal of the product of the selected extents, built as
// ones * (xmax - xmin + 1) * (ymax - ymin + 1) in scalar_t; rounded mode ceils/floors first.
template <class T>
T inverse_extent(T xmin, T xmax, T ymin, T ymax, bool exact, bool use_x, bool use_y) {
    if (!exact) {
        xmin = std::ceil(xmin); ymin = std::ceil(ymin);
        xmax = std::floor(xmax); ymax = std::floor(ymax);
    }
    T acc = T(1);
    if (use_x) { T e = xmax - xmin; e += T(1); acc *= e; }
    if (use_y) { T e = ymax - ymin; e += T(1); acc *= e; }
    return T(1) / acc;
}

// View of one (h+1) x (w+1) integral plane.
template <class T>
struct Plane {
    const T* p; int64_t pitch;
    T operator()(int r, int c) const { return p[(int64_t)r * pitch + c]; }
};

// ---------------------------------------------------------------------------------------------
// Forward value of one output pixel, src/box_convolution.cpp:157-254.
template <class T>
T forward_pixel(const Plane<T>& I, const Split<T>& s, int x, int y, int h, int w, bool exact) {
    const int t = clampi(x + s.xlo, 0, h), b = clampi(x + s.xhi, 0, h);
    const int l = clampi(y + s.ylo, 0, w), r = clampi(y + s.yhi, 0, w);
    const int bAdv = clampi(x + s.xhi + 1, 0, h), rAdv = clampi(y + s.yhi + 1, 0, w);
    const int tAdv = clampi(x + s.xlo - 1, 0, h), lAdv = clampi(y + s.ylo - 1, 0, w);

    T v = I(b, r) - I(t, r) - I(b, l) + I(t, l);
    if (!exact) return v;

    v += (I(bAdv, r) - I(b, r) - I(bAdv, l) + I(b, l)) * s.fxhi;
    v += (I(b, rAdv) - I(b, r) - I(t, rAdv) + I(t, r)) * s.fyhi;
    v += (I(t, r) - I(tAdv, r) - I(t, l) + I(tAdv, l)) * s.fxlo;
    v += (I(b, l) - I(b, lAdv) - I(t, l) + I(t, lAdv)) * s.fylo;

    const int xb = x + s.xhi, xt = x + s.xlo, yr = y + s.yhi, yl = y + s.ylo;
    if (!((xb >= h) | (yr >= w) | (xb < 0) | (yr < 0)))
        v += s.fxhi * s.fyhi * (I(b + 1, r + 1) - I(b, r + 1) - I(b + 1, r) + I(b, r));
    if (!((xt > h) | (yr >= w) | (xt <= 0) | (yr < 0)))
        v += s.fxlo * s.fyhi * (I(t, r + 1) - I(t - 1, r + 1) - I(t, r) + I(t - 1, r));
    if (!((xb >= h) | (yl > w) | (xb < 0) | (yl <= 0)))
        v += s.fxhi * s.fylo * (I(b + 1, l) - I(b, l) - I(b + 1, l - 1) + I(b, l - 1));
    if (!((xt > h) | (yl > w) | (xt <= 0) | (yl <= 0)))
        v += s.fxlo * s.fylo * (I(t, l) - I(t - 1, l) - I(t, l - 1) + I(t - 1, l - 1));
    return v;
}

// Same quantity as written for the grad-input pass, src/box_convolution.cpp:337-444: the
// advanced indices are derived from the clamped ones and the corner terms are zeroed when the
// advanced index coincides with the plain one.
template <class T>
T grad_input_pixel(const Plane<T>& G, const Split<T>& s, int x, int y, int h, int w, bool exact) {
    const int t = clampi(x + s.xlo, 0, h), b = clampi(x + s.xhi, 0, h);
    const int l = clampi(y + s.ylo, 0, w), r = clampi(y + s.yhi, 0, w);
    const int tAdv = (x + s.xlo - 1 < h) ? clampi(t - 1, 0, h) : t;
    const int bAdv = (x + s.xhi >= 0) ? clampi(b + 1, 0, h) : b;
    const int lAdv = (y + s.ylo - 1 < w) ? clampi(l - 1, 0, w) : l;
    const int rAdv = (y + s.yhi >= 0) ? clampi(r + 1, 0, w) : r;

    T v = G(b, r) - G(t, r) - G(b, l) + G(t, l);
    if (!exact) return v;

    v += (G(bAdv, r) - G(b, r) - G(bAdv, l) + G(b, l)) * s.fxhi;
    v += (G(b, rAdv) - G(b, r) - G(t, rAdv) + G(t, r)) * s.fyhi;
    v += (G(t, r) - G(tAdv, r) - G(t, l) + G(tAdv, l)) * s.fxlo;
    v += (G(b, l) - G(b, lAdv) - G(t, l) + G(t, lAdv)) * s.fylo;

    const int xb = x + s.xhi, xt = x + s.xlo, yr = y + s.yhi, yl = y + s.ylo;
    const bool noBR = (xb >= h) || (yr >= w) || (xb < 0) || (yr < 0) || (b == bAdv) || (r == rAdv);
    v += s.fxhi * s.fyhi *
         (noBR ? T(0) : (G(b + 1, r + 1) - G(b, r + 1) - G(b + 1, r) + G(b, r)));
    const bool noTR = (xt > h) || (yr >= w) || (xt <= 0) || (yr < 0) || (t == tAdv) || (r == rAdv);
    v += s.fxlo * s.fyhi *
         (noTR ? T(0) : (G(tAdv + 1, r + 1) - G(tAdv + 1, r) - G(tAdv, r + 1) + G(tAdv, r)));
    const bool noBL = (xb >= h) || (yl > w) || (xb < 0) || (yl <= 0) || (b == bAdv) || (l == lAdv);
    v += s.fxhi * s.fylo *
         (noBL ? T(0) : (G(b + 1, lAdv + 1) - G(b, lAdv + 1) - G(b + 1, lAdv) + G(b, lAdv)));
    const bool noTL = (xt > h) || (yl > w) || (xt <= 0) || (yl <= 0) || (t == tAdv) || (l == lAdv);
    v += s.fxlo * s.fylo *
         (noTL ? T(0) : (G(tAdv + 1, lAdv + 1) - G(tAdv + 1, lAdv) - G(tAdv, lAdv + 1) + G(tAdv, lAdv)));
    return v;
}

// One input pixel recovered from the integral plane, indices clamped into the image,
// src/box_convolution.cpp:539-545 and its seven siblings.
template <class T>
T pixel_from_integral(const Plane<T>& I, int px, int py, int h, int w) {
    const int cx = clampi(px, 0, h - 1), cy = clampi(py, 0, w - 1);
    return I(cx + 1, cy + 1) - I(cx, cy + 1) - I(cx + 1, cy) + I(cx, cy);
}

// d(box sum)/d(parameter) at one output pixel; (x, y) are the reference's 1-based loop
// variables and `s` comes from split_grad_params. src/box_convolution.cpp:527-708.
// which: 0 xMin, 1 xMax, 2 yMin, 3 yMax (enum class Parameter, src/box_convolution.h:3).
template <class T>
T box_grad_param_pixel(const Plane<T>& I, const Split<T>& s, int which, int x, int y,
                       int h, int w, bool exact) {
    const int X0 = x + s.xlo, X1 = x + s.xhi, Y0 = y + s.ylo, Y1 = y + s.yhi;
    auto at = [&](int r, int c) { return I(clampi(r, 0, h), clampi(c, 0, w)); };
    T d = T(0);
    switch (which) {
    case 0: {
        if (exact) {
            int ok = !(Y0 < 1) & !(Y0 > w) & !(X0 < 1);
            const T tl = ok * pixel_from_integral(I, X0 - 1, Y0 - 1, h, w);
            ok = !(Y1 < 0) & !(Y1 >= w) & !(X0 < 1);
            const T tr = ok * pixel_from_integral(I, X0 - 1, Y1, h, w);
            d += tr * s.fyhi;
            d += tl * s.fylo;
        }
        d += at(X0, Y1); d -= at(X0 - 1, Y1); d -= at(X0, Y0); d += at(X0 - 1, Y0);
        d *= (X0 >= 1) & (X0 <= h);
        return -d;
    }
    case 1: {
        if (exact) {
            int ok = !(Y0 < 1) & !(Y0 > w) & !(X1 >= h);
            const T bl = ok * pixel_from_integral(I, X1, Y0 - 1, h, w);
            ok = !(Y1 < 0) & !(Y1 >= w) & !(X1 >= h);
            const T br = ok * pixel_from_integral(I, X1, Y1, h, w);
            d += br * s.fyhi;
            d += bl * s.fylo;
        }
        d += at(X1 + 1, Y1); d -= at(X1, Y1); d -= at(X1 + 1, Y0); d += at(X1, Y0);
        d *= (X1 >= 0) & (X1 < h);
        return d;
    }
    case 2: {
        if (exact) {
            int ok = !(Y0 < 1) & !(X0 < 1) & !(X0 > h);
            const T tl = ok * pixel_from_integral(I, X0 - 1, Y0 - 1, h, w);
            ok = !(Y0 < 1) & !(X1 < 0) & !(X1 >= h);
            const T bl = ok * pixel_from_integral(I, X1, Y0 - 1, h, w);
            d += tl * s.fxlo;
            d += bl * s.fxhi;
        }
        d += at(X1, Y0); d -= at(X1, Y0 - 1); d -= at(X0, Y0); d += at(X0, Y0 - 1);
        d *= (Y0 >= 1) & (Y0 <= w);
        return -d;
    }
    default: {
        if (exact) {
            int ok = !(Y1 >= w) & !(X0 < 1) & !(X0 > h);
            const T tr = ok * pixel_from_integral(I, X0 - 1, Y1, h, w);
            ok = !(Y1 >= w) & !(X1 < 0) & !(X1 >= h);
            const T br = ok * pixel_from_integral(I, X1, Y1, h, w);
            d += tr * s.fxlo;
            d += br * s.fxhi;
        }
        d += at(X1, Y1 + 1); d -= at(X1, Y1); d -= at(X0, Y1 + 1); d += at(X0, Y1);
        d *= (Y1 >= 0) & (Y1 < w);
        return d;
    }
    }
}

// ---------------------------------------------------------------------------------------------
// box_convolution_forward, src/box_convolution_interface.cpp:13-139 + box_convolution.cpp:129-259.
// integ: [B,C,h+1,w+1]; params: [C,F] in real (pixel) units; out: [B,C,F,h,w].
template <class T>
void box_forward(const T* integ, const T* xmin, const T* xmax, const T* ymin, const T* ymax,
                 T* out, int B, int C, int F, int h, int w, bool normalize, bool exact) {
    const int64_t ipl = (int64_t)(h + 1) * (w + 1);
    for (int b = 0; b < B; ++b)
        for (int c = 0; c < C; ++c) {
            Plane<T> I{integ + ((int64_t)b * C + c) * ipl, w + 1};
            for (int f = 0; f < F; ++f) {
                const int k = c * F + f;
                const Split<T> s = split_forward(xmin[k], xmax[k], ymin[k], ymax[k]);
                const T scale = normalize
                    ? inverse_extent(xmin[k], xmax[k], ymin[k], ymax[k], exact, true, true) : T(1);
                T* o = out + (((int64_t)b * C + c) * F + f) * (int64_t)h * w;
                for (int x = 0; x < h; ++x)
                    for (int y = 0; y < w; ++y)
                        o[(int64_t)x * w + y] = forward_pixel(I, s, x, y, h, w, exact) * scale;
            }
        }
}

// Per-(b,c,f) planes of the grad-input pass before the reduction over f,
// src/box_convolution_interface.cpp:198-272. tmp: [B,C,F,h,w].
template <class T>
void box_grad_input_planes(const T* gint, const T* xmin, const T* xmax, const T* ymin,
                           const T* ymax, T* tmp, int B, int C, int F, int h, int w,
                           bool normalize, bool exact) {
    const int64_t ipl = (int64_t)(h + 1) * (w + 1);
    for (int b = 0; b < B; ++b)
        for (int c = 0; c < C; ++c)
            for (int f = 0; f < F; ++f) {
                const int k = c * F + f;
                const int64_t plane = ((int64_t)b * C + c) * F + f;
                Plane<T> G{gint + plane * ipl, w + 1};
                const Split<T> s = split_grad_input(xmin[k], xmax[k], ymin[k], ymax[k]);
                const T scale = normalize
                    ? inverse_extent(xmin[k], xmax[k], ymin[k], ymax[k], exact, true, true) : T(1);
                T* o = tmp + plane * (int64_t)h * w;
                for (int x = 0; x < h; ++x)
                    for (int y = 0; y < w; ++y)
                        o[(int64_t)x * w + y] = grad_input_pixel(G, s, x, y, h, w, exact) * scale;
            }
}

// box_convolution_backward, src/box_convolution_interface.cpp:141-395.
// needs[0]: input grad, needs[1..4]: xMin, xMax, yMin, yMax. Unneeded outputs are left untouched.
template <class T>
void box_backward(const T* integ, const T* xmin, const T* xmax, const T* ymin, const T* ymax,
                  const T* grad_out, const T* output, float reparam_h, float reparam_w,
                  bool normalize, bool exact, const int* needs, T* grad_in, T* const* gparam,
                  int B, int C, int F, int h, int w) {
    const int64_t hw = (int64_t)h * w;
    const int64_t nout = (int64_t)B * C * F * hw;

    if (needs[0]) {
        // :199 integral image of the 5-D grad_output, :274 tmpArray.sum(2) (in order, scalar_t)
        std::vector<T> gint((size_t)B * C * F * (h + 1) * (w + 1));
        integral_image(grad_out, gint.data(), (int64_t)B * C * F, h, w);
        std::vector<T> tmp((size_t)nout);
        box_grad_input_planes(gint.data(), xmin, xmax, ymin, ymax, tmp.data(),
                              B, C, F, h, w, normalize, exact);
        for (int64_t bc = 0; bc < (int64_t)B * C; ++bc)
            for (int64_t px = 0; px < hw; ++px) {
                T acc = tmp[(size_t)((bc * F) * hw + px)];
                for (int f = 1; f < F; ++f) acc += tmp[(size_t)((bc * F + f) * hw + px)];
                grad_in[bc * hw + px] = acc;
            }
    }

    if (!(needs[1] | needs[2] | needs[3] | needs[4])) return;

    const int64_t ipl = (int64_t)(h + 1) * (w + 1);
    for (int which = 0; which < 4; ++which) {
        if (!needs[1 + which]) continue;
        for (int c = 0; c < C; ++c)
            for (int f = 0; f < F; ++f) {
                const int k = c * F + f;
                const Split<T> s = split_grad_params(xmin[k], xmax[k], ymin[k], ymax[k]);
                double acc = 0.0;    // deliberate: see file header, item (1)
                for (int b = 0; b < B; ++b) {
                    Plane<T> I{integ + ((int64_t)b * C + c) * ipl, w + 1};
                    const T* g = grad_out + (((int64_t)b * C + c) * F + f) * hw;
                    for (int x = 1; x <= h; ++x)
                        for (int y = 1; y <= w; ++y) {
                            T v = box_grad_param_pixel(I, s, which, x, y, h, w, exact);
                            v *= g[(int64_t)(x - 1) * w + (y - 1)];          // :343 tmpArray.mul_
                            acc += v;
                        }
                }
                T gsum = static_cast<T>(acc);                                    // :345-346
                if (normalize)                                                  // :348-350
                    gsum *= inverse_extent(xmin[k], xmax[k], ymin[k], ymax[k], exact, true, true);
                gparam[which][k] = gsum;
            }
    }

    if (normalize) {
        // :354-379 second summand: sum(grad_output * output) * (+-1) / extent along the
        // parameter's own axis.
        for (int c = 0; c < C; ++c)
            for (int f = 0; f < F; ++f) {
                const int k = c * F + f;
                double acc = 0.0;    // deliberate: see file header, item (1)
                for (int b = 0; b < B; ++b) {
                    const int64_t off = (((int64_t)b * C + c) * F + f) * hw;
                    for (int64_t px = 0; px < hw; ++px) {
                        const T v = grad_out[off + px] * output[off + px];     // :357
                        acc += v;
                    }
                }
                const T s = static_cast<T>(acc);
                for (int which = 0; which < 4; ++which) {
                    if (!needs[1 + which]) continue;
                    const bool is_x = which < 2;
                    const T inv = inverse_extent(xmin[k], xmax[k], ymin[k], ymax[k], exact,
                                                 is_x, !is_x);
                    const T sign = (which == 1 || which == 3) ? T(-1) : T(1);
                    gparam[which][k] = gparam[which][k] + sign * s * inv;      // :377 addcmul_
                }
            }
    }

    // :383-391: reparametrization arrives as C float, is widened to double and applied by an
    // in-place multiply on a scalar_t tensor (the multiply itself runs in scalar_t for float,
    // in double for double).
    for (int which = 0; which < 4; ++which) {
        if (!needs[1 + which]) continue;
        const double scale = which < 2 ? reparam_h : reparam_w;
        for (int k = 0; k < C * F; ++k) gparam[which][k] = gparam[which][k] * static_cast<T>(scale);
    }
}

// src/box_convolution.cpp:740-761, one (min, max) pair; all arithmetic in double except `mean`.
template <class T>
void clip_pair(T& pmin, T& pmax, double reparam, double min_size, double max_size) {
    const double inv = 1.0 / reparam;
    double lo = std::max(-(max_size + 1) * inv, std::min((max_size - 1) * inv, (double)pmin));
    double hi = std::max(-(max_size + 1) * inv, std::min((max_size - 1) * inv, (double)pmax));
    if (lo + (min_size - 0.9999) * inv > hi) {
        const T mean = static_cast<T>(0.5 * (lo + hi));
        lo = mean - 0.5 * (min_size - 0.9999) * inv;
        hi = mean + 0.5 * (min_size - 0.9999) * inv;
    }
    pmin = static_cast<T>(lo);
    pmax = static_cast<T>(hi);
}

template <class T>
void clip_parameters(T* xmin, T* xmax, T* ymin, T* ymax, int n, double reparam_h,
                     double reparam_w, double max_h, double max_w, bool exact) {
    // src/box_convolution_interface.cpp:405-406: float literals widened to double
    const float min_h = exact ? 1.001f : 2.001f;
    const float min_w = exact ? 1.001f : 2.001f;
    for (int i = 0; i < n; ++i) clip_pair(xmin[i], xmax[i], reparam_h, (double)min_h, max_h);
    for (int i = 0; i < n; ++i) clip_pair(ymin[i], ymax[i], reparam_w, (double)min_w, max_w);
}

template <class T>
void split_dump(int variant, const T* p4, int* ints, T* fracs) {
    Split<T> s = variant == 0 ? split_forward(p4[0], p4[1], p4[2], p4[3])
               : variant == 1 ? split_grad_input(p4[0], p4[1], p4[2], p4[3])
                              : split_grad_params(p4[0], p4[1], p4[2], p4[3]);
    ints[0] = s.xlo; ints[1] = s.xhi; ints[2] = s.ylo; ints[3] = s.yhi;
    fracs[0] = s.fxlo; fracs[1] = s.fxhi; fracs[2] = s.fylo; fracs[3] = s.fyhi;
}

template <class T>
void grad_param_planes(const T* integ, const T* xmin, const T* xmax, const T* ymin, const T* ymax,
                       T* tmp, int which, int B, int C, int F, int h, int w, bool exact) {
    const int64_t ipl = (int64_t)(h + 1) * (w + 1), hw = (int64_t)h * w;
    for (int b = 0; b < B; ++b)
        for (int c = 0; c < C; ++c) {
            Plane<T> I{integ + ((int64_t)b * C + c) * ipl, w + 1};
            for (int f = 0; f < F; ++f) {
                const int k = c * F + f;
                const Split<T> s = split_grad_params(xmin[k], xmax[k], ymin[k], ymax[k]);
                T* o = tmp + (((int64_t)b * C + c) * F + f) * hw;
                for (int x = 1; x <= h; ++x)
                    for (int y = 1; y <= w; ++y)
                        o[(int64_t)(x - 1) * w + (y - 1)] =
                            box_grad_param_pixel(I, s, which, x, y, h, w, exact);
            }
        }
}

}  // namespace

#define ORACLE_API(SUFFIX, T)                                                                     \
    extern "C" int oracle_integral_image_##SUFFIX(const T* in, T* out, int64_t planes, int h,    \
                                                  int w) {                                        \
        integral_image<T>(in, out, planes, h, w);                                                 \
        return 0;                                                                                 \
    }                                                                                             \
    extern "C" int oracle_box_forward_##SUFFIX(const T* integ, const T* xmin, const T* xmax,      \
                                               const T* ymin, const T* ymax, T* out, int B,       \
                                               int C, int F, int h, int w, int normalize,         \
                                               int exact) {                                       \
        box_forward<T>(integ, xmin, xmax, ymin, ymax, out, B, C, F, h, w, normalize != 0,         \
                       exact != 0);                                                               \
        return 0;                                                                                 \
    }                                                                                             \
    extern "C" int oracle_box_grad_input_planes_##SUFFIX(                                         \
        const T* gint, const T* xmin, const T* xmax, const T* ymin, const T* ymax, T* tmp, int B, \
        int C, int F, int h, int w, int normalize, int exact) {                                   \
        box_grad_input_planes<T>(gint, xmin, xmax, ymin, ymax, tmp, B, C, F, h, w,                \
                                 normalize != 0, exact != 0);                                     \
        return 0;                                                                                 \
    }                                                                                             \
    extern "C" int oracle_box_grad_param_planes_##SUFFIX(                                         \
        const T* integ, const T* xmin, const T* xmax, const T* ymin, const T* ymax, T* tmp,       \
        int which, int B, int C, int F, int h, int w, int exact) {                                \
        grad_param_planes<T>(integ, xmin, xmax, ymin, ymax, tmp, which, B, C, F, h, w,            \
                             exact != 0);                                                         \
        return 0;                                                                                 \
    }                                                                                             \
    extern "C" int oracle_box_backward_##SUFFIX(                                                  \
        const T* integ, const T* xmin, const T* xmax, const T* ymin, const T* ymax,               \
        const T* grad_out, const T* output, float reparam_h, float reparam_w, int normalize,      \
        int exact, const int* needs, T* grad_in, T* gxmin, T* gxmax, T* gymin, T* gymax, int B,   \
        int C, int F, int h, int w) {                                                             \
        T* gp[4] = {gxmin, gxmax, gymin, gymax};                                                  \
        box_backward<T>(integ, xmin, xmax, ymin, ymax, grad_out, output, reparam_h, reparam_w,    \
                        normalize != 0, exact != 0, needs, grad_in, gp, B, C, F, h, w);           \
        return 0;                                                                                 \
    }                                                                                             \
    extern "C" int oracle_clip_parameters_##SUFFIX(T* xmin, T* xmax, T* ymin, T* ymax, int n,     \
                                                   double reparam_h, double reparam_w,            \
                                                   double max_h, double max_w, int exact) {       \
        clip_parameters<T>(xmin, xmax, ymin, ymax, n, reparam_h, reparam_w, max_h, max_w,         \
                           exact != 0);                                                           \
        return 0;                                                                                 \
    }                                                                                             \
    extern "C" int oracle_split_##SUFFIX(int variant, const T* p4, int* ints, T* fracs) {         \
        split_dump<T>(variant, p4, ints, fracs);                                                  \
        return 0;                                                                                 \
    }

ORACLE_API(f32, float)
ORACLE_API(f64, double)

#define ORACLE_INT_INTEGRAL(SUFFIX, T)                                                            \
    extern "C" int oracle_integral_image_##SUFFIX(const T* in, T* out, int64_t planes, int h,    \
                                                  int w) {                                        \
        integral_image<T>(in, out, planes, h, w);                                                 \
        return 0;                                                                                 \
    }
ORACLE_INT_INTEGRAL(u8, uint8_t)
ORACLE_INT_INTEGRAL(i8, int8_t)
ORACLE_INT_INTEGRAL(i16, int16_t)
ORACLE_INT_INTEGRAL(i32, int32_t)
ORACLE_INT_INTEGRAL(i64, int64_t)
