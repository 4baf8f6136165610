// TEST INFRASTRUCTURE, NOT PRODUCT CODE. Built only where /root/reference exists.
//
// C-ABI driver around the reference's own CPU kernels. oracle/build_ref.sh compiles
// /root/reference/src/integral_image.cpp and /root/reference/src/box_convolution.cpp *where they
// lie* (no copy enters this repository) and links them with this file into
// oracle/_ref/libboxconv_ref.so. The kernels in namespace cpu:: are therefore the reference's
// machine code; what this file adds is the host orchestration of
// src/box_convolution_interface.cpp:13-139 (forward), :141-395 (backward) and :397-415 (clip),
// written against the same ATen calls (sum, mul_, addcmul_) because that file itself cannot be
// compiled here: it includes <TH/THGeneral.h>, which torch 2.10 no longer ships.
//
// Exported symbols mirror oracle/boxconv_oracle.cpp with the prefix ref_ so that one Python
// wrapper drives both.

#include <ATen/ATen.h>

#include <cstdint>
#include <cstring>
#include <vector>

#include "box_convolution.h"   // from /root/reference/src (include path set by build_ref.sh)
#include "integral_image.h"

namespace {

template <class T>
at::Tensor view_of(const T* p, at::IntArrayRef sizes) {
    return at::from_blob(const_cast<T*>(p), sizes,
                         at::TensorOptions().dtype(c10::CppTypeToScalarType<T>::value));
}

struct SplitBuffers {
    at::Tensor xi, Xi, yi, Yi, xf, Xf, yf, Yf;
    explicit SplitBuffers(const at::Tensor& like) {
        auto io = like.options().dtype(at::kInt);
        xi = at::empty(like.sizes(), io); Xi = at::empty(like.sizes(), io);
        yi = at::empty(like.sizes(), io); Yi = at::empty(like.sizes(), io);
        xf = at::empty_like(like); Xf = at::empty_like(like);
        yf = at::empty_like(like); Yf = at::empty_like(like);
    }
};

#define BOOL2_DISPATCH(FN, n, e, ...)                         \
    do {                                                      \
        if (n) { if (e) FN<true, true>(__VA_ARGS__); else FN<true, false>(__VA_ARGS__); } \
        else   { if (e) FN<false, true>(__VA_ARGS__); else FN<false, false>(__VA_ARGS__); } \
    } while (0)

template <class T>
void forward_impl(const T* integ, const T* xmin, const T* xmax, const T* ymin, const T* ymax,
                  T* out, int B, int C, int F, int h, int w, bool normalize, bool exact) {
    at::Tensor I = view_of(integ, {B, C, h + 1, w + 1});
    at::Tensor a = view_of(xmin, {C, F}), b = view_of(xmax, {C, F});
    at::Tensor c = view_of(ymin, {C, F}), d = view_of(ymax, {C, F});
    SplitBuffers s(a);
    cpu::splitParameters(a, b, c, d, s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf);
    at::Tensor area;
    if (normalize) area = cpu::computeArea(a, b, c, d, exact);
    at::Tensor o = view_of(out, {B, C, F, h, w});
    BOOL2_DISPATCH(cpu::boxConvUpdateOutput, normalize, exact,
                   s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf, area, I, o);
}

template <class T>
void grad_input_planes_impl(const T* gint, const T* xmin, const T* xmax, const T* ymin,
                            const T* ymax, T* tmp, int B, int C, int F, int h, int w,
                            bool normalize, bool exact) {
    at::Tensor G = view_of(gint, {B, C, F, h + 1, w + 1});
    at::Tensor a = view_of(xmin, {C, F}), b = view_of(xmax, {C, F});
    at::Tensor c = view_of(ymin, {C, F}), d = view_of(ymax, {C, F});
    SplitBuffers s(a);
    cpu::splitParametersUpdateGradInput(a, b, c, d, s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf);
    at::Tensor area;
    if (normalize) area = cpu::computeArea(a, b, c, d, exact);
    at::Tensor o = view_of(tmp, {B, C, F, h, w});
    BOOL2_DISPATCH(cpu::boxConvUpdateGradInput, normalize, exact,
                   s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf, area, G, o);
}

template <class T>
void grad_param_planes_impl(const T* integ, const T* xmin, const T* xmax, const T* ymin,
                            const T* ymax, T* tmp, int which, int B, int C, int F, int h, int w,
                            bool exact) {
    at::Tensor I = view_of(integ, {B, C, h + 1, w + 1});
    at::Tensor a = view_of(xmin, {C, F}), b = view_of(xmax, {C, F});
    at::Tensor c = view_of(ymin, {C, F}), d = view_of(ymax, {C, F});
    SplitBuffers s(a);
    cpu::splitParametersAccGradParameters(a, b, c, d, s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf);
    at::Tensor o = view_of(tmp, {B, C, F, h, w});
    const Parameter p = static_cast<Parameter>(which);
    if (exact) cpu::boxConvAccGradParameters<true>(s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf, I, o, p);
    else       cpu::boxConvAccGradParameters<false>(s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf, I, o, p);
}

template <class T>
void backward_impl(const T* integ, const T* xmin, const T* xmax, const T* ymin, const T* ymax,
                   const T* grad_out, const T* output, float reparam_h, float reparam_w,
                   bool normalize, bool exact, const int* needs, T* grad_in, T* const* gparam,
                   int B, int C, int F, int h, int w) {
    at::Tensor I = view_of(integ, {B, C, h + 1, w + 1});
    at::Tensor a = view_of(xmin, {C, F}), b = view_of(xmax, {C, F});
    at::Tensor c = view_of(ymin, {C, F}), d = view_of(ymax, {C, F});
    at::Tensor go = view_of(grad_out, {B, C, F, h, w});
    SplitBuffers s(a);

    if (needs[0]) {
        at::Tensor gint = at::empty({B, C, F, h + 1, w + 1}, go.options());
        cpu::integral_image(go, gint);
        at::Tensor tmp = at::empty({B, C, F, h, w}, go.options());
        cpu::splitParametersUpdateGradInput(a, b, c, d, s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf);
        at::Tensor area;
        if (normalize) area = cpu::computeArea(a, b, c, d, exact);
        BOOL2_DISPATCH(cpu::boxConvUpdateGradInput, normalize, exact,
                       s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf, area, gint, tmp);
        at::Tensor gi = tmp.sum(2);
        view_of(grad_in, {B, C, h, w}).copy_(gi);
    }

    if (!(needs[1] | needs[2] | needs[3] | needs[4])) return;

    at::Tensor grads[4];
    at::Tensor tmp = at::empty({B, C, F, h, w}, a.options());
    cpu::splitParametersAccGradParameters(a, b, c, d, s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf);
    at::Tensor area;
    if (normalize) area = cpu::computeArea(a, b, c, d, exact);

    for (int k = 0; k < 4; ++k) {
        if (!needs[1 + k]) continue;
        const Parameter p = static_cast<Parameter>(k);
        if (exact) cpu::boxConvAccGradParameters<true>(s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf, I, tmp, p);
        else       cpu::boxConvAccGradParameters<false>(s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf, I, tmp, p);
        tmp.mul_(go);
        grads[k] = tmp.reshape({B, C, F, (int64_t)h * w}).sum(c10::IntArrayRef({0, 3}));
        if (normalize) grads[k].mul_(area);
    }

    if (normalize) {
        at::Tensor out5 = view_of(output, {B, C, F, h, w});
        at::Tensor prod = go.mul(out5);
        prod = prod.reshape({B, C, F, (int64_t)h * w}).sum(c10::IntArrayRef({0, 3}));
        for (int k = 0; k < 4; ++k) {
            if (!needs[1 + k]) continue;
            const bool is_x = k < 2;
            at::Tensor inv = cpu::computeArea(a, b, c, d, exact, is_x, !is_x);
            grads[k].addcmul_(prod, inv, (k == 1 || k == 3) ? -1.0 : 1.0);
        }
    }

    for (int k = 0; k < 4; ++k) {
        if (!needs[1 + k]) continue;
        const double scale = k < 2 ? reparam_h : reparam_w;
        grads[k].mul_(scale);
        view_of(gparam[k], {C, F}).copy_(grads[k]);
    }
}

template <class T>
void clip_impl(T* xmin, T* xmax, T* ymin, T* ymax, int n, double reparam_h, double reparam_w,
               double max_h, double max_w, bool exact) {
    at::Tensor a = view_of(xmin, {n}), b = view_of(xmax, {n});
    at::Tensor c = view_of(ymin, {n}), d = view_of(ymax, {n});
    const float min_w = exact ? 1.001f : 2.001f;
    const float min_h = exact ? 1.001f : 2.001f;
    cpu::clipParameters(a, b, reparam_h, min_h, max_h);
    cpu::clipParameters(c, d, reparam_w, min_w, max_w);
}

template <class T>
void split_impl(int variant, const T* p4, int* ints, T* fracs) {
    at::Tensor a = view_of(p4 + 0, {1, 1}), b = view_of(p4 + 1, {1, 1});
    at::Tensor c = view_of(p4 + 2, {1, 1}), d = view_of(p4 + 3, {1, 1});
    SplitBuffers s(a);
    if (variant == 0) cpu::splitParameters(a, b, c, d, s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf);
    else if (variant == 1) cpu::splitParametersUpdateGradInput(a, b, c, d, s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf);
    else cpu::splitParametersAccGradParameters(a, b, c, d, s.xi, s.Xi, s.yi, s.Yi, s.xf, s.Xf, s.yf, s.Yf);
    ints[0] = s.xi.item<int>(); ints[1] = s.Xi.item<int>();
    ints[2] = s.yi.item<int>(); ints[3] = s.Yi.item<int>();
    fracs[0] = s.xf.item<T>(); fracs[1] = s.Xf.item<T>();
    fracs[2] = s.yf.item<T>(); fracs[3] = s.Yf.item<T>();
}

}  // namespace

#define REF_API(SUFFIX, T)                                                                        \
    extern "C" int ref_integral_image_##SUFFIX(const T* in, T* out, int64_t planes, int h,       \
                                               int w) {                                           \
        at::Tensor i = view_of(in, {planes, h, w});                                               \
        at::Tensor o = view_of(out, {planes, h + 1, w + 1});                                      \
        cpu::integral_image(i, o);                                                                \
        return 0;                                                                                 \
    }                                                                                             \
    extern "C" int ref_box_forward_##SUFFIX(const T* integ, const T* xmin, const T* xmax,         \
                                            const T* ymin, const T* ymax, T* out, int B, int C,   \
                                            int F, int h, int w, int normalize, int exact) {      \
        forward_impl<T>(integ, xmin, xmax, ymin, ymax, out, B, C, F, h, w, normalize != 0,        \
                        exact != 0);                                                              \
        return 0;                                                                                 \
    }                                                                                             \
    extern "C" int ref_box_grad_input_planes_##SUFFIX(                                            \
        const T* gint, const T* xmin, const T* xmax, const T* ymin, const T* ymax, T* tmp, int B, \
        int C, int F, int h, int w, int normalize, int exact) {                                   \
        grad_input_planes_impl<T>(gint, xmin, xmax, ymin, ymax, tmp, B, C, F, h, w,               \
                                  normalize != 0, exact != 0);                                    \
        return 0;                                                                                 \
    }                                                                                             \
    extern "C" int ref_box_grad_param_planes_##SUFFIX(                                            \
        const T* integ, const T* xmin, const T* xmax, const T* ymin, const T* ymax, T* tmp,       \
        int which, int B, int C, int F, int h, int w, int exact) {                                \
        grad_param_planes_impl<T>(integ, xmin, xmax, ymin, ymax, tmp, which, B, C, F, h, w,       \
                                  exact != 0);                                                    \
        return 0;                                                                                 \
    }                                                                                             \
    extern "C" int ref_box_backward_##SUFFIX(                                                     \
        const T* integ, const T* xmin, const T* xmax, const T* ymin, const T* ymax,               \
        const T* grad_out, const T* output, float reparam_h, float reparam_w, int normalize,      \
        int exact, const int* needs, T* grad_in, T* gxmin, T* gxmax, T* gymin, T* gymax, int B,   \
        int C, int F, int h, int w) {                                                             \
        T* gp[4] = {gxmin, gxmax, gymin, gymax};                                                  \
        backward_impl<T>(integ, xmin, xmax, ymin, ymax, grad_out, output, reparam_h, reparam_w,   \
                         normalize != 0, exact != 0, needs, grad_in, gp, B, C, F, h, w);          \
        return 0;                                                                                 \
    }                                                                                             \
    extern "C" int ref_clip_parameters_##SUFFIX(T* xmin, T* xmax, T* ymin, T* ymax, int n,        \
                                                double reparam_h, double reparam_w,               \
                                                double max_h, double max_w, int exact) {          \
        clip_impl<T>(xmin, xmax, ymin, ymax, n, reparam_h, reparam_w, max_h, max_w, exact != 0);  \
        return 0;                                                                                 \
    }                                                                                             \
    extern "C" int ref_split_##SUFFIX(int variant, const T* p4, int* ints, T* fracs) {            \
        split_impl<T>(variant, p4, ints, fracs);                                                  \
        return 0;                                                                                 \
    }

REF_API(f32, float)
REF_API(f64, double)

// the reference's integral image of integer tensors (AT_DISPATCH_ALL_TYPES)
#define REF_INT_INTEGRAL(SUFFIX, T)                                                               \
    extern "C" int ref_integral_image_##SUFFIX(const T* in, T* out, int64_t planes, int h,       \
                                               int w) {                                           \
        at::Tensor i = view_of(in, {planes, h, w});                                               \
        at::Tensor o = view_of(out, {planes, h + 1, w + 1});                                      \
        cpu::integral_image(i, o);                                                                \
        return 0;                                                                                 \
    }
REF_INT_INTEGRAL(u8, uint8_t)
REF_INT_INTEGRAL(i8, int8_t)
REF_INT_INTEGRAL(i16, int16_t)
REF_INT_INTEGRAL(i32, int32_t)
REF_INT_INTEGRAL(i64, int64_t)
