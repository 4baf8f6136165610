"""Autograd glue: ``reparametrize`` and ``BoxConvolutionFunction``.

Same public surface as the reference's box_convolution/box_convolution_function.py:5-65; the
native calls go to the HIP library instead of ``box_convolution_cpp_cuda``.
"""
import torch

from . import _native


def reparametrize(
        x_min, x_max, y_min, y_max, reparametrization_h, reparametrization_w,
        inplace=False, inverse=False):
    """Convert box bounds between stored units (about [-1, 1], friendly to SGD step sizes) and
    real pixel units. ``inverse=False``: real -> stored (divide); ``inverse=True``: stored -> real.

    With ``inplace`` the four tensors are modified and nothing is returned; otherwise four new
    tensors are returned. Never recorded by autograd.
    (reference box_convolution_function.py:5-27)
    """
    scale_h = reparametrization_h if inverse else (1 / reparametrization_h)
    scale_w = reparametrization_w if inverse else (1 / reparametrization_w)

    with torch.no_grad():
        if inplace:
            x_min *= scale_h
            x_max *= scale_h
            y_min *= scale_w
            y_max *= scale_w
            return None
        # one multi-tensor launch instead of four; element-wise identical to `t * scale`
        return tuple(torch._foreach_mul([x_min, x_max, y_min, y_max],
                                        [scale_h, scale_h, scale_w, scale_w]))


class BoxConvolutionFunction(torch.autograd.Function):
    """``apply(input, x_min, x_max, y_min, y_max, reparametrization_h, reparametrization_w,
    normalize, exact) -> output [B, C*F, h, w]``; parameters in stored units.
    (reference box_convolution_function.py:30-65)

    One optional trailing argument that the reference does not have: ``clip_to``, the pair
    ``(max_input_h, max_input_w)``. When given, the stored parameters are first clipped in place
    to those limits (what ``BoxConv2d.forward`` does in training mode before calling ``apply``),
    and clip, unit conversion, integral image and sampling run as one native call.
    """

    @staticmethod
    def forward(ctx, input, x_min, x_max, y_min, y_max,
                reparametrization_h, reparametrization_w, normalize, exact, clip_to=None):
        ctx.normalize = normalize
        ctx.reparametrization_h = reparametrization_h
        ctx.reparametrization_w = reparametrization_w
        ctx.exact = exact

        ctx.param_dtype = x_min.dtype
        if input.dtype in (torch.float16, torch.bfloat16):
            # half-precision input: float32 integral image and sums, read and written by the
            # kernels in the half type (no float32 copies of input, output or their gradients);
            # the bounds are used in float32
            if clip_to is not None:
                _native.clip_parameters(x_min.detach(), x_max.detach(), y_min.detach(), y_max.detach(),
                                        reparametrization_h, reparametrization_w, clip_to[0],
                                        clip_to[1], exact)
            x_min, x_max, y_min, y_max = reparametrize(
                x_min.float(), x_max.float(), y_min.float(), y_max.float(),
                reparametrization_h, reparametrization_w, inverse=True)
            input_integrated = _native.integral_image(input)
            output = _native.box_convolution_forward_fused(
                input_integrated, x_min, x_max, y_min, y_max, normalize, exact, input.dtype)
        elif clip_to is not None:
            # (the native call only takes the parameters' addresses: nothing autograd could record)
            input_integrated, output, (x_min, x_max, y_min, y_max) = _native.training_forward(
                input, x_min, x_max, y_min, y_max,
                reparametrization_h, reparametrization_w, clip_to[0], clip_to[1], normalize, exact)
        else:
            x_min, x_max, y_min, y_max = reparametrize(
                x_min, x_max, y_min, y_max, reparametrization_h, reparametrization_w, inverse=True)
            input_integrated = _native.integral_image(input)
            output = _native.box_convolution_forward(
                input_integrated, x_min, x_max, y_min, y_max, normalize, exact)

        # The saved forward output of the reference is not kept: the backward kernels rebuild the
        # one sum that needs it from the integral image.
        ctx.save_for_backward(input_integrated, x_min, x_max, y_min, y_max)
        return output

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_output):
        input_integrated, x_min, x_max, y_min, y_max = ctx.saved_tensors
        grads = _native.box_convolution_backward(
            input_integrated, x_min, x_max, y_min, y_max, grad_output, None,
            ctx.reparametrization_h, ctx.reparametrization_w,
            ctx.normalize, ctx.exact, *ctx.needs_input_grad[:5])
        if ctx.param_dtype != input_integrated.dtype:     # half-precision parameters
            grads = [grads[0]] + [None if g is None else g.to(ctx.param_dtype) for g in grads[1:]]
        # no gradients for reparametrization_h, reparametrization_w, normalize, exact, clip_to
        return tuple(grads) + (None,) * 5
