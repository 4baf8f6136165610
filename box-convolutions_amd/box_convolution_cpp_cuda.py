"""Stand-in for the reference's native module ``box_convolution_cpp_cuda`` (reference
src/bind.cpp:29-34) for callers that import it directly: the same four functions, backed by the
HIP library. ``box_convolution_backward`` returns 0-element tensors for gradients that were not
requested, as the reference does (src/box_convolution_interface.cpp:181-183,394)."""
import torch

from box_convolution import _native

integral_image = _native.integral_image
box_convolution_forward = _native.box_convolution_forward
clip_parameters = _native.clip_parameters


def box_convolution_backward(input_integrated, x_min, x_max, y_min, y_max, grad_output, output,
                             reparametrization_h, reparametrization_w, normalize, exact,
                             input_needs_grad, x_min_needs_grad, x_max_needs_grad,
                             y_min_needs_grad, y_max_needs_grad):
    grads = _native.box_convolution_backward(
        input_integrated, x_min, x_max, y_min, y_max, grad_output, output,
        reparametrization_h, reparametrization_w, normalize, exact,
        input_needs_grad, x_min_needs_grad, x_max_needs_grad, y_min_needs_grad, y_max_needs_grad)
    return [torch.empty(0) if g is None else g for g in grads]
