"""``BoxConv2d``: depthwise convolution with learnable box (rectangular averaging) kernels.

Drop-in for the reference's box_convolution/box_convolution_module.py:6-222: same constructor,
attributes, parameter names/shapes (so ``state_dict``s interchange) and methods.
"""
import random

import torch

from . import _native
from .box_convolution_function import BoxConvolutionFunction, reparametrize


class BoxConv2d(torch.nn.Module):
    """Convolves every input channel with ``num_filters`` box filters whose four bounds are
    learnable real numbers.

    Input ``[B, in_planes, h, w]`` -> output ``[B, in_planes*num_filters, h, w]`` (output channel
    ``c*num_filters + f``). ``x_*`` bounds run along the height axis, ``y_*`` along the width.

    Arguments:
        in_planes, num_filters: channels in, filters per channel.
        max_input_h, max_input_w: expected largest input size; only used to initialise the boxes
            and to clip boxes that grew or drifted too far (``_clip_parameters``).
        reparametrization_factor: parameters are stored divided by
            ``max_input_{h,w} * reparametrization_factor`` so that plain SGD step sizes work.
        stride_h, stride_w: must be 1.
        normalize: ``True`` -> box averages, ``False`` -> box sums.

    Attribute ``exact`` (default ``True``): ``False`` rounds the bounds towards the smaller box
    before filtering (cheaper, no fractional borders).
    """

    def __init__(self, in_planes, num_filters, max_input_h, max_input_w,
                 reparametrization_factor=8, stride_h=1, stride_w=1, normalize=True):
        super().__init__()
        self.in_planes = in_planes
        self.num_filters = num_filters
        self.max_input_h, self.max_input_w = max_input_h, max_input_w
        self.reparametrization_h = max_input_h * reparametrization_factor
        self.reparametrization_w = max_input_w * reparametrization_factor
        self.stride_h, self.stride_w = stride_h, stride_w
        assert stride_h == 1 and stride_w == 1, 'Sorry, strides are NYI'
        self.normalize = normalize
        self.exact = True

        self.x_min, self.x_max, self.y_min, self.y_max = \
            (torch.nn.Parameter(torch.empty(in_planes, num_filters)) for _ in range(4))
        self.reset_parameters()

    def reset_parameters(self):
        """Random boxes centred inside the middle of the image, drawn from Python's global
        ``random`` in the reference's order (per box: centre_h, centre_w, height, width;
        reference box_convolution_module.py:69-97), then stored in reparametrized units."""
        max_h, max_w = self.max_input_h, self.max_input_w
        min_h, min_w = 2, 2
        lim_h, lim_w = max_h * 2 / 4.8, max_w * 2 / 4.8
        rows = [[], [], [], []]
        for _ in range(self.in_planes * self.num_filters):
            center_h = random.uniform(-lim_h + 1 + min_h / 2, lim_h - 1 - min_h / 2)
            center_w = random.uniform(-lim_w + 1 + min_w / 2, lim_w - 1 - min_w / 2)
            height = 2 * random.uniform(
                min_h / 2, min((lim_h - 1) - center_h, center_h - (-lim_h + 1)))
            width = 2 * random.uniform(
                min_w / 2, min((lim_w - 1) - center_w, center_w - (-lim_w + 1)))
            rows[0].append((center_h - height / 2) * 1.5)
            rows[1].append((center_h + height / 2) * 1.5)
            rows[2].append((center_w - width / 2) * 1.5)
            rows[3].append((center_w + width / 2) * 1.5)

        with torch.no_grad():
            for param, values in zip((self.x_min, self.x_max, self.y_min, self.y_max), rows):
                host = torch.tensor(values, dtype=torch.float64).to(param.dtype)
                param.copy_(host.view(self.in_planes, self.num_filters))

        reparametrize(
            self.x_min, self.x_max, self.y_min, self.y_max,
            self.reparametrization_h, self.reparametrization_w, inplace=True)

    # colours of draw_boxes, one per filter (single-channel plots) or per input channel
    _BOX_COLORS = (
        (255, 0, 0), (0, 255, 0), (0, 0, 255), (255, 255, 255), (255, 255, 0), (255, 0, 255),
        (0, 255, 255), (47, 20, 255), (255, 60, 160), (60, 170, 255), (30, 105, 210),
        (222, 196, 176), (212, 255, 127), (250, 206, 135), (50, 205, 50), (0, 165, 255),
        (60, 20, 220), (170, 178, 32))

    def draw_boxes(self, channels=None, resolution=(600, 600), weights=None):
        """Plot the rectangles of the box filters; returns an ``(H, W, 3)`` uint8 numpy array.

        Same arguments, canvas, centre lines, colours, weighting and box -> pixel mapping as the
        reference (box_convolution/box_convolution_module.py:99-181). The reference rasterises
        with ``cv2.rectangle``; here the outlines are drawn with numpy (OpenCV is not a
        dependency), so line pixels may differ from OpenCV's by a pixel at thick lines.

        channels:   input channels to draw boxes for (default: all).
        resolution: ``(h, w)`` of the returned image.
        weights:    ``len(channels) x num_filters`` values in [0, 1]: importance of each box;
                    unimportant boxes are drawn darker. Default: all ones.
        """
        import numpy as np

        if channels is None:
            channels = range(self.in_planes)
        channels = list(channels)
        shape = (len(channels), self.num_filters)
        if weights is None:
            weights = np.ones(shape, dtype=np.float32)
        elif torch.is_tensor(weights):
            weights = weights.detach().cpu().float().numpy()
        weights = np.asarray(weights, dtype=np.float32).reshape(shape).clip(0.01, 1.0)

        height, width = resolution
        image = np.zeros((height, width, 3), dtype=np.uint8)
        center = (height // 2, width // 2)
        image[center[0], :] = 70
        image[:, center[1]] = 70

        x_min, x_max, y_min, y_max = (p.detach().float().cpu() for p in self.get_actual_parameters())
        x_min = x_min / self.max_input_h * (height / 2) + center[0]
        y_min = y_min / self.max_input_w * (width / 2) + center[1]
        x_max = (x_max + 1) / self.max_input_h * (height / 2) + center[0]
        y_max = (y_max + 1) / self.max_input_w * (width / 2) + center[1]

        thickness = int(round(height / 500 + 0.5))

        def fill(r0, r1, c0, c1, color):          # inclusive pixel ranges, clipped to the canvas
            r0, r1 = max(min(r0, r1), 0), min(max(r0, r1), height - 1)
            c0, c1 = max(min(c0, c1), 0), min(max(c0, c1), width - 1)
            if r0 <= r1 and c0 <= c1:
                image[r0:r1 + 1, c0:c1 + 1] = color

        for row, channel in enumerate(channels):
            for f in range(self.num_filters):
                base = self._BOX_COLORS[(f if len(channels) == 1 else channel) % len(self._BOX_COLORS)]
                # (the reference indexes the weights by channel number, test it with all channels)
                color = (np.array(base, dtype=np.float32) * weights[row, f]).astype(np.uint8)
                top, bottom = float(x_min[channel, f]), float(x_max[channel, f])
                left, right = float(y_min[channel, f]), float(y_max[channel, f])
                r0, r1, c0, c1 = (int(round(v)) for v in (top, bottom, left, right))
                if top > bottom or left > right:   # a box of negative size is drawn filled
                    fill(r0, r1, c0, c1, color)
                    continue
                before, after = thickness // 2, (thickness - 1) // 2
                fill(r0 - before, r0 + after, c0 - before, c1 + after, color)
                fill(r1 - before, r1 + after, c0 - before, c1 + after, color)
                fill(r0 - before, r1 + after, c0 - before, c0 + after, color)
                fill(r0 - before, r1 + after, c1 - before, c1 + after, color)
        return image

    def get_actual_parameters(self):
        """The four bounds in real pixel units (new tensors)."""
        return reparametrize(
            self.x_min, self.x_max, self.y_min, self.y_max,
            self.reparametrization_h, self.reparametrization_w, inplace=False, inverse=True)

    def _clip_parameters(self):
        """Projection step after an optimizer update: keep every box within
        ``[-(max_input+1), max_input-1]`` pixels and at least ~1 pixel (2 when ``not exact``)
        thick. In place, outside autograd. (reference box_convolution_module.py:195-206)"""
        _native.clip_parameters(
            self.x_min, self.x_max, self.y_min, self.y_max,
            self.reparametrization_h, self.reparametrization_w,
            self.max_input_h, self.max_input_w, self.exact)

    def train(self, mode=True):
        self.training = mode
        if mode is False:
            self._clip_parameters()
        return self

    _HALF_TYPES = (torch.float16, torch.bfloat16)
    _GLUE_TYPES = (torch.float32, torch.float64)

    # The native library indexes a tensor with 32 bits: batch * in_planes * num_filters *
    # (h+1) * (w+1) must stay below 2^31 (include/boxconv.h, BOXCONV_E_TOO_LARGE).
    _MAX_ELEMENTS = 2 ** 31 - 1

    def _batch_limit(self, input):
        """How many batch items one native call can take (None: no limit applies)."""
        if input.dim() != 4 or not input.is_cuda:
            return None
        per_item = self.in_planes * max(self.num_filters, 1) * (input.size(2) + 1) * (input.size(3) + 1)
        limit = self._MAX_ELEMENTS // max(per_item, 1)
        return limit if 1 <= limit < input.size(0) else None

    def forward(self, input):
        limit = self._batch_limit(input)
        if limit is not None:
            # A batch too large for one native call goes through in slices: box convolution is
            # independent per batch item, and autograd adds the slices' parameter gradients up.
            # (The clip of a training-mode forward is a projection: repeating it changes nothing.)
            return torch.cat([self.forward(part) for part in input.split(limit, dim=0)], dim=0)
        if input.dtype in self._HALF_TYPES:
            return self._forward_half(input)
        clip_to = None
        native = self.x_min.is_cuda and input.is_cuda and input.dim() == 4 and input.dtype == self.x_min.dtype
        if native and _native.glue() is not None and input.dtype in self._GLUE_TYPES:
            # the whole call's host side in C++ (same native calls, autograd node included); the
            # parameters are clipped on the way in only in training mode
            return _native.training_step(
                input, self.x_min, self.x_max, self.y_min, self.y_max,
                self.reparametrization_h, self.reparametrization_w,
                self.max_input_h, self.max_input_w, self.normalize, self.exact, clip=self.training)
        if self.training:
            if native:
                # the projection rides along in the native forward call
                clip_to = (self.max_input_h, self.max_input_w)
            else:
                self._clip_parameters()

        return BoxConvolutionFunction.apply(
            input, self.x_min, self.x_max, self.y_min, self.y_max,
            self.reparametrization_h, self.reparametrization_w, self.normalize, self.exact,
            clip_to)

    def _forward_half(self, input):
        """float16 / bfloat16 input (not offered by the reference's CPU path, and its CUDA path
        would integrate in half precision): the integral image and all sums are float32, and the
        kernels read and write the half type directly, forward and backward (grad_output is
        widened as it is loaded, grad_input rounded once in the store; parameter gradients are
        float32, or the parameters' own half type after ``module.half()``)."""
        params = (self.x_min, self.x_max, self.y_min, self.y_max)
        h, w = input.shape[-2:]
        if (input.is_cuda and input.dim() == 4 and self.x_min.is_cuda and self.x_min.dtype == torch.float32
                and _native.glue() is not None and _native.half_rows_read_directly(h, w)):
            # the whole call's host side in C++, as for float32 (same native kernels)
            return _native.training_step(
                input, *params, self.reparametrization_h, self.reparametrization_w,
                self.max_input_h, self.max_input_w, self.normalize, self.exact, clip=self.training)
        if torch.is_grad_enabled() and (input.requires_grad or any(p.requires_grad for p in params)):
            clip_to = (self.max_input_h, self.max_input_w) if self.training else None
            return BoxConvolutionFunction.apply(
                input, *params, self.reparametrization_h, self.reparametrization_w,
                self.normalize, self.exact, clip_to)
        if self.training:
            self._clip_parameters()
        return self.forward_fused(input)

    def forward_fused(self, input, channel_scale=None, channel_shift=None, residual=None,
                      relu=False, output_dtype=None):
        """Inference-only forward with the next element-wise steps of a block folded into the
        kernel's store: ``y = boxconv(input) * channel_scale[ch] + channel_shift[ch] + residual``,
        then ``max(y, 0)`` if ``relu``. That is the tail of the reference's BottleneckBoxConv in
        eval mode (BoxConv2d -> BatchNorm2d -> Dropout2d -> ``+ x`` -> ReLU,
        examples/Cityscapes/models/ENet.py:290-304); ``fold_batch_norm`` turns an eval-mode
        BatchNorm2d into the two per-channel vectors.

        ``input`` may be float32, float16 or bfloat16; the integral image and the sums are
        float32, the result is ``output_dtype`` (default: the input's). Not differentiable."""
        if output_dtype is None:
            output_dtype = input.dtype
        with torch.no_grad():
            real = reparametrize(
                self.x_min.float(), self.x_max.float(), self.y_min.float(), self.y_max.float(),
                self.reparametrization_h, self.reparametrization_w, inverse=True)
            if input.dtype == torch.float64:
                input = input.float()
            integrated = _native.integral_image(input)       # float32 also for half-precision input
            return _native.box_convolution_forward_fused(
                integrated, *real, self.normalize, self.exact, output_dtype,
                channel_scale, channel_shift, residual, relu)

    @staticmethod
    def fold_batch_norm(batch_norm):
        """``(scale, shift)`` with ``batch_norm(x) == x * scale[ch] + shift[ch]`` in eval mode."""
        with torch.no_grad():
            scale = torch.rsqrt(batch_norm.running_var.float() + batch_norm.eps)
            if batch_norm.weight is not None:
                scale = scale * batch_norm.weight.float()
            shift = -batch_norm.running_mean.float() * scale
            if batch_norm.bias is not None:
                shift = shift + batch_norm.bias.float()
        return scale, shift
