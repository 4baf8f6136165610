"""The two places the reference's own examples use BoxConv2d, as GPU smoke tests on synthetic
tensors (no dataset, no torchvision, no OpenCV):

* the MNIST classifier, BoxConv2d(1, 40, 28, 28) -> 1x1 convolution -> max-pool 4 + ReLU -> linear
  -> log-softmax (reference examples/mnist.py:17-31), trained for a few SGD steps: the loss must
  go down and the boxes must move;
* the block of the segmentation networks, 1x1 convolution -> BatchNorm -> ReLU -> BoxConv2d ->
  BatchNorm -> Dropout2d -> + x -> ReLU in training mode
  (reference examples/Cityscapes/models/ENet.py:282-304): forward and every gradient against the
  same stack with the box convolution replaced by a dense depthwise convolution whose kernels are
  the boxes' pixel-coverage weights (what the reference's test compares with, test.py:60-134).
"""
import math
import random

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from box_convolution import BoxConv2d

pytestmark = pytest.mark.gpu
DEV = "cuda"


class MnistNet(nn.Module):
    def __init__(self):
        super().__init__()
        self.conv1 = BoxConv2d(1, 40, 28, 28)
        self.conv1_1x1 = nn.Conv2d(40, 40, 1, 1)
        self.fc1 = nn.Linear(7 * 7 * 40, 10)

    def forward(self, x):
        x = self.conv1_1x1(self.conv1(x))
        x = F.relu(F.max_pool2d(x, 4))
        return F.log_softmax(self.fc1(x.view(-1, 7 * 7 * 40)), dim=1)


def synthetic_digits(n, generator):
    """n images of 28x28 in [0,1] whose class (0..9) is where a bright blob sits and how wide it
    is: something box filters can tell apart."""
    labels = torch.randint(0, 10, (n,), generator=generator)
    yy, xx = torch.meshgrid(torch.arange(28.0), torch.arange(28.0), indexing="ij")
    images = torch.rand(n, 1, 28, 28, generator=generator) * 0.2
    for i, c in enumerate(labels.tolist()):
        cy, cx = 6 + 4 * (c % 5), 8 + 12 * (c // 5)
        images[i, 0] += torch.exp(-((yy - cy) ** 2 + (xx - cx) ** 2) / (2.0 * (1.5 + 0.3 * c) ** 2))
    return images.clamp_(0, 1), labels


def test_mnist_example_network_trains():
    random.seed(7)
    torch.manual_seed(7)
    gen = torch.Generator().manual_seed(7)
    net = MnistNet().to(DEV)
    images, labels = synthetic_digits(256, gen)
    images, labels = images.to(DEV), labels.to(DEV)
    opt = torch.optim.Adam(net.parameters(), lr=3e-3)
    boxes_before = [p.detach().clone() for p in (net.conv1.x_min, net.conv1.x_max,
                                                  net.conv1.y_min, net.conv1.y_max)]
    net.train()
    losses = []
    for step in range(80):
        idx = torch.arange(64, device=DEV) + 64 * (step % 4)
        opt.zero_grad()
        loss = F.nll_loss(net(images[idx]), labels[idx])
        loss.backward()
        for p in net.parameters():
            assert p.grad is not None and torch.isfinite(p.grad).all()
        opt.step()
        losses.append(loss.item())
    assert all(math.isfinite(v) for v in losses)
    print("loss every 8 steps:", ["%.3f" % v for v in losses[::8]])
    assert sum(losses[-4:]) / 4 < 0.5 * sum(losses[:4]) / 4, ["%.3f" % v for v in losses]
    moved = [(a - b).abs().max().item() for a, b in zip(
        (net.conv1.x_min, net.conv1.x_max, net.conv1.y_min, net.conv1.y_max), boxes_before)]
    assert min(moved) > 0, "every box bound must have received gradient steps"
    net.eval()
    with torch.no_grad():
        acc = (net(images).argmax(1) == labels).float().mean().item()
    assert acc > 0.5, acc


def coverage(lo, hi, size):
    """[n, 2*size+1] weights: how much of pixel offset d (-size..size) the interval [lo, hi+1) covers."""
    d = torch.arange(-size, size + 1, dtype=lo.dtype, device=lo.device)[None, :]
    return (torch.minimum(hi[:, None] + 1, d + 1) - torch.maximum(lo[:, None], d)).clamp_min(0)


class DenseBoxConv(nn.Module):
    """The same function as BoxConv2d, computed as a dense depthwise convolution whose kernels are
    built from the four (stored) bounds with differentiable torch operations, so that autograd
    gives the reference gradients for the input and for the bounds."""

    def __init__(self, box):
        super().__init__()
        self.C, self.F, self.h, self.w = box.in_planes, box.num_filters, box.max_input_h, box.max_input_w
        self.rh, self.rw = box.reparametrization_h, box.reparametrization_w
        for name in ("x_min", "x_max", "y_min", "y_max"):
            setattr(self, name, nn.Parameter(getattr(box, name).detach().clone()))

    def forward(self, x):
        xmin, xmax = (self.x_min * self.rh).reshape(-1), (self.x_max * self.rh).reshape(-1)
        ymin, ymax = (self.y_min * self.rw).reshape(-1), (self.y_max * self.rw).reshape(-1)
        rows, cols = coverage(xmin, xmax, self.h), coverage(ymin, ymax, self.w)
        area = (xmax - xmin + 1) * (ymax - ymin + 1)
        kernel = rows[:, :, None] * cols[:, None, :] / area[:, None, None]
        return F.conv2d(x, kernel[:, None], padding=(self.h, self.w), groups=self.C)


class Bottleneck(nn.Module):
    def __init__(self, in_channels, num_boxes, max_input_h, max_input_w, dropout_prob=0.0,
                 reparam_factor=1.5625):
        super().__init__()
        bt = in_channels // num_boxes
        self.main_branch = nn.Sequential(
            nn.Conv2d(in_channels, bt, (1, 1), bias=False),
            nn.BatchNorm2d(bt),
            nn.ReLU(True),
            BoxConv2d(bt, num_boxes, max_input_h, max_input_w, reparametrization_factor=reparam_factor),
            nn.BatchNorm2d(in_channels),
            nn.Dropout2d(dropout_prob))

    def forward(self, x):
        return (x + self.main_branch(x)).relu_()


@pytest.mark.parametrize("in_channels,num_boxes,h,w", [(16, 4, 24, 40), (8, 2, 33, 20)])
def test_bottleneck_block_training_step_matches_dense_convolution(in_channels, num_boxes, h, w):
    random.seed(3)
    torch.manual_seed(3)
    block = Bottleneck(in_channels, num_boxes, h, w).to(DEV).double()
    dense = Bottleneck(in_channels, num_boxes, h, w).to(DEV).double()
    dense.load_state_dict(block.state_dict())
    block.train()
    dense.train()
    box = block.main_branch[3]
    box._clip_parameters()                       # what the first training forward will do anyway
    dense.main_branch[3] = DenseBoxConv(box).to(DEV)
    x = torch.randn(3, in_channels, h, w, device=DEV, dtype=torch.float64)
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    ya, yb = block(xa), dense(xb)
    assert torch.allclose(ya, yb, rtol=1e-9, atol=1e-9)
    go = torch.randn_like(ya)
    ya.backward(go)
    yb.backward(go)
    assert torch.allclose(xa.grad, xb.grad, rtol=1e-8, atol=1e-9)
    pa, pb = dict(block.named_parameters()), dict(dense.named_parameters())
    assert set(pa) == set(pb)
    for name in pa:
        scale = pb[name].grad.abs().max().item() + 1e-12
        assert (pa[name].grad - pb[name].grad).abs().max().item() <= 1e-7 * scale, name
    # BatchNorm's running statistics moved the same way
    for (na, ba), (nb_, bb) in zip(block.named_buffers(), dense.named_buffers()):
        assert na == nb_ and torch.allclose(ba.double(), bb.double(), rtol=1e-9, atol=1e-9)


def test_bottleneck_block_float32_smoke():
    """The same block in float32 at a segmentation-network shape: a few optimiser steps run and
    reduce a regression loss."""
    random.seed(5)
    torch.manual_seed(5)
    block = Bottleneck(64, 4, 64, 128, dropout_prob=0.1).to(DEV)
    opt = torch.optim.Adam(block.parameters(), lr=1e-3)
    x = torch.randn(2, 64, 64, 128, device=DEV)
    target = torch.relu(torch.roll(x, shifts=(3, -5), dims=(2, 3)))
    block.train()
    losses = []
    for _ in range(12):
        opt.zero_grad()
        loss = F.mse_loss(block(x), target)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert all(math.isfinite(v) for v in losses) and losses[-1] < losses[0], losses
