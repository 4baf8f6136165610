"""Box convolution for AMD MI355X (gfx950): ``from box_convolution import BoxConv2d``."""
from .box_convolution_module import BoxConv2d

__all__ = ["BoxConv2d"]
