"""MI355X-native WTConv layer: hand-written gfx950 HIP kernels behind the reference's
module API.  ``WTConv2d`` / ``WTConv1d`` mirror ``wtconv.WTConv2d`` / ``wtconv.wtconv1d.WTConv1d``;
``FastWTConv2d`` mirrors ``fast_wtconv.wtconv_cuda.WTConv2d``."""
from .functional import check_kernel_size, wtconv1d, wtconv2d
from .modules import FastWTConv2d, WTConv1d, WTConv2d

__all__ = ["WTConv2d", "WTConv1d", "FastWTConv2d", "wtconv2d", "wtconv1d", "check_kernel_size"]
