"""``from fast_wtconv.wtconv_cuda import WTConv2d`` keeps working on ROCm, where the torch
device type is still "cuda"; the class is the gfx950 HIP implementation."""
from wtconv_amd.modules import FastWTConv2d as WTConv2d  # noqa: F401
