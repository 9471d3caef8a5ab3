"""Import surface of the reference package (wtconv/__init__.py:1), backed by the HIP kernels."""
from .wtconv2d import WTConv2d
