"""Import surface of the reference's fast_wtconv package; one HIP implementation, no dispatch."""
from .wtconv_cuda import WTConv2d  # noqa: F401
