"""Import path of the fast twin's operator-level utilities (fast_wtconv/cuda_haar/__init__.py:8-67 of the reference),
as far as they exist as operators here: the single-level Haar transforms and the kernel-size check.  The reference's
fused pieces (wavelet_branch, fused_haar_conv_scale, the multi-level ihaar2d_* cascades, scaled_depthwise_conv) are
stages of its two-kernel layer; here the layer is one kernel (fast_wtconv.wtconv_cuda.WTConv2d), so they have no
counterpart of their own."""
import torch
import torch.nn.functional as F

from wtconv_amd import _lib
from wtconv_amd.wavelet import _Haar, _prep

MAX_KERNEL_SIZE = 7             # wtconv_max_kernel_size() of the built library (haar_cuda.py:62: the default ceiling)
HARD_MAX_KERNEL_SIZE = 7        # the kernels are instantiated for K = 1, 3, 5, 7; nothing larger can be built in


def check_kernel_size(kernel_size: int) -> None:
    """Reject kernel sizes the kernels do not cover (haar_cuda.py:86-105)."""
    K = int(kernel_size)
    if K < 1 or K % 2 == 0:
        raise ValueError(f"kernel_size must be odd and positive, got {K}")
    if K > MAX_KERNEL_SIZE:
        raise ValueError(f"kernel_size must be <= {MAX_KERNEL_SIZE}, got {K}")


def haar2d(x: torch.Tensor) -> torch.Tensor:
    """(B, C, H, W) -> (B, C, 4, ceil(H/2), ceil(W/2)), sub-bands [LL, LH, HL, HH]; odd extents are zero padded on the
    right / bottom (haar_cuda.py:597-599)."""
    x = _prep(x, 4, "haar2d")
    if x.shape[2] % 2 or x.shape[3] % 2:
        x = F.pad(x, (0, x.shape[3] % 2, 0, x.shape[2] % 2))
    return _Haar.apply(x, 2, False)


def ihaar2d(x: torch.Tensor, output_size=None) -> torch.Tensor:
    """(B, C, 4, h, w) -> (B, C, 2h, 2w), cropped to `output_size` (H, W) if given (haar_cuda.py:536-537)."""
    out = _Haar.apply(_prep(x, 5, "ihaar2d"), 2, True)
    if output_size is not None:
        out = out[:, :, :output_size[0], :output_size[1]]
    return out


def ihaar2d_fused(x: torch.Tensor, add_tensor: torch.Tensor, output_size=None) -> torch.Tensor:
    """ihaar2d(x) + add_tensor (haar_cuda.py:558-560; here the add is a pass of its own)."""
    return ihaar2d(x, output_size) + add_tensor


__all__ = ["MAX_KERNEL_SIZE", "HARD_MAX_KERNEL_SIZE", "check_kernel_size", "haar2d", "ihaar2d", "ihaar2d_fused"]
assert MAX_KERNEL_SIZE >= 1 and _lib is not None
