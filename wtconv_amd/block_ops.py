"""The two passes a WTConvNeXt block makes around its WTConv layer, each as one HIP kernel
(`wtconv_channel_norm`, `wtconv_block_residual` of the C ABI): inference only, GPU only.

Reference semantics: `x.permute(0, 2, 3, 1)` + `nn.LayerNorm` after `conv_dw`
(wtconvnext/wtconvnext.py:132-133), `LayerNorm2d` of the stem and downsample layers (:171, :296), and
`permute(0, 3, 1, 2)` + `mul(gamma)` + shortcut add at the end of the block (:135-140)."""
import ctypes

import torch

from . import _lib

_DT = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16}


def usable(x, *params):
    """Whether the kernels take this call: inference (nothing recorded for autograd), a contiguous fp32 / bf16
    GPU tensor with an even channel count, parameters of one fp32 / bf16 dtype on the same device."""
    if torch.is_grad_enabled() and (x.requires_grad or any(p is not None and p.requires_grad for p in params)):
        return False
    if torch.compiler.is_compiling():
        return False
    if torch.is_autocast_enabled():      # autocast keeps LayerNorm outputs and the residual stream in fp32; the kernels return x.dtype
        return False
    if not x.is_cuda or x.dtype not in _DT or x.dim() != 4 or x.shape[1] % 2 or not x.is_contiguous():
        return False
    pd = None
    for p in params:
        if p is None:
            continue
        if p.device != x.device or p.dtype not in _DT or not p.is_contiguous() or (pd is not None and p.dtype != pd):
            return False
        pd = p.dtype
    return True


def usable_nhwc(y, shortcut):
    """Whether block_residual takes the MLP output `y` (B, H, W, C) for this shortcut: nothing recorded for autograd
    on it, same dtype and device as the shortcut."""
    if torch.is_grad_enabled() and y.requires_grad:
        return False
    return y.dtype == shortcut.dtype and y.device == shortcut.device and y.dim() == 4


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def channel_norm(x, weight, bias, eps, nhwc):
    """LayerNorm over the channels of x (B, C, H, W); returns (B, H, W, C) if `nhwc` else (B, C, H, W)."""
    lib = _lib.load()
    B, C, H, W = x.shape
    with torch.cuda.device(x.device):
        out = torch.empty((B, H, W, C) if nhwc else (B, C, H, W), dtype=x.dtype, device=x.device)
        rc = lib.wtconv_channel_norm(x.data_ptr(), out.data_ptr(), weight.data_ptr(), bias.data_ptr(), B, C, H * W,
                                     float(eps), _DT[x.dtype], _DT[weight.dtype], int(bool(nhwc)), _stream())
    if rc:
        _lib.check(rc, "wtconv_channel_norm")
    return out


def block_residual(y, shortcut, gamma):
    """shortcut (B, C, H, W) + gamma[c] * y, with y (B, H, W, C); gamma may be None.  Returns (B, C, H, W)."""
    lib = _lib.load()
    B, C, H, W = shortcut.shape
    if tuple(y.shape) != (B, H, W, C) or y.dtype != shortcut.dtype or not y.is_contiguous():
        raise ValueError(f"block_residual: y {tuple(y.shape)} {y.dtype} does not match shortcut {tuple(shortcut.shape)}")
    with torch.cuda.device(shortcut.device):
        out = torch.empty_like(shortcut)
        rc = lib.wtconv_block_residual(y.data_ptr(), shortcut.data_ptr(), gamma.data_ptr() if gamma is not None else None,
                                       out.data_ptr(), B, C, H * W, _DT[shortcut.dtype],
                                       _DT[gamma.dtype] if gamma is not None else _lib.F32, _stream())
    if rc:
        _lib.check(rc, "wtconv_block_residual")
    return out
