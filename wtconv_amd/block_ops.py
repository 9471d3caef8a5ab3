"""The two passes a WTConvNeXt block makes around its WTConv layer, each as one HIP kernel
(`wtconv_channel_norm`, `wtconv_block_residual` of the C ABI), GPU only; with their backward kernels
(`wtconv_channel_norm_backward`, `wtconv_block_residual_backward`) behind autograd functions for training.

Reference semantics: `x.permute(0, 2, 3, 1)` + `nn.LayerNorm` after `conv_dw`
(wtconvnext/wtconvnext.py:132-133), `LayerNorm2d` of the stem and downsample layers (:171, :296), and
`permute(0, 3, 1, 2)` + `mul(gamma)` + shortcut add at the end of the block (:135-140)."""
import ctypes

import torch

from . import _lib

_DT = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16}


def records(x, *params):
    """Whether autograd would record an operation on these tensors."""
    return torch.is_grad_enabled() and (x.requires_grad or any(p is not None and p.requires_grad for p in params))


def usable(x, *params, training=False):
    """Whether the kernels take this call: a contiguous fp32 / bf16 GPU tensor with an even channel count, parameters
    of one fp32 / bf16 dtype on the same device, no autocast, not under torch.compile.  With training=False also:
    nothing recorded for autograd (the plain functions below take raw pointers; the *_fn variants are the ones that
    autograd can differentiate)."""
    if not training and records(x, *params):
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
    """Whether the residual kernels take the MLP output `y` (B, H, W, C) for this shortcut: same dtype and device."""
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


def _workspace(x, B, C, HW):
    lib = _lib.load()
    n = lib.wtconv_block_workspace_bytes(B, C, HW, _DT[x.dtype])
    if n == 0:
        raise RuntimeError(f"block backward: no tile plan for C={C}, HW={HW}")
    return torch.empty(n, dtype=torch.uint8, device=x.device), n


def channel_norm_backward(x, dy, weight, eps, nhwc):
    """Gradients of channel_norm: dx (B, C, H, W) in x.dtype, dweight and dbias (C) in float32."""
    lib = _lib.load()
    B, C, H, W = x.shape
    with torch.cuda.device(x.device):
        dx = torch.empty_like(x)
        dwb = torch.empty(2, C, dtype=torch.float32, device=x.device)
        ws, n = _workspace(x, B, C, H * W)
        rc = lib.wtconv_channel_norm_backward(x.data_ptr(), dy.data_ptr(), weight.data_ptr(), dx.data_ptr(),
                                              dwb[0].data_ptr(), dwb[1].data_ptr(), B, C, H * W, float(eps),
                                              _DT[x.dtype], _DT[weight.dtype], int(bool(nhwc)), ws.data_ptr(), n, _stream())
    if rc:
        _lib.check(rc, "wtconv_channel_norm_backward")
    return dx, dwb[0], dwb[1]


def block_residual_backward(dout, y, gamma):
    """Gradients of block_residual with a layer scale: dy (B, H, W, C) in dout.dtype, dgamma (C) in float32."""
    lib = _lib.load()
    B, C, H, W = dout.shape
    with torch.cuda.device(dout.device):
        dy = torch.empty_like(y)
        dg = torch.empty(C, dtype=torch.float32, device=dout.device)
        ws, n = _workspace(dout, B, C, H * W)
        rc = lib.wtconv_block_residual_backward(dout.data_ptr(), y.data_ptr(), gamma.data_ptr(), dy.data_ptr(),
                                                dg.data_ptr(), B, C, H * W, _DT[dout.dtype], _DT[gamma.dtype],
                                                ws.data_ptr(), n, _stream())
    if rc:
        _lib.check(rc, "wtconv_block_residual_backward")
    return dy, dg


class _ChannelNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, eps, nhwc):
        ctx.eps, ctx.nhwc = eps, nhwc
        ctx.save_for_backward(x, weight)
        return channel_norm(x, weight, bias, eps, nhwc)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        if dy.dtype != x.dtype:
            dy = dy.to(x.dtype)
        dx, dw, db = channel_norm_backward(x, dy.contiguous(), weight, ctx.eps, ctx.nhwc)
        return dx, dw.to(weight.dtype), db.to(weight.dtype), None, None


class _BlockResidualFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, y, shortcut, gamma):
        ctx.save_for_backward(y, gamma)
        return block_residual(y, shortcut, gamma)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dout):
        y, gamma = ctx.saved_tensors
        if dout.dtype != y.dtype:
            dout = dout.to(y.dtype)
        dout = dout.contiguous()
        dy, dg = block_residual_backward(dout, y, gamma)
        return dy, dout, dg.to(gamma.dtype)


def channel_norm_fn(x, weight, bias, eps, nhwc):
    """channel_norm that autograd can differentiate (gradients of x, weight and bias from the backward kernel)."""
    return _ChannelNormFn.apply(x, weight, bias, eps, nhwc)


def block_residual_fn(y, shortcut, gamma):
    """block_residual (with a layer scale) that autograd can differentiate (gradients of y, shortcut and gamma)."""
    return _BlockResidualFn.apply(y, shortcut, gamma)
