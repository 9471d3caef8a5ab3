"""Autograd entry points of the WTConv layer on MI355X.

One ``torch.autograd.Function`` per layer kind owns the whole layer (base conv, every
wavelet level, the inverse cascade); PyTorch only supplies device memory and the stream.
Semantics follow the reference layer (wtconv/wtconv2d.py:38-87, wtconv/wtconv1d.py:38-87).
"""
import ctypes

import torch

from . import _lib

_DT = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16}


def check_kernel_size(kernel_size):
    """Raise early if no built kernel covers this size (cf. the reference's
    fast_wtconv/cuda_haar/haar_cuda.py:86-105)."""
    if not isinstance(kernel_size, int) or kernel_size < 1 or kernel_size % 2 == 0:
        raise ValueError(f"kernel_size must be odd and positive, got {kernel_size}")
    kmax = _lib.load().wtconv_max_kernel_size()
    if kernel_size > kmax:
        raise ValueError(f"kernel_size {kernel_size} exceeds the largest built kernel ({kmax})")


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(None)


def _prep_params(x, base_w, base_b, base_s, wt_ws, wt_ss):
    """Contiguous parameter tensors in one dtype the kernels accept (fp32 or bf16)."""
    tensors = [base_w, base_s] + list(wt_ws) + list(wt_ss) + ([base_b] if base_b is not None else [])
    dts = {t.dtype for t in tensors}
    pd = dts.pop() if len(dts) == 1 else torch.float32
    if pd not in _DT:
        pd = torch.float32
    conv = lambda t: None if t is None else t.detach().to(device=x.device, dtype=pd).contiguous()
    return pd, conv(base_w), conv(base_b), conv(base_s), [conv(w) for w in wt_ws], [conv(s) for s in wt_ss]


def _table(cls, base_w, base_b, base_s, wt_ws, wt_ss):
    tab = cls()
    tab.base_weight, tab.base_bias, tab.base_scale = _ptr(base_w), _ptr(base_b), _ptr(base_s)
    for i, (w, s) in enumerate(zip(wt_ws, wt_ss)):
        tab.wt_weight[i] = w.data_ptr()
        tab.wt_scale[i] = s.data_ptr()
    return tab


def _check_input(x, ndim, what):
    if x.dim() != ndim:
        raise ValueError(f"{what} expects a {ndim}-D input, got shape {tuple(x.shape)}")
    if not x.is_cuda:
        raise RuntimeError(f"{what} runs on the GPU only (got a {x.device} tensor); there is no CPU path")
    if x.dtype not in _DT:
        raise TypeError(f"{what} supports float32 and bfloat16 activations, got {x.dtype}")


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


class _WTConvFn(torch.autograd.Function):
    """dims = 2: x (B,C,H,W); dims = 1: x (B,C,N).  Argument order:
    x, base_w, base_b, base_s, dims, K, L, wt_w[0..L-1], wt_s[0..L-1]."""

    @staticmethod
    def forward(ctx, x, base_w, base_b, base_s, dims, K, L, *wt):
        wt_ws, wt_ss = wt[:L], wt[L:]
        lib = _lib.load()
        x = x.contiguous()
        pd, bw, bb, bs, ws, ss = _prep_params(x, base_w, base_b, base_s, wt_ws, wt_ss)
        out = torch.empty_like(x)
        tab = _table(_lib.Params, bw, bb, bs, ws, ss)
        stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
        with torch.cuda.device(x.device):
            if dims == 2:
                B, C, H, W = x.shape
                wsz = lib.wtconv2d_workspace_bytes(B, C, H, W, K, L, _lib.PASS_FORWARD)
                wsp = _workspace(wsz, x.device)
                rc = lib.wtconv2d_forward(_ptr(x), _ptr(out), ctypes.byref(tab), B, C, H, W, K, L,
                                          _DT[x.dtype], _DT[pd], _ptr(wsp), wsp.numel(), stream)
            else:
                B, C, N = x.shape
                wsz = lib.wtconv1d_workspace_bytes(B, C, N, K, L, _lib.PASS_FORWARD)
                wsp = _workspace(wsz, x.device)
                rc = lib.wtconv1d_forward(_ptr(x), _ptr(out), ctypes.byref(tab), B, C, N, K, L,
                                          _DT[x.dtype], _DT[pd], _ptr(wsp), wsp.numel(), stream)
        _lib.check(rc, "wtconv forward")
        ctx.dims, ctx.K, ctx.L, ctx.has_bias = dims, K, L, base_b is not None
        ctx.save_for_backward(x, base_w, base_b, base_s, *wt)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, base_w, base_b, base_s, *wt = ctx.saved_tensors
        dims, K, L = ctx.dims, ctx.K, ctx.L
        wt_ws, wt_ss = wt[:L], wt[L:]
        lib = _lib.load()
        g = grad_out.to(x.dtype).contiguous()
        pd, bw, bb, bs, ws, ss = _prep_params(x, base_w, base_b, base_s, wt_ws, wt_ss)
        tab = _table(_lib.Params, bw, bb, bs, ws, ss)
        stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
        shape = tuple(x.shape)
        grad_x = None
        grads = [None] * (3 + 2 * L)
        need_params = any(ctx.needs_input_grad[i] for i in (1, 2, 3)) or any(ctx.needs_input_grad[7:])
        with torch.cuda.device(x.device):
            if ctx.needs_input_grad[0]:
                grad_x = torch.empty_like(x)
                if dims == 2:
                    wsz = lib.wtconv2d_workspace_bytes(*shape, K, L, _lib.PASS_BACKWARD_INPUT)
                    wsp = _workspace(wsz, x.device)
                    rc = lib.wtconv2d_backward_input(_ptr(g), _ptr(grad_x), ctypes.byref(tab), *shape, K, L,
                                                     _DT[x.dtype], _DT[pd], _ptr(wsp), wsp.numel(), stream)
                else:
                    wsz = lib.wtconv1d_workspace_bytes(*shape, K, L, _lib.PASS_BACKWARD_INPUT)
                    wsp = _workspace(wsz, x.device)
                    rc = lib.wtconv1d_backward_input(_ptr(g), _ptr(grad_x), ctypes.byref(tab), *shape, K, L,
                                                     _DT[x.dtype], _DT[pd], _ptr(wsp), wsp.numel(), stream)
                _lib.check(rc, "wtconv backward_input")
            if need_params:
                f32 = lambda t: torch.empty(t.shape, dtype=torch.float32, device=x.device)
                gbw, gbs = f32(bw), f32(bs)
                gbb = f32(bb) if bb is not None else None
                gws, gss = [f32(w) for w in ws], [f32(s) for s in ss]
                gtab = _table(_lib.ParamGrads, gbw, gbb, gbs, gws, gss)
                if dims == 2:
                    wsz = lib.wtconv2d_workspace_bytes(*shape, K, L, _lib.PASS_BACKWARD_PARAMS)
                    wsp = _workspace(wsz, x.device)
                    rc = lib.wtconv2d_backward_params(_ptr(x), _ptr(g), ctypes.byref(tab), ctypes.byref(gtab),
                                                      *shape, K, L, _DT[x.dtype], _DT[pd], _ptr(wsp),
                                                      wsp.numel(), stream)
                else:
                    wsz = lib.wtconv1d_workspace_bytes(*shape, K, L, _lib.PASS_BACKWARD_PARAMS)
                    wsp = _workspace(wsz, x.device)
                    rc = lib.wtconv1d_backward_params(_ptr(x), _ptr(g), ctypes.byref(tab), ctypes.byref(gtab),
                                                      *shape, K, L, _DT[x.dtype], _DT[pd], _ptr(wsp),
                                                      wsp.numel(), stream)
                _lib.check(rc, "wtconv backward_params")
                like = lambda gt, p: None if gt is None else gt.to(p.dtype).reshape(p.shape)
                grads[0] = like(gbw, base_w)
                grads[1] = like(gbb, base_b) if base_b is not None else None
                grads[2] = like(gbs, base_s)
                for i in range(L):
                    grads[3 + i] = like(gws[i], wt_ws[i])
                    grads[3 + L + i] = like(gss[i], wt_ss[i])
        return (grad_x, grads[0], grads[1], grads[2], None, None, None, *grads[3:])


def _check_params(C, K, L, S, dims, base_w, base_b, base_s, wt_ws, wt_ss):
    kk = K ** dims
    if base_w.numel() != C * kk:
        raise ValueError(f"base weight has {base_w.numel()} elements, expected {C * kk}")
    if base_b is not None and base_b.numel() != C:
        raise ValueError(f"base bias has {base_b.numel()} elements, expected {C}")
    if base_s.numel() != C:
        raise ValueError(f"base scale has {base_s.numel()} elements, expected {C}")
    if len(wt_ws) != L or len(wt_ss) != L:
        raise ValueError(f"expected {L} levels of wavelet weights and scales")
    for w, s in zip(wt_ws, wt_ss):
        if w.numel() != S * C * kk or s.numel() != S * C:
            raise ValueError("wavelet weight/scale shape does not match channels and kernel size")


def wtconv2d(x, base_weight, base_bias, base_scale, wt_weights, wt_scales, stride=1):
    """WTConv2d forward (differentiable).  x (B,C,H,W) fp32/bf16 on the GPU;
    base_weight (C,1,K,K); base_bias (C,) or None; base_scale (1,C,1,1);
    wt_weights[l] (4C,1,K,K); wt_scales[l] (1,4C,1,1).  Stride sub-samples the stride-1
    result, as the reference does (wtconv2d.py:33-36,84-85)."""
    _check_input(x, 4, "wtconv2d")
    C, K, L = x.shape[1], base_weight.shape[-1], len(wt_weights)
    if not 1 <= L <= _lib.MAX_LEVELS:
        raise ValueError(f"wt_levels must be 1-{_lib.MAX_LEVELS}, got {L}")
    check_kernel_size(int(K))
    _check_params(C, K, L, 4, 2, base_weight, base_bias, base_scale, wt_weights, wt_scales)
    out = _WTConvFn.apply(x, base_weight, base_bias, base_scale, 2, int(K), L, *wt_weights, *wt_scales)
    if stride > 1:
        out = out[:, :, ::stride, ::stride]
    return out


def wtconv1d(x, base_weight, base_bias, base_scale, wt_weights, wt_scales, stride=1):
    """WTConv1d forward (differentiable).  x (B,C,N); base_weight (C,1,K);
    wt_weights[l] (2C,1,K); scales (1,C,1) / (1,2C,1).  Stride is a true average pool
    (wtconv1d.py:33-36)."""
    _check_input(x, 3, "wtconv1d")
    C, K, L = x.shape[1], base_weight.shape[-1], len(wt_weights)
    if not 1 <= L <= _lib.MAX_LEVELS:
        raise ValueError(f"wt_levels must be 1-{_lib.MAX_LEVELS}, got {L}")
    check_kernel_size(int(K))
    _check_params(C, K, L, 2, 1, base_weight, base_bias, base_scale, wt_weights, wt_scales)
    out = _WTConvFn.apply(x, base_weight, base_bias, base_scale, 1, int(K), L, *wt_weights, *wt_scales)
    if stride > 1:
        out = torch.nn.functional.avg_pool1d(out, kernel_size=stride, stride=stride)
    return out
