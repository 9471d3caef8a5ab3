"""Autograd entry points of the WTConv layer on MI355X.

One ``torch.autograd.Function`` per layer kind owns the whole layer (base conv, every
wavelet level, the inverse cascade); PyTorch only supplies device memory and the stream.
Semantics follow the reference layer (wtconv/wtconv2d.py:38-87, wtconv/wtconv1d.py:38-87).
"""
import ctypes
from typing import List, Optional

import torch

from . import _ext, _lib

_DT = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}


def check_kernel_size(kernel_size):
    """Raise early if no built kernel covers this size (cf. the reference's
    fast_wtconv/cuda_haar/haar_cuda.py:86-105)."""
    if not isinstance(kernel_size, int) or kernel_size < 1 or kernel_size % 2 == 0:
        raise ValueError(f"kernel_size must be odd and positive, got {kernel_size}")
    if torch.compiler.is_compiling():     # no ctypes under tracing; modules check at construction
        return
    kmax = _lib.load().wtconv_max_kernel_size()
    if kernel_size > kmax:
        raise ValueError(f"kernel_size {kernel_size} exceeds the largest built kernel ({kmax})")


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(None)


def _prep_params(x, base_w, base_b, base_s, wt_ws, wt_ss):
    """Contiguous parameter tensors in one dtype the kernels accept (fp32, bf16 or fp16)."""
    tensors = [base_w, base_s] + list(wt_ws) + list(wt_ss) + ([base_b] if base_b is not None else [])
    pd = base_w.dtype
    if pd not in _DT or any(t.dtype != pd for t in tensors):
        pd = torch.float32
    dev = x.device

    def conv(t):
        if t is None:
            return None
        t = t.detach()
        if t.dtype != pd or t.device != dev:
            t = t.to(device=dev, dtype=pd)
        return t if t.is_contiguous() else t.contiguous()

    return pd, conv(base_w), conv(base_b), conv(base_s), [conv(w) for w in wt_ws], [conv(s) for s in wt_ss]


_TABLES = {}


def _params_table(x, base_w, base_b, base_s, wt_ws, wt_ss):
    """(param dtype, Params table, tensors kept alive).  Fast path: parameters that already sit
    on x's device, contiguous, in one kernel dtype are passed as they are, and the table of
    their addresses is cached under those addresses (a table is nothing but its key)."""
    pd = base_w.dtype
    dev = x.device
    tensors = (base_w, base_s, *wt_ws, *wt_ss) if base_b is None else (base_w, base_s, base_b, *wt_ws, *wt_ss)
    if pd in _DT:
        for t in tensors:
            if t.dtype != pd or t.device != dev or not t.is_contiguous():
                break
        else:
            key = (pd, base_b is not None, *[t.data_ptr() for t in tensors])
            tab = _TABLES.get(key)
            if tab is None:
                if len(_TABLES) > 4096:
                    _TABLES.clear()
                tab = _TABLES[key] = _table(_lib.Params, base_w, base_b, base_s, wt_ws, wt_ss)
            return pd, tab, tensors
    pd, bw, bb, bs, ws, ss = _prep_params(x, base_w, base_b, base_s, wt_ws, wt_ss)
    return pd, _table(_lib.Params, bw, bb, bs, ws, ss), (bw, bb, bs, ws, ss)


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
        raise TypeError(f"{what} supports float32, bfloat16 and float16 activations, got {x.dtype}")


_WS_BYTES = {}


def _workspace_bytes(lib, dims, shape, K, L, which):
    """Workspace size of one pass (the library's answer depends on the sizes only: cached)."""
    key = (dims, shape, K, L, which)
    n = _WS_BYTES.get(key)
    if n is None:
        fn = lib.wtconv2d_workspace_bytes if dims == 2 else lib.wtconv1d_workspace_bytes
        n = max(int(fn(*shape, K, L, which)), 256)
        _WS_BYTES[key] = n
    return n


class _on_device:
    """Makes x's device current for the launches, only if it is not already."""

    def __init__(self, device):
        self.idx = device.index if device.index is not None else torch.cuda.current_device()
        self.prev = None

    def __enter__(self):
        cur = torch.cuda.current_device()
        if cur != self.idx:
            self.prev = cur
            torch.cuda.set_device(self.idx)

    def __exit__(self, *exc):
        if self.prev is not None:
            torch.cuda.set_device(self.prev)
        return False


def _forward_impl(x, base_w, base_b, base_s, wt_ws, wt_ss, dims, K, L, tabinfo=None):
    """One forward launch sequence; returns (out, contiguous x).  `tabinfo`, a list, receives the
    parameter table of the call for the backward pass to reuse."""
    lib = _lib.load()
    if not x.is_contiguous():
        x = x.contiguous()
    # float16 activations (the reference trainer's default AMP dtype, train.py:180,438; its fused twin dispatches
    # fp16 too, haar_common.cuh:55-77) go through the vector kernels: fp16 in HBM, fp32 arithmetic, one rounding.
    pd, tab, _keep = _params_table(x, base_w, base_b, base_s, wt_ws, wt_ss)
    if tabinfo is not None:
        tabinfo.append((pd, tab, _keep))
    shape = tuple(x.shape)
    with _on_device(x.device):
        out = torch.empty_like(x)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        wsz = _workspace_bytes(lib, dims, shape, K, L, _lib.PASS_FORWARD)
        wsp = torch.empty(wsz, dtype=torch.uint8, device=x.device)
        fn = lib.wtconv2d_forward if dims == 2 else lib.wtconv1d_forward
        rc = fn(x.data_ptr(), out.data_ptr(), ctypes.byref(tab), *shape, K, L, _DT[x.dtype], _DT[pd],
                wsp.data_ptr(), wsz, stream)
    if rc:
        _lib.check(rc, "wtconv forward")
    return out, x


def _backward_impl(grad_out, x, base_w, base_b, base_s, wt_ws, wt_ss, dims, K, L, need_x, need_params, tabinfo=None):
    """grad_x (or None) and the parameter gradients in the order base_w, base_b (or None),
    base_s, wt_ws[0..L-1], wt_ss[0..L-1] (all None when not needed), in the parameters' dtypes."""
    lib = _lib.load()
    g = grad_out
    if g.dtype != x.dtype:
        g = g.to(x.dtype)
    if not g.is_contiguous():
        g = g.contiguous()
    # (the forward pass's table of the same, unmodified tensors, when it left one)
    pd, tab, _keep = tabinfo if tabinfo is not None else _params_table(x, base_w, base_b, base_s, wt_ws, wt_ss)
    has_bias = base_b is not None
    shape = tuple(x.shape)
    grad_x = None
    grads = [None] * (3 + 2 * L)
    with _on_device(x.device):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        which = (_lib.PASS_BACKWARD if need_x and need_params else
                 _lib.PASS_BACKWARD_INPUT if need_x else _lib.PASS_BACKWARD_PARAMS)
        wsz = _workspace_bytes(lib, dims, shape, K, L, which)
        wsp = torch.empty(wsz, dtype=torch.uint8, device=x.device)
        dt, pdt = _DT[x.dtype], _DT[pd]
        if need_x:
            grad_x = torch.empty_like(x)
        if need_params:
            plist = [base_w, base_s] + ([base_b] if has_bias else []) + list(wt_ws) + list(wt_ss)
            nb = 3 if has_bias else 2
            same_f32 = all(t.dtype == torch.float32 for t in plist)
            if same_f32:
                # fp32 parameters: every gradient is written in place, in its parameter's shape
                views = [torch.empty_like(t, memory_format=torch.contiguous_format) for t in plist]
            else:
                # other parameter dtypes: one flat fp32 buffer, so that one cast serves every gradient
                sizes = [t.numel() for t in plist]
                flat = torch.empty(sum(sizes), dtype=torch.float32, device=x.device)
                views = flat.split(sizes)
            gtab = _table(_lib.ParamGrads, views[0], views[2] if has_bias else None, views[1],
                          views[nb:nb + L], views[nb + L:])
        if need_x and need_params:        # the whole backward pass in one library call
            fn = lib.wtconv2d_backward if dims == 2 else lib.wtconv1d_backward
            rc = fn(x.data_ptr(), g.data_ptr(), grad_x.data_ptr(), ctypes.byref(tab), ctypes.byref(gtab), *shape, K, L,
                    dt, pdt, wsp.data_ptr(), wsz, stream)
            if rc:
                _lib.check(rc, "wtconv backward")
        elif need_x:
            fn = lib.wtconv2d_backward_input if dims == 2 else lib.wtconv1d_backward_input
            rc = fn(g.data_ptr(), grad_x.data_ptr(), ctypes.byref(tab), *shape, K, L, dt, pdt,
                    wsp.data_ptr(), wsz, stream)
            if rc:
                _lib.check(rc, "wtconv backward_input")
        elif need_params:
            fn = lib.wtconv2d_backward_params if dims == 2 else lib.wtconv1d_backward_params
            rc = fn(x.data_ptr(), g.data_ptr(), ctypes.byref(tab), ctypes.byref(gtab), *shape, K, L, dt, pdt,
                    wsp.data_ptr(), wsz, stream)
            if rc:
                _lib.check(rc, "wtconv backward_params")
        if need_params:
            if same_f32:
                outg = views
            else:
                out_dt = base_w.dtype
                if all(t.dtype == out_dt for t in plist):
                    outg = [v.view(t.shape) for v, t in zip(flat.to(out_dt).split(sizes), plist)]
                else:
                    outg = [v.to(t.dtype).view(t.shape) for v, t in zip(views, plist)]
            grads[0], grads[2] = outg[0], outg[1]
            if has_bias:
                grads[1] = outg[2]
            for i in range(L):
                grads[3 + i] = outg[nb + i]
                grads[3 + L + i] = outg[nb + L + i]
    return grad_x, grads


class _WTConvFn(torch.autograd.Function):
    """dims = 2: x (B,C,H,W); dims = 1: x (B,C,N).  Argument order:
    x, base_w, base_b, base_s, dims, K, L, wt_w[0..L-1], wt_s[0..L-1]."""

    # Under torch.autocast the inputs are taken as they come (fp32, bf16 or fp16 activations, parameters in any of
    # the three, any mix): the kernels accumulate in fp32 either way, so there is nothing
    # to down-cast, and neither pass runs a torch operator that autocast would touch (hence no
    # custom_fwd / custom_bwd wrappers: entering an autocast context costs more host time than the
    # rest of the backward prelude).
    @staticmethod
    def forward(ctx, x, base_w, base_b, base_s, dims, K, L, *wt):
        info = []
        out, x = _forward_impl(x, base_w, base_b, base_s, wt[:L], wt[L:], dims, K, L, info)
        ctx.dims, ctx.K, ctx.L = dims, K, L
        ctx.tabinfo = info[0] if info else None
        ctx.save_for_backward(x, base_w, base_b, base_s, *wt)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, base_w, base_b, base_s, *wt = ctx.saved_tensors
        dims, K, L = ctx.dims, ctx.K, ctx.L
        need_params = any(ctx.needs_input_grad[i] for i in (1, 2, 3)) or any(ctx.needs_input_grad[7:])
        # Under create_graph=True a second-order term through this layer is refused, not dropped: the gradients come
        # from raw pointers and carry no graph, so every result that something differentiable went into (the upstream
        # gradient or any saved tensor -- once_differentiable looks at the upstream gradient only) gets a node that
        # raises when it is differentiated.
        twice = torch.is_grad_enabled() and any(
            t is not None and t.requires_grad for t in (grad_out, x, base_w, base_b, base_s, *wt))
        with torch.no_grad():
            grad_x, grads = _backward_impl(grad_out, x, base_w, base_b, base_s, wt[:L], wt[L:], dims, K, L,
                                           ctx.needs_input_grad[0], need_params, ctx.tabinfo)
        res = (grad_x, grads[0], grads[1], grads[2], None, None, None, *grads[3:])
        if twice:
            res = _refuse_second_order(res)
        return res


def _refuse_second_order(outputs):
    err = torch._C._functions.DelayedError(
        b"the backward pass of the WTConv layer is not differentiable (double backward / create_graph=True through "
        b"this layer is not supported)", len(outputs))

    def fake(v):      # an input that requires grad makes DelayedError attach its raising node to the matching output
        return v.detach().requires_grad_(True) if v is not None else None
    return err(*[fake(v) for v in outputs])


# ---------------------------------------------------------------------------------------------
# The same two steps as opaque operators for torch.compile (train.py:629-632 of the reference
# offers --torchcompile): Dynamo cannot trace through ctypes, so while compiling the layer is
# routed through torch.library custom ops with shape-only fake implementations.
@torch.library.custom_op("wtconv_amd::layer_forward", mutates_args=())
def _op_forward(x: torch.Tensor, base_w: torch.Tensor, base_b: Optional[torch.Tensor], base_s: torch.Tensor,
                wt_ws: List[torch.Tensor], wt_ss: List[torch.Tensor], dims: int) -> torch.Tensor:
    out, _ = _forward_impl(x, base_w, base_b, base_s, wt_ws, wt_ss, dims, int(base_w.shape[-1]), len(wt_ws))
    return out


@_op_forward.register_fake
def _(x, base_w, base_b, base_s, wt_ws, wt_ss, dims):
    return torch.empty_like(x, memory_format=torch.contiguous_format)


@torch.library.custom_op("wtconv_amd::layer_backward", mutates_args=())
def _op_backward(grad_out: torch.Tensor, x: torch.Tensor, base_w: torch.Tensor, base_b: Optional[torch.Tensor],
                 base_s: torch.Tensor, wt_ws: List[torch.Tensor], wt_ss: List[torch.Tensor],
                 dims: int) -> List[torch.Tensor]:
    """[grad_x, grad_base_w, grad_base_s, grad_base_b (empty without bias), grads of wt_ws, grads of wt_ss]."""
    L = len(wt_ws)
    gx, gr = _backward_impl(grad_out, x.contiguous(), base_w, base_b, base_s, wt_ws, wt_ss, dims,
                            int(base_w.shape[-1]), L, True, True)
    # the eager path hands out views of one flat buffer; operator outputs may not alias
    gb = gr[1].clone() if gr[1] is not None else x.new_empty(0)
    return [gx, gr[0].clone(), gr[2].clone(), gb] + [t.clone() for t in gr[3:]]


@_op_backward.register_fake
def _(grad_out, x, base_w, base_b, base_s, wt_ws, wt_ss, dims):
    gb = torch.empty_like(base_b) if base_b is not None else x.new_empty(0)
    return ([torch.empty_like(x, memory_format=torch.contiguous_format), torch.empty_like(base_w),
             torch.empty_like(base_s), gb] + [torch.empty_like(t) for t in wt_ws] + [torch.empty_like(t) for t in wt_ss])


def _op_setup_context(ctx, inputs, output):
    x, base_w, base_b, base_s, wt_ws, wt_ss, dims = inputs
    ctx.dims, ctx.L, ctx.has_bias = dims, len(wt_ws), base_b is not None
    ctx.save_for_backward(x, base_w, base_s, *wt_ws, *wt_ss, *([base_b] if base_b is not None else []))


def _op_autograd_backward(ctx, grad_out):
    saved = ctx.saved_tensors
    L = ctx.L
    x, base_w, base_s = saved[:3]
    wt_ws, wt_ss = list(saved[3:3 + L]), list(saved[3 + L:3 + 2 * L])
    base_b = saved[3 + 2 * L] if ctx.has_bias else None
    res = _op_backward(grad_out, x, base_w, base_b, base_s, wt_ws, wt_ss, ctx.dims)
    return (res[0], res[1], res[3] if ctx.has_bias else None, res[2], list(res[4:4 + L]), list(res[4 + L:]), None)


_op_forward.register_autograd(_op_autograd_backward, setup_context=_op_setup_context)


def _apply(x, base_weight, base_bias, base_scale, wt_weights, wt_scales, dims, K, L):
    if torch.compiler.is_compiling():
        return _op_forward(x, base_weight, base_bias, base_scale, list(wt_weights), list(wt_scales), dims)
    ext = _ext.get()
    if ext is not None:
        # the same launches from a C++ autograd node (no interpreter between PyTorch's engine and the library);
        # None: parameters that need a conversion first (mixed dtypes, another device, not contiguous)
        out = ext.layer(x, base_weight, base_bias, base_scale, list(wt_weights), list(wt_scales), dims, K, L)
        if out is not None:
            return out
    return _WTConvFn.apply(x, base_weight, base_bias, base_scale, dims, K, L, *wt_weights, *wt_scales)


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
    out = _apply(x, base_weight, base_bias, base_scale, wt_weights, wt_scales, 2, int(K), L)
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
    out = _apply(x, base_weight, base_bias, base_scale, wt_weights, wt_scales, 1, int(K), L)
    if stride > 1:
        out = torch.nn.functional.avg_pool1d(out, kernel_size=stride, stride=stride)
    return out
