"""nn.Module front ends of the WTConv layer, API-compatible with the reference.

* ``WTConv2d`` / ``WTConv1d`` keep the reference constructor, attribute and state-dict
  names (wtconv/wtconv2d.py:8-36, wtconv/wtconv1d.py:8-36): ``base_conv.{weight,bias}``,
  ``base_scale.weight``, ``wavelet_convs.{i}.weight``, ``wavelet_scale.{i}.weight``,
  ``wt_filter``, ``iwt_filter``.  The ``nn.Conv*`` sub-modules only hold parameters (and
  give the reference's default initialisation in the reference's draw order); the
  arithmetic runs in the fused HIP kernels.
* ``FastWTConv2d`` keeps the constructor and parameter names of the reference's fused
  twin (fast_wtconv/wtconv_cuda.py:43-117): ``base_weight``, ``base_scale``,
  ``base_bias``, ``wt_weights.{i}``, ``wt_scales.{i}``.
"""
import math

import torch
import torch.nn as nn

from . import functional as Fn

_R = 0.7071067811865476


def _db1_banks_2d(channels):
    """Closed-form db1 analysis/synthesis banks, (4C,1,2,2) each, built the way
    wavelet.py:23-43 builds them (float32 products of the float32 taps)."""
    lo = torch.tensor([_R, _R], dtype=torch.float32)
    hi = torch.tensor([_R, -_R], dtype=torch.float32)
    quad = torch.stack([lo[None, :] * lo[:, None], lo[None, :] * hi[:, None],
                        hi[None, :] * lo[:, None], hi[None, :] * hi[:, None]], dim=0)
    bank = quad[:, None].repeat(channels, 1, 1, 1)
    return bank, bank.clone()


def _db1_banks_1d(channels):
    lo = torch.tensor([_R, _R], dtype=torch.float32)
    hi = torch.tensor([_R, -_R], dtype=torch.float32)
    bank = torch.stack([lo, hi], dim=0)[:, None].repeat(channels, 1, 1)
    return bank, bank.clone()


def _check_wt_type(wt_type):
    if wt_type not in ("db1", "haar"):
        raise NotImplementedError(
            f"wt_type={wt_type!r}: only the Haar wavelet ('db1') is built into the HIP kernels")


class _ScaleModule(nn.Module):
    """Learnable broadcast multiplier (wtconv2d.py:89-97)."""

    def __init__(self, dims, init_scale=1.0, init_bias=0):
        super().__init__()
        self.dims = dims
        self.weight = nn.Parameter(torch.ones(*dims) * init_scale)
        self.bias = None

    def forward(self, x):
        return torch.mul(self.weight, x)


class WTConv2d(nn.Module):
    def __init__(self, in_channels, out_channels, kernel_size=5, stride=1, bias=True, wt_levels=1,
                 wt_type='db1'):
        super().__init__()
        assert in_channels == out_channels
        _check_wt_type(wt_type)
        Fn.check_kernel_size(kernel_size)
        if not 1 <= wt_levels <= 5:
            raise ValueError(f"wt_levels must be 1-5, got {wt_levels}")
        self.in_channels = in_channels
        self.wt_levels = wt_levels
        self.stride = stride
        self.dilation = 1
        self.kernel_size = kernel_size

        dec, rec = _db1_banks_2d(in_channels)
        self.wt_filter = nn.Parameter(dec, requires_grad=False)
        self.iwt_filter = nn.Parameter(rec, requires_grad=False)

        c = in_channels
        self.base_conv = nn.Conv2d(c, c, kernel_size, padding='same', stride=1, dilation=1, groups=c, bias=bias)
        self.base_scale = _ScaleModule([1, c, 1, 1])
        self.wavelet_convs = nn.ModuleList([
            nn.Conv2d(c * 4, c * 4, kernel_size, padding='same', stride=1, dilation=1, groups=c * 4, bias=False)
            for _ in range(wt_levels)])
        self.wavelet_scale = nn.ModuleList([
            _ScaleModule([1, c * 4, 1, 1], init_scale=0.1) for _ in range(wt_levels)])
        self.do_stride = nn.AvgPool2d(kernel_size=1, stride=stride) if stride > 1 else None

    def forward(self, x):
        return Fn.wtconv2d(x, self.base_conv.weight, self.base_conv.bias, self.base_scale.weight,
                           [m.weight for m in self.wavelet_convs],
                           [m.weight for m in self.wavelet_scale], stride=self.stride)

    def extra_repr(self):
        return (f"{self.in_channels}, kernel_size={self.kernel_size}, wt_levels={self.wt_levels}, "
                f"stride={self.stride}, backend=hip-gfx950")


class WTConv1d(nn.Module):
    def __init__(self, in_channels, out_channels, kernel_size=5, stride=1, bias=True, wt_levels=1,
                 wt_type='db1'):
        super().__init__()
        assert in_channels == out_channels
        _check_wt_type(wt_type)
        Fn.check_kernel_size(kernel_size)
        if not 1 <= wt_levels <= 5:
            raise ValueError(f"wt_levels must be 1-5, got {wt_levels}")
        self.in_channels = in_channels
        self.wt_levels = wt_levels
        self.stride = stride
        self.dilation = 1
        self.kernel_size = kernel_size

        dec, rec = _db1_banks_1d(in_channels)
        self.wt_filter = nn.Parameter(dec, requires_grad=False)
        self.iwt_filter = nn.Parameter(rec, requires_grad=False)

        c = in_channels
        self.base_conv = nn.Conv1d(c, c, kernel_size, padding='same', stride=1, dilation=1, groups=c, bias=bias)
        self.base_scale = _ScaleModule([1, c, 1])
        self.wavelet_convs = nn.ModuleList([
            nn.Conv1d(c * 2, c * 2, kernel_size, padding='same', stride=1, dilation=1, groups=c * 2, bias=False)
            for _ in range(wt_levels)])
        self.wavelet_scale = nn.ModuleList([
            _ScaleModule([1, c * 2, 1], init_scale=0.1) for _ in range(wt_levels)])
        self.do_stride = nn.AvgPool1d(kernel_size=stride, stride=stride) if stride > 1 else None

    def forward(self, x):
        return Fn.wtconv1d(x, self.base_conv.weight, self.base_conv.bias, self.base_scale.weight,
                           [m.weight for m in self.wavelet_convs],
                           [m.weight for m in self.wavelet_scale], stride=self.stride)

    def extra_repr(self):
        return (f"{self.in_channels}, kernel_size={self.kernel_size}, wt_levels={self.wt_levels}, "
                f"stride={self.stride}, backend=hip-gfx950")


class FastWTConv2d(nn.Module):
    """Drop-in for the reference's ``fast_wtconv.wtconv_cuda.WTConv2d`` (note its positional
    order: kernel_size, stride, wt_levels, bias)."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size: int = 5, stride: int = 1,
                 wt_levels: int = 1, bias: bool = True):
        super().__init__()
        assert in_channels == out_channels, "WTConv2d requires in_channels == out_channels"
        assert wt_levels in [1, 2, 3, 4, 5], "wt_levels must be 1-5"
        Fn.check_kernel_size(kernel_size)
        self.in_channels = in_channels
        self.wt_levels = wt_levels
        self.kernel_size = kernel_size
        self.stride = stride
        self.do_stride = nn.AvgPool2d(kernel_size=1, stride=stride) if stride > 1 else None

        self.base_weight = nn.Parameter(torch.empty(in_channels, 1, kernel_size, kernel_size))
        self.base_scale = nn.Parameter(torch.ones(1, in_channels, 1, 1))
        if bias:
            self.base_bias = nn.Parameter(torch.empty(in_channels))
        else:
            self.register_parameter('base_bias', None)
        self.wt_weights = nn.ParameterList()
        self.wt_scales = nn.ParameterList()
        for _ in range(wt_levels):
            self.wt_weights.append(nn.Parameter(torch.empty(in_channels * 4, 1, kernel_size, kernel_size)))
            self.wt_scales.append(nn.Parameter(torch.ones(1, in_channels * 4, 1, 1) * 0.1))
        self.reset_parameters()

    def reset_parameters(self):
        """nn.Conv2d's default initialisation, drawn base weight, base bias, then levels."""
        nn.init.kaiming_uniform_(self.base_weight, a=math.sqrt(5))
        if self.base_bias is not None:
            fan_in = self.base_weight.shape[1] * self.base_weight.shape[2] * self.base_weight.shape[3]
            if fan_in != 0:
                bound = 1 / math.sqrt(fan_in)
                nn.init.uniform_(self.base_bias, -bound, bound)
        for w in self.wt_weights:
            nn.init.kaiming_uniform_(w, a=math.sqrt(5))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return Fn.wtconv2d(x, self.base_weight, self.base_bias, self.base_scale,
                           list(self.wt_weights), list(self.wt_scales), stride=self.stride)
