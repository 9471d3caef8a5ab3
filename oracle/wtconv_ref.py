"""CPU oracle for the WTConv layer (test infrastructure, never the product path).

This file restates, with ``torch.nn.functional`` library routines only, what the
reference PyTorch layer computes:

* 2-D layer ............ reference ``wtconv/wtconv2d.py:38-87``
* 1-D layer ............ reference ``wtconv/wtconv1d.py:38-87``
* db1 filter banks ..... reference ``wtconv/util/wavelet.py:6-43`` (the four
  PyWavelets 1.6.0 ``db1`` tap vectors are written out in closed form because
  PyWavelets is not importable here; they are ``dec_lo=[r,r]``, ``dec_hi=[-r,r]``,
  ``rec_lo=[r,r]``, ``rec_hi=[r,-r]`` with ``r = 1/sqrt(2)``)
* analysis/synthesis ... reference ``wtconv/util/wavelet.py:46-75``

Only tests, the smoke check and the benchmark's CPU-baseline leg may import it.
Gradients come from autograd of this forward.

What pins it (see tests/test_oracle_*.py): the closed-form sub-band formulas,
perfect reconstruction, Parseval, the brute-force loops in ``oracle/brute.py``,
special cases that collapse to a plain depthwise convolution or to block means,
and ``torch.autograd.gradcheck`` in float64.  The reference repository ships no
tests, golden vectors or fixtures for this path, so nothing reference-held pins
it beyond the sub-band convention quoted in
``fast_wtconv/cuda_haar/haar_common.cuh:4-15``; the timm-dependent model shell is
pinned only by the parameter counts in ``logs/val_*.out:4`` ("parity unpinned"
for everything else in the shell).
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence

import torch
import torch.nn as nn
import torch.nn.functional as F

_R = 0.7071067811865476  # 1/sqrt(2): every db1 tap has this magnitude


# --------------------------------------------------------------------------- filters
def db1_taps(dtype=torch.float32):
    """(dec_lo, dec_hi, rec_lo, rec_hi) after the reversal of the decomposition taps
    done at wavelet.py:8-9 / :25-26."""
    dec_lo = torch.tensor([_R, _R], dtype=dtype)          # reversed [r, r]
    dec_hi = torch.tensor([_R, -_R], dtype=dtype)         # reversed [-r, r]
    rec_lo = torch.tensor([_R, _R], dtype=dtype)
    rec_hi = torch.tensor([_R, -_R], dtype=dtype)
    return dec_lo, dec_hi, rec_lo, rec_hi


def haar_filters_2d(channels: int, dtype=torch.float32):
    """Analysis and synthesis banks of shape (4*C, 1, 2, 2); sub-band order
    LL, LH, HL, HH (wavelet.py:27-43)."""
    dlo, dhi, rlo, rhi = db1_taps(dtype)

    def bank(lo, hi):
        quad = torch.stack([
            lo[None, :] * lo[:, None],
            lo[None, :] * hi[:, None],
            hi[None, :] * lo[:, None],
            hi[None, :] * hi[:, None],
        ], dim=0)
        return quad[:, None].repeat(channels, 1, 1, 1)

    return bank(dlo, dhi), bank(rlo, rhi)


def haar_filters_1d(channels: int, dtype=torch.float32):
    """Analysis and synthesis banks of shape (2*C, 1, 2) (wavelet.py:6-20)."""
    dlo, dhi, rlo, rhi = db1_taps(dtype)
    dec = torch.stack([dlo, dhi], dim=0)[:, None].repeat(channels, 1, 1)
    rec = torch.stack([rlo, rhi], dim=0)[:, None].repeat(channels, 1, 1)
    return dec, rec


# --------------------------------------------------------------------------- transforms
def analysis_2d(x, bank):
    """(B,C,H,W) with even H,W -> (B,C,4,H/2,W/2)   (wavelet.py:62-67)."""
    b, c, h, w = x.shape
    y = F.conv2d(x, bank, stride=2, groups=c)
    return y.reshape(b, c, 4, h // 2, w // 2)


def synthesis_2d(coeffs, bank):
    """(B,C,4,h,w) -> (B,C,2h,2w)   (wavelet.py:70-75)."""
    b, c, _, h, w = coeffs.shape
    return F.conv_transpose2d(coeffs.reshape(b, 4 * c, h, w), bank, stride=2, groups=c)


def analysis_1d(x, bank):
    b, c, n = x.shape
    y = F.conv1d(x, bank, stride=2, groups=c)
    return y.reshape(b, c, 2, n // 2)


def synthesis_1d(coeffs, bank):
    b, c, _, n = coeffs.shape
    return F.conv_transpose1d(coeffs.reshape(b, 2 * c, n), bank, stride=2, groups=c)


# --------------------------------------------------------------------------- the layer
def wtconv2d_ref(x, base_w, base_b, base_scale, wt_ws: Sequence[torch.Tensor],
                 wt_scales: Sequence[torch.Tensor], stride: int = 1):
    """Forward of the 2-D layer.

    x (B,C,H,W); base_w (C,1,K,K); base_b (C,) or None; base_scale (1,C,1,1);
    wt_ws[i] (4C,1,K,K); wt_scales[i] (1,4C,1,1).  Everything in x.dtype.
    """
    c = x.shape[1]
    k = base_w.shape[-1]
    dec, rec = haar_filters_2d(c, x.dtype)
    dec, rec = dec.to(x.device), rec.to(x.device)

    low = x
    stash = []
    for w_l, s_l in zip(wt_ws, wt_scales):
        hh, ww = low.shape[2], low.shape[3]
        if hh % 2 or ww % 2:                                   # wtconv2d.py:49-51
            low = F.pad(low, (0, ww % 2, 0, hh % 2))
        sub = analysis_2d(low, dec)                            # :53
        low = sub[:, :, 0]                                     # :54 raw LL feeds next level
        bb, cc, _, h2, w2 = sub.shape
        filt = F.conv2d(sub.reshape(bb, 4 * cc, h2, w2), w_l, padding=k // 2, groups=4 * cc)
        filt = (s_l * filt).reshape(bb, cc, 4, h2, w2)         # :57-59
        stash.append((filt, (hh, ww)))

    carry = 0
    for filt, (hh, ww) in reversed(stash):                    # :66-76
        merged = torch.cat([(filt[:, :, 0] + carry).unsqueeze(2), filt[:, :, 1:4]], dim=2)
        carry = synthesis_2d(merged, rec)[:, :, :hh, :ww]

    out = base_scale * F.conv2d(x, base_w, base_b, padding=k // 2, groups=c) + carry  # :81-82
    if stride > 1:                                             # :33-36,:84-85
        out = F.avg_pool2d(out, kernel_size=1, stride=stride)
    return out


def wtconv1d_ref(x, base_w, base_b, base_scale, wt_ws, wt_scales, stride: int = 1):
    """Forward of the 1-D layer.  x (B,C,N); base_w (C,1,K); wt_ws[i] (2C,1,K);
    scales (1,C,1) / (1,2C,1).  Stride is a true average pool (wtconv1d.py:34)."""
    c = x.shape[1]
    k = base_w.shape[-1]
    dec, rec = haar_filters_1d(c, x.dtype)
    dec, rec = dec.to(x.device), rec.to(x.device)

    low = x
    stash = []
    for w_l, s_l in zip(wt_ws, wt_scales):
        n = low.shape[2]
        if n % 2:
            low = F.pad(low, (0, 1))
        sub = analysis_1d(low, dec)
        low = sub[:, :, 0]
        bb, cc, _, n2 = sub.shape
        filt = F.conv1d(sub.reshape(bb, 2 * cc, n2), w_l, padding=k // 2, groups=2 * cc)
        filt = (s_l * filt).reshape(bb, cc, 2, n2)
        stash.append((filt, n))

    carry = 0
    for filt, n in reversed(stash):
        merged = torch.cat([(filt[:, :, 0] + carry).unsqueeze(2), filt[:, :, 1:2]], dim=2)
        carry = synthesis_1d(merged, rec)[:, :, :n]

    out = base_scale * F.conv1d(x, base_w, base_b, padding=k // 2, groups=c) + carry
    if stride > 1:
        out = F.avg_pool1d(out, kernel_size=stride, stride=stride)
    return out


# --------------------------------------------------------------------------- modules
class _Scale(nn.Module):
    """Broadcast multiply by a learnable tensor (wtconv2d.py:89-97)."""

    def __init__(self, dims, init_scale=1.0):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(*dims) * init_scale)

    def forward(self, x):
        return torch.mul(self.weight, x)


class RefWTConv2d(nn.Module):
    """Oracle twin of the reference module: same sub-module names, the same order of
    random draws at construction (base conv, then level convs; wtconv2d.py:19-31), so
    a state dict or a seed gives the same parameters as the reference class would."""

    def __init__(self, in_channels, out_channels, kernel_size=5, stride=1, bias=True,
                 wt_levels=1, wt_type='db1'):
        super().__init__()
        assert in_channels == out_channels
        if wt_type not in ('db1', 'haar'):
            raise ValueError("oracle restates db1 only")
        c = in_channels
        self.in_channels, self.wt_levels, self.stride, self.dilation = c, wt_levels, stride, 1
        dec, rec = haar_filters_2d(c, torch.float32)
        self.wt_filter = nn.Parameter(dec, requires_grad=False)
        self.iwt_filter = nn.Parameter(rec, requires_grad=False)
        self.base_conv = nn.Conv2d(c, c, kernel_size, padding='same', groups=c, bias=bias)
        self.base_scale = _Scale([1, c, 1, 1])
        self.wavelet_convs = nn.ModuleList([
            nn.Conv2d(4 * c, 4 * c, kernel_size, padding='same', groups=4 * c, bias=False)
            for _ in range(wt_levels)])
        self.wavelet_scale = nn.ModuleList([
            _Scale([1, 4 * c, 1, 1], init_scale=0.1) for _ in range(wt_levels)])

    def forward(self, x):
        return wtconv2d_ref(
            x, self.base_conv.weight, self.base_conv.bias, self.base_scale.weight,
            [m.weight for m in self.wavelet_convs], [m.weight for m in self.wavelet_scale],
            self.stride)


class RefWTConv1d(nn.Module):
    """Oracle twin of the reference 1-D module (wtconv1d.py:8-36)."""

    def __init__(self, in_channels, out_channels, kernel_size=5, stride=1, bias=True,
                 wt_levels=1, wt_type='db1'):
        super().__init__()
        assert in_channels == out_channels
        if wt_type not in ('db1', 'haar'):
            raise ValueError("oracle restates db1 only")
        c = in_channels
        self.in_channels, self.wt_levels, self.stride, self.dilation = c, wt_levels, stride, 1
        dec, rec = haar_filters_1d(c, torch.float32)
        self.wt_filter = nn.Parameter(dec, requires_grad=False)
        self.iwt_filter = nn.Parameter(rec, requires_grad=False)
        self.base_conv = nn.Conv1d(c, c, kernel_size, padding='same', groups=c, bias=bias)
        self.base_scale = _Scale([1, c, 1])
        self.wavelet_convs = nn.ModuleList([
            nn.Conv1d(2 * c, 2 * c, kernel_size, padding='same', groups=2 * c, bias=False)
            for _ in range(wt_levels)])
        self.wavelet_scale = nn.ModuleList([
            _Scale([1, 2 * c, 1], init_scale=0.1) for _ in range(wt_levels)])

    def forward(self, x):
        return wtconv1d_ref(
            x, self.base_conv.weight, self.base_conv.bias, self.base_scale.weight,
            [m.weight for m in self.wavelet_convs], [m.weight for m in self.wavelet_scale],
            self.stride)


# --------------------------------------------------------------------------- helpers
def layer_grads(module: nn.Module, x: torch.Tensor, g: torch.Tensor):
    """Run forward + backward of an oracle module; returns (out, grad_x, {name: grad})."""
    for p in module.parameters():
        p.grad = None
    xr = x.detach().clone().requires_grad_(True)
    out = module(xr)
    out.backward(g)
    grads = {n: p.grad.detach().clone() for n, p in module.named_parameters() if p.grad is not None}
    return out.detach(), xr.grad.detach(), grads


def level_shapes(h: int, w: int, levels: int):
    """[(h0,w0), (h1,w1), ...]: the coefficient grid of level l is ceil of half the
    previous one (per-level padding, wtconv2d.py:47-51)."""
    out = [(h, w)]
    for _ in range(levels):
        h, w = (h + 1) // 2, (w + 1) // 2
        out.append((h, w))
    return out


def mac_per_pixel_2d(k: int, levels: int) -> float:
    return k * k * (1.0 + sum(4.0 ** (1 - l) for l in range(1, levels + 1)))


__all__ = [
    "db1_taps", "haar_filters_2d", "haar_filters_1d", "analysis_2d", "synthesis_2d",
    "analysis_1d", "synthesis_1d", "wtconv2d_ref", "wtconv1d_ref", "RefWTConv2d",
    "RefWTConv1d", "layer_grads", "level_shapes", "mac_per_pixel_2d",
]
