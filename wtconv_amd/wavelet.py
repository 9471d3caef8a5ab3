"""The reference's wavelet utilities (wtconv/util/wavelet.py:6-75) for the Haar wavelet: the db1 filter banks in closed
form and the single-level transforms as HIP kernels (`wtconv_haar2d`, `wtconv_haar1d` of the C ABI).

PyWavelets is not a dependency: `create_*_wavelet_filter` knows 'db1' / 'haar' only (the four db1 tap vectors are
+-1/sqrt 2) and raises NotImplementedError for any other wavelet.  The transforms take the filter bank argument the
reference passes around, check that it is the db1 bank, and run on the GPU; they are differentiable (each transform is
the other's adjoint).  CPU tensors are refused: there is no fallback implementation.
"""
import ctypes

import torch

from . import _lib

_R = 0.7071067811865476
_DT = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}


def _taps(wave, dtype):
    if wave not in ("db1", "haar"):
        raise NotImplementedError(f"wavelet {wave!r}: only the Haar wavelet ('db1') is built in (no PyWavelets tables)")
    # dec_lo[::-1], dec_hi[::-1], rec_lo, rec_hi of PyWavelets' db1
    lo = torch.tensor([_R, _R], dtype=dtype)
    hi = torch.tensor([_R, -_R], dtype=dtype)
    return lo, hi, lo.clone(), hi.clone()


def create_1d_wavelet_filter(wave, in_size, out_size, type=torch.float):
    """(dec_filters (2*in_size, 1, 2), rec_filters (2*out_size, 1, 2)), built as wavelet.py:6-20 builds them."""
    dlo, dhi, rlo, rhi = _taps(wave, type)
    dec = torch.stack([dlo, dhi], dim=0)[:, None].repeat(in_size, 1, 1)
    rec = torch.stack([rlo, rhi], dim=0)[:, None].repeat(out_size, 1, 1)
    return dec, rec


def create_2d_wavelet_filter(wave, in_size, out_size, type=torch.float):
    """(dec_filters (4*in_size, 1, 2, 2), rec_filters (4*out_size, 1, 2, 2)), built as wavelet.py:23-43 builds them."""
    dlo, dhi, rlo, rhi = _taps(wave, type)

    def bank(lo, hi, n):
        quad = torch.stack([lo.unsqueeze(0) * lo.unsqueeze(1), lo.unsqueeze(0) * hi.unsqueeze(1),
                            hi.unsqueeze(0) * lo.unsqueeze(1), hi.unsqueeze(0) * hi.unsqueeze(1)], dim=0)
        return quad[:, None].repeat(n, 1, 1, 1)
    return bank(dlo, dhi, in_size), bank(rlo, rhi, out_size)


def _check_bank(filters, channels, dims):
    """The kernels compute the db1 transform whatever `filters` holds, so anything else must be refused."""
    S = 4 if dims == 2 else 2
    shape = (S * channels, 1, 2, 2) if dims == 2 else (S * channels, 1, 2)
    if tuple(filters.shape) != shape:
        raise ValueError(f"filters of shape {tuple(filters.shape)}: expected the db1 bank {shape}")
    ref = (create_2d_wavelet_filter if dims == 2 else create_1d_wavelet_filter)("db1", 1, 1, torch.float32)[0]
    got = filters[:S].detach().to(device="cpu", dtype=torch.float32)      # (a few values: the first channel's bank)
    if not torch.allclose(got, ref, rtol=0, atol=4e-3):                   # bf16 banks included
        raise NotImplementedError("only the Haar (db1) filter bank is supported by the HIP transforms")


def _launch(x, out, dims, inverse):
    lib = _lib.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    with torch.cuda.device(x.device):
        if dims == 2:
            H, W = (out.shape[-2:] if inverse else x.shape[-2:])
            planes = x.shape[0] * x.shape[1]
            rc = lib.wtconv_haar2d(x.data_ptr(), out.data_ptr(), planes, H, W, _DT[x.dtype], int(inverse), stream)
        else:
            N = out.shape[-1] if inverse else x.shape[-1]
            rc = lib.wtconv_haar1d(x.data_ptr(), out.data_ptr(), x.shape[0] * x.shape[1], N, _DT[x.dtype], int(inverse),
                                   stream)
    if rc:
        _lib.check(rc, "wtconv_haar%dd" % dims)
    return out


def _prep(x, ndim, what):
    if not x.is_cuda:
        raise RuntimeError(f"{what}: CPU tensor; the HIP transforms have no CPU fallback")
    if x.dtype not in _DT:
        raise TypeError(f"{what}: dtype {x.dtype} is not float32, bfloat16 or float16")
    if x.dim() != ndim:
        raise ValueError(f"{what}: expected a {ndim}-dimensional tensor, got shape {tuple(x.shape)}")
    return x.contiguous()


class _Haar(torch.autograd.Function):
    """dims, inverse: which transform; the backward pass is the opposite one (the transforms are orthogonal)."""

    @staticmethod
    def forward(ctx, x, dims, inverse):
        ctx.dims, ctx.inverse = dims, inverse
        if dims == 2:
            if inverse:
                b, c, _, h, w = x.shape
                out = x.new_empty((b, c, 2 * h, 2 * w))
            else:
                b, c, h, w = x.shape
                out = x.new_empty((b, c, 4, h // 2, w // 2))
        else:
            if inverse:
                b, c, _, n = x.shape
                out = x.new_empty((b, c, 2 * n))
            else:
                b, c, n = x.shape
                out = x.new_empty((b, c, 2, n // 2))
        return _launch(x, out, dims, inverse)

    @staticmethod
    def backward(ctx, g):
        return _Haar.apply(g.contiguous(), ctx.dims, not ctx.inverse), None, None


def wavelet_2d_transform(x, filters):
    """x (b, c, h, w), h and w even -> (b, c, 4, h/2, w/2), sub-bands LL, LH, HL, HH (wavelet.py:62-67)."""
    x = _prep(x, 4, "wavelet_2d_transform")
    if x.shape[2] % 2 or x.shape[3] % 2:
        raise ValueError(f"wavelet_2d_transform: extents must be even, got {tuple(x.shape[2:])} (pad first, as wtconv2d.py:49-51 does)")
    _check_bank(filters, x.shape[1], 2)
    return _Haar.apply(x, 2, False)


def inverse_2d_wavelet_transform(x, filters):
    """x (b, c, 4, h, w) -> (b, c, 2h, 2w) (wavelet.py:70-75)."""
    x = _prep(x, 5, "inverse_2d_wavelet_transform")
    if x.shape[2] != 4:
        raise ValueError(f"inverse_2d_wavelet_transform: expected 4 sub-bands, got shape {tuple(x.shape)}")
    _check_bank(filters, x.shape[1], 2)
    return _Haar.apply(x, 2, True)


def wavelet_1d_transform(x, filters):
    """x (b, c, l), l even -> (b, c, 2, l/2), low-pass then high-pass (wavelet.py:46-51)."""
    x = _prep(x, 3, "wavelet_1d_transform")
    if x.shape[2] % 2:
        raise ValueError(f"wavelet_1d_transform: the length must be even, got {x.shape[2]} (pad first, as wtconv1d.py:49-51 does)")
    _check_bank(filters, x.shape[1], 1)
    return _Haar.apply(x, 1, False)


def inverse_1d_wavelet_transform(x, filters):
    """x (b, c, 2, l) -> (b, c, 2l) (wavelet.py:54-59)."""
    x = _prep(x, 4, "inverse_1d_wavelet_transform")
    if x.shape[2] != 2:
        raise ValueError(f"inverse_1d_wavelet_transform: expected 2 sub-bands, got shape {tuple(x.shape)}")
    _check_bank(filters, x.shape[1], 1)
    return _Haar.apply(x, 1, True)
