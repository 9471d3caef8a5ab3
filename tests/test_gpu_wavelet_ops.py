"""The stand-alone Haar transforms (wtconv.util.wavelet, fast_wtconv.cuda_haar) on the GPU against the oracle's
analysis / synthesis (the library restatement of wtconv/util/wavelet.py:46-75) and against their own algebra."""
import pytest
import torch

from oracle import wtconv_ref as R
import parity_util as U

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(2, 3, 8, 12), (1, 5, 2, 2), (3, 4, 56, 56), (1, 2, 30, 6)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_wavelet_2d_roundtrip_and_oracle(hip_device, shape, dtype):
    from wtconv.util import wavelet as Wv
    B, C, H, W = shape
    gen = torch.Generator().manual_seed(H * 100 + W)
    x = torch.randn(shape, generator=gen).to(dtype)
    dec, rec = Wv.create_2d_wavelet_filter("db1", C, C, torch.float)
    xd = x.to(hip_device)
    coef = Wv.wavelet_2d_transform(xd, dec.to(hip_device))
    assert coef.shape == (B, C, 4, H // 2, W // 2) and coef.dtype == dtype
    want = R.analysis_2d(x.double(), R.haar_filters_2d(C, torch.float64)[0])
    tol = {torch.float32: (1e-5, 1e-5), torch.bfloat16: (2e-2, 2e-2), torch.float16: (2e-3, 2e-3)}[dtype]
    torch.testing.assert_close(coef.double().cpu(), want, rtol=tol[0], atol=tol[1])
    back = Wv.inverse_2d_wavelet_transform(coef, rec.to(hip_device))
    assert back.shape == x.shape
    torch.testing.assert_close(back.double().cpu(), R.synthesis_2d(coef.double().cpu(), R.haar_filters_2d(C, torch.float64)[1]), rtol=tol[0], atol=tol[1])
    torch.testing.assert_close(back.double().cpu(), x.double(), rtol=3 * tol[0], atol=3 * tol[1])      # perfect reconstruction


@pytest.mark.parametrize("shape", [(2, 3, 64), (1, 1, 2), (2, 4, 4096), (1, 2, 1000)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_wavelet_1d_roundtrip_and_oracle(hip_device, shape, dtype):
    from wtconv.util import wavelet as Wv
    B, C, N = shape
    x = torch.randn(shape, generator=torch.Generator().manual_seed(N)).to(dtype)
    dec, rec = Wv.create_1d_wavelet_filter("db1", C, C, torch.float)
    coef = Wv.wavelet_1d_transform(x.to(hip_device), dec.to(hip_device))
    assert coef.shape == (B, C, 2, N // 2)
    tol = (1e-5, 1e-5) if dtype == torch.float32 else (2e-2, 2e-2)
    torch.testing.assert_close(coef.double().cpu(), R.analysis_1d(x.double(), R.haar_filters_1d(C, torch.float64)[0]), rtol=tol[0], atol=tol[1])
    back = Wv.inverse_1d_wavelet_transform(coef, rec.to(hip_device))
    torch.testing.assert_close(back.double().cpu(), R.synthesis_1d(coef.double().cpu(), R.haar_filters_1d(C, torch.float64)[1]), rtol=tol[0], atol=tol[1])
    torch.testing.assert_close(back.double().cpu(), x.double(), rtol=3 * tol[0], atol=3 * tol[1])


def test_wavelet_transforms_are_differentiable_adjoints(hip_device):
    """<A x, y> = <x, A^T y> with A^T = the inverse transform, through autograd."""
    from wtconv.util import wavelet as Wv
    dec, rec = Wv.create_2d_wavelet_filter("db1", 3, 3)
    dec, rec = dec.to(hip_device), rec.to(hip_device)
    x = torch.randn(2, 3, 10, 14, device=hip_device, dtype=torch.float32, requires_grad=True)
    y = torch.randn(2, 3, 4, 5, 7, device=hip_device)
    (Wv.wavelet_2d_transform(x, dec) * y).sum().backward()
    torch.testing.assert_close(x.grad, Wv.inverse_2d_wavelet_transform(y, rec), rtol=1e-6, atol=1e-6)
    c = torch.randn(2, 3, 4, 5, 7, device=hip_device, requires_grad=True)
    z = torch.randn(2, 3, 10, 14, device=hip_device)
    (Wv.inverse_2d_wavelet_transform(c, rec) * z).sum().backward()
    torch.testing.assert_close(c.grad, Wv.wavelet_2d_transform(z, dec), rtol=1e-6, atol=1e-6)


def test_filter_creation_and_argument_checks(hip_device):
    from wtconv.util import wavelet as Wv
    dec, rec = Wv.create_2d_wavelet_filter("db1", 2, 3)
    assert dec.shape == (8, 1, 2, 2) and rec.shape == (12, 1, 2, 2)
    r = 0.7071067811865476
    want = torch.tensor([[r * r, r * r], [r * r, r * r]], dtype=torch.float32)
    torch.testing.assert_close(dec[0, 0], want)
    torch.testing.assert_close(dec[3, 0], torch.tensor([[r * r, -r * r], [-r * r, r * r]], dtype=torch.float32))
    d1, r1 = Wv.create_1d_wavelet_filter("haar", 2, 2)
    assert d1.shape == (4, 1, 2) and torch.equal(d1, r1)
    with pytest.raises(NotImplementedError):
        Wv.create_2d_wavelet_filter("db2", 1, 1)
    x = torch.randn(1, 2, 4, 4, device=hip_device)
    with pytest.raises(NotImplementedError):
        Wv.wavelet_2d_transform(x, torch.ones(8, 1, 2, 2))
    with pytest.raises(ValueError, match="even"):
        Wv.wavelet_2d_transform(torch.randn(1, 2, 5, 4, device=hip_device), dec)
    with pytest.raises(RuntimeError, match="CPU"):
        Wv.wavelet_2d_transform(torch.randn(1, 2, 4, 4), dec)


def test_fast_twin_haar_utilities(hip_device):
    """haar2d pads odd extents, ihaar2d crops back: the round trip returns the input."""
    from fast_wtconv import cuda_haar as H
    x = torch.randn(2, 3, 7, 9, device=hip_device)
    c = H.haar2d(x)
    assert c.shape == (2, 3, 4, 4, 5)
    torch.testing.assert_close(H.ihaar2d(c, (7, 9)), x, rtol=1e-6, atol=1e-6)
    add = torch.randn_like(x)
    torch.testing.assert_close(H.ihaar2d_fused(c, add, (7, 9)), x + add, rtol=1e-6, atol=1e-6)
    H.check_kernel_size(7)
    with pytest.raises(ValueError):
        H.check_kernel_size(9)
    with pytest.raises(ValueError):
        H.check_kernel_size(4)
