"""CPU-side checks of the wavelet utilities: the closed-form db1 banks against the oracle's (built as
wtconv/util/wavelet.py:6-43 builds them) and the refusals that need no GPU."""
import pytest
import torch

from oracle import wtconv_ref as R


def test_db1_banks_match_the_oracle():
    from wtconv.util import wavelet as Wv
    for c_in, c_out in ((1, 1), (3, 5)):
        dec, rec = Wv.create_2d_wavelet_filter("db1", c_in, c_out, torch.float)
        assert torch.equal(dec, R.haar_filters_2d(c_in)[0]) and torch.equal(rec, R.haar_filters_2d(c_out)[1])
        d1, r1 = Wv.create_1d_wavelet_filter("db1", c_in, c_out, torch.float)
        assert torch.equal(d1, R.haar_filters_1d(c_in)[0]) and torch.equal(r1, R.haar_filters_1d(c_out)[1])
    dec64, _ = Wv.create_2d_wavelet_filter("haar", 2, 2, torch.float64)
    assert dec64.dtype == torch.float64 and dec64.shape == (8, 1, 2, 2)


def test_refusals_without_a_gpu():
    from wtconv.util import wavelet as Wv
    with pytest.raises(NotImplementedError):
        Wv.create_1d_wavelet_filter("sym4", 1, 1)
    dec, _ = Wv.create_2d_wavelet_filter("db1", 2, 2)
    with pytest.raises(RuntimeError, match="CPU"):
        Wv.wavelet_2d_transform(torch.zeros(1, 2, 4, 4), dec)
    from fast_wtconv import cuda_haar
    cuda_haar.check_kernel_size(5)
    with pytest.raises(ValueError):
        cuda_haar.check_kernel_size(6)
