"""Import path of the reference's wavelet utilities (wtconv/util/wavelet.py), backed by the HIP kernels."""
from wtconv_amd.wavelet import (create_1d_wavelet_filter, create_2d_wavelet_filter, wavelet_1d_transform,  # noqa: F401
                                inverse_1d_wavelet_transform, wavelet_2d_transform, inverse_2d_wavelet_transform)
