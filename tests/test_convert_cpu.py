"""Checkpoint interop: key converters between the reference layer, its fused twin and the
mmseg backbone naming (CPU only: no kernel is called, modules are only constructed)."""
import torch

import wtconv
from fast_wtconv.wtconv_cuda import WTConv2d as FastWTConv2d
from wtconv.wtconv1d import WTConv1d
from wtconv_amd import convert


def test_reference_to_fast_and_back_strict():
    torch.manual_seed(0)
    ref = wtconv.WTConv2d(6, 6, kernel_size=5, wt_levels=3)
    fast = FastWTConv2d(6, 6, kernel_size=5, wt_levels=3)
    sd = convert.reference_to_fast(ref.state_dict())
    assert set(sd) == set(fast.state_dict())
    fast.load_state_dict(sd, strict=True)
    for a, b in ((ref.base_conv.weight, fast.base_weight), (ref.base_conv.bias, fast.base_bias),
                 (ref.base_scale.weight, fast.base_scale),
                 (ref.wavelet_convs[2].weight, fast.wt_weights[2]),
                 (ref.wavelet_scale[1].weight, fast.wt_scales[1])):
        assert torch.equal(a, b)
    back = convert.fast_to_reference(fast.state_dict())
    ref2 = wtconv.WTConv2d(6, 6, kernel_size=5, wt_levels=3)
    ref2.load_state_dict(back, strict=True)
    for k, v in ref.state_dict().items():
        assert torch.equal(v, ref2.state_dict()[k]), k


def test_filters_recreated_match_module_1d_and_2d():
    m2 = wtconv.WTConv2d(3, 3, wt_levels=1)
    wt, iwt = convert.haar_filter_bank(3, dims=2)
    assert torch.equal(wt, m2.wt_filter) and torch.equal(iwt, m2.iwt_filter)
    m1 = WTConv1d(3, 3, wt_levels=1)
    wt, iwt = convert.haar_filter_bank(3, dims=1)
    assert torch.equal(wt, m1.wt_filter) and torch.equal(iwt, m1.iwt_filter)


def test_whole_model_state_dict_round_trip():
    import wtconvnext
    torch.manual_seed(0)
    model = wtconvnext.wtconvnext_tiny()
    sd = model.state_dict()
    fast = convert.reference_to_fast(sd)
    assert not any(k.endswith("wt_filter") for k in fast)
    assert any(k.endswith("conv_dw.wt_weights.0") for k in fast)
    back = convert.fast_to_reference(fast)
    assert set(back) == set(sd)
    model2 = wtconvnext.wtconvnext_tiny()
    model2.load_state_dict(back, strict=True)


def test_timm_mmseg_round_trip():
    import wtconvnext
    sd = wtconvnext.wtconvnext_tiny().state_dict()
    mm = convert.timm_to_mmseg(sd)
    assert "backbone.downsample_layers.0.0.weight" in mm
    assert "backbone.stages.0.0.depthwise_conv.base_conv.weight" in mm
    assert "backbone.stages.2.5.pointwise_conv2.bias" in mm
    assert not any(k.startswith("backbone.head") for k in mm)
    back = convert.mmseg_to_timm(mm)
    kept = {k for k in sd if not k.startswith(("head.", "norm_pre."))}
    assert set(back) == kept
    for k in kept:
        assert back[k] is sd[k]
