"""State-dict converters between the key schemes the reference uses for the same weights.

* reference layer (wtconv/wtconv2d.py:19-31): ``base_conv.weight``, ``base_conv.bias``,
  ``base_scale.weight``, ``wavelet_convs.{i}.weight``, ``wavelet_scale.{i}.weight`` and the
  frozen filter banks ``wt_filter`` / ``iwt_filter``;
* fused twin (fast_wtconv/wtconv_cuda.py:86-104): ``base_weight``, ``base_bias``,
  ``base_scale``, ``wt_weights.{i}``, ``wt_scales.{i}`` (no filter banks);
* mmseg backbone (semantic_segmentation/translate_model_to_mmseg.py:8-41): the timm model's
  ``stem.*`` / ``stages.S.downsample.*`` / ``stages.S.blocks.B.*`` keys renamed to
  ``backbone.downsample_layers.*`` / ``backbone.stages.S.B.*``.

Tensors are passed through untouched (same layouts in every scheme: conv channel 4c+s is
sub-band s of channel c); only names change and the constant filter banks are dropped or
recreated.  Works on whole-model state dicts: every WTConv layer inside is found by its
parameter names.
"""
import re
from collections import OrderedDict

import torch

_REF_TO_FAST = (
    (re.compile(r"(^|\.)base_conv\.weight$"), r"\1base_weight"),
    (re.compile(r"(^|\.)base_conv\.bias$"), r"\1base_bias"),
    (re.compile(r"(^|\.)base_scale\.weight$"), r"\1base_scale"),
    (re.compile(r"(^|\.)wavelet_convs\.(\d+)\.weight$"), r"\1wt_weights.\2"),
    (re.compile(r"(^|\.)wavelet_scale\.(\d+)\.weight$"), r"\1wt_scales.\2"),
)
_FAST_TO_REF = (
    (re.compile(r"(^|\.)base_weight$"), r"\1base_conv.weight"),
    (re.compile(r"(^|\.)base_bias$"), r"\1base_conv.bias"),
    (re.compile(r"(^|\.)base_scale$"), r"\1base_scale.weight"),
    (re.compile(r"(^|\.)wt_weights\.(\d+)$"), r"\1wavelet_convs.\2.weight"),
    (re.compile(r"(^|\.)wt_scales\.(\d+)$"), r"\1wavelet_scale.\2.weight"),
)
_FILTER_KEY = re.compile(r"(^|\.)i?wt_filter$")


def _rename(key, table):
    for pat, rep in table:
        new, n = pat.subn(rep, key)
        if n:
            return new
    return key


def haar_filter_bank(channels, dims=2, dtype=torch.float32):
    """The frozen db1 banks the reference layer stores per module: (wt_filter, iwt_filter),
    each (4C,1,2,2) for dims=2 (wavelet.py:23-43) or (2C,1,2) for dims=1 (wavelet.py:6-20)."""
    from .modules import _db1_banks_1d, _db1_banks_2d
    dec, rec = (_db1_banks_2d if dims == 2 else _db1_banks_1d)(channels)
    return dec.to(dtype), rec.to(dtype)


def reference_to_fast(state_dict):
    """Reference-layer keys -> fused-twin keys; filter banks are dropped."""
    out = OrderedDict()
    for k, v in state_dict.items():
        if _FILTER_KEY.search(k):
            continue
        out[_rename(k, _REF_TO_FAST)] = v
    return out


def fast_to_reference(state_dict, with_filters=True):
    """Fused-twin keys -> reference-layer keys.  With `with_filters` the frozen db1 banks the
    reference module expects under strict loading are recreated next to every layer."""
    out = OrderedDict()
    for k, v in state_dict.items():
        new = _rename(k, _FAST_TO_REF)
        out[new] = v
        if with_filters and new.endswith("base_conv.weight") and new != k:
            prefix = new[: -len("base_conv.weight")]
            wt, iwt = haar_filter_bank(v.shape[0], dims=v.dim() - 2, dtype=v.dtype)
            out[prefix + "wt_filter"] = wt.to(v.device)
            out[prefix + "iwt_filter"] = iwt.to(v.device)
    return out


def timm_to_mmseg(state_dict):
    """WTConvNeXt (timm layout) -> the mmseg backbone's names; keys that the backbone does not
    hold (classifier head, final norm) are dropped, as the reference's script does."""
    out = OrderedDict()
    for k, v in state_dict.items():
        p = k.split(".")
        if p[0] == "stem" and len(p) >= 3:
            out["backbone.downsample_layers.0." + ".".join(p[1:])] = v
        elif p[0] == "stages" and len(p) >= 5 and p[2] == "downsample":
            out[f"backbone.downsample_layers.{p[1]}." + ".".join(p[3:])] = v
        elif p[0] == "stages" and len(p) >= 5 and p[2] == "blocks":
            s, b, what = p[1], p[3], p[4]
            if what == "gamma":
                out[f"backbone.stages.{s}.{b}.gamma"] = v
            elif what == "mlp":
                n = 1 if p[5] == "fc1" else 2
                out[f"backbone.stages.{s}.{b}.pointwise_conv{n}." + ".".join(p[6:])] = v
            elif what == "norm":
                out[f"backbone.stages.{s}.{b}.norm." + ".".join(p[5:])] = v
            elif what == "conv_dw":
                out[f"backbone.stages.{s}.{b}.depthwise_conv." + ".".join(p[5:])] = v
    return out


def mmseg_to_timm(state_dict):
    """Inverse of timm_to_mmseg for the keys it keeps."""
    out = OrderedDict()
    for k, v in state_dict.items():
        if not k.startswith("backbone."):
            continue
        p = k[len("backbone."):].split(".")
        if p[0] == "downsample_layers":
            rest = ".".join(p[2:])
            out[("stem." if p[1] == "0" else f"stages.{p[1]}.downsample.") + rest] = v
        elif p[0] == "stages":
            s, b, what = p[1], p[2], p[3]
            rest = ".".join(p[4:])
            if what == "gamma":
                out[f"stages.{s}.blocks.{b}.gamma"] = v
            elif what.startswith("pointwise_conv"):
                out[f"stages.{s}.blocks.{b}.mlp.fc{what[-1]}.{rest}"] = v
            elif what == "norm":
                out[f"stages.{s}.blocks.{b}.norm.{rest}"] = v
            elif what == "depthwise_conv":
                out[f"stages.{s}.blocks.{b}.conv_dw.{rest}"] = v
    return out
