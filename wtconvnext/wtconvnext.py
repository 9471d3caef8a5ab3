"""WTConvNeXt in plain PyTorch: the caller harness of the WTConv layer.

Mirrors the structure of the reference model (``wtconvnext/wtconvnext.py:49-140`` block,
``:143-213`` stage, ``:216-480`` model, ``:483-493`` init, ``:570-588`` variants) without
timm, which is not importable here: ConvNeXt macro layout with the 7x7 depthwise conv of
every block replaced by a ``WTConv2d`` (``kernel_size=5``, ``wt_levels=(5,4,3,2)`` per
stage).  Module and parameter names follow the reference's state dict
(``stem.0``, ``stages.i.downsample.1``, ``stages.i.blocks.j.conv_dw.*``, ``.norm``,
``.mlp.fc1/fc2``, ``.gamma``, ``head.norm``, ``head.fc``).  The only thing the reference
holds that pins this shell is the parameter count printed in ``logs/val_*.out:4``; timm's
layer internals (LayerNorm2d, Mlp, NormMlpClassifierHead, trunc_normal_) are restated from
their documented behaviour.
"""
from functools import partial
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from wtconv import WTConv2d


def _block_ops():
    """The fused block passes of the HIP library, or None where it is not importable (CPU-only use of the harness)."""
    try:
        from wtconv_amd import block_ops
        return block_ops
    except ImportError:
        return None


class LayerNorm2d(nn.LayerNorm):
    """LayerNorm over the channel dimension of an NCHW tensor."""

    def __init__(self, num_channels, eps=1e-6):
        super().__init__(num_channels, eps=eps)

    def forward(self, x):
        ops = _block_ops()
        if (ops is not None and self.elementwise_affine and self.bias is not None and x.is_contiguous()
                and ops.usable(x, self.weight, self.bias, training=True)):
            if ops.records(x, self.weight, self.bias):      # one kernel each way
                return ops.channel_norm_fn(x, self.weight, self.bias, self.eps, False)
            return ops.channel_norm(x, self.weight, self.bias, self.eps, nhwc=False)
        x = x.permute(0, 2, 3, 1)
        x = F.layer_norm(x, self.normalized_shape, self.weight, self.bias, self.eps)
        return x.permute(0, 3, 1, 2)


class Mlp(nn.Module):
    def __init__(self, dim, hidden):
        super().__init__()
        self.fc1 = nn.Linear(dim, hidden)
        self.act = nn.GELU()
        self.fc2 = nn.Linear(hidden, dim)

    def forward(self, x):
        return self.fc2(self.act(self.fc1(x)))


class DropPath(nn.Module):
    """Stochastic depth per sample: in training a sample's residual branch is dropped with
    probability `drop_prob` and the kept ones are scaled by 1 / (1 - drop_prob)."""

    def __init__(self, drop_prob: float = 0.):
        super().__init__()
        self.drop_prob = float(drop_prob)

    def forward(self, x):
        if self.drop_prob == 0. or not self.training:
            return x
        keep = 1. - self.drop_prob
        mask = x.new_empty((x.shape[0],) + (1,) * (x.dim() - 1)).bernoulli_(keep)
        return x * mask.div_(keep)


class WTConvNeXtBlock(nn.Module):
    """conv_dw (WTConv2d) -> NHWC LayerNorm -> Linear -> GELU -> Linear -> layer scale -> + shortcut."""

    def __init__(self, dim, kernel_size=5, mlp_ratio=4, conv_bias=True, ls_init_value=1e-6, wt_levels=0,
                 wtconv_class=None, norm_eps=1e-6, drop_path=0.):
        super().__init__()
        conv_class = wtconv_class if wtconv_class is not None else WTConv2d
        self.conv_dw = conv_class(dim, dim, kernel_size=kernel_size, stride=1, bias=conv_bias, wt_levels=wt_levels)
        self.norm = nn.LayerNorm(dim, eps=norm_eps)
        self.mlp = Mlp(dim, int(mlp_ratio * dim))
        self.gamma = nn.Parameter(ls_init_value * torch.ones(dim)) if ls_init_value is not None else None
        self.drop_path = DropPath(drop_path) if drop_path > 0. else nn.Identity()

    def forward(self, x):
        shortcut = x
        x = self.conv_dw(x)
        ops = _block_ops()
        drops = self.training and not isinstance(self.drop_path, nn.Identity)
        if (ops is not None and not drops and x.is_contiguous() and shortcut.is_contiguous()
                and ops.usable(x, self.norm.weight, self.norm.bias, self.gamma, training=True)
                and ops.usable(shortcut, training=True)):
            # on the GPU: NCHW -> LayerNorm -> NHWC, and NHWC -> layer scale -> + shortcut -> NCHW, are one kernel
            # each instead of a layout copy plus an elementwise pass each; where autograd records, through the
            # functions that carry the backward kernels
            if ops.records(x, self.norm.weight, self.norm.bias):
                y = ops.channel_norm_fn(x, self.norm.weight, self.norm.bias, self.norm.eps, True)
            else:
                y = ops.channel_norm(x, self.norm.weight, self.norm.bias, self.norm.eps, nhwc=True)
            y = self.mlp(y)
            # the MLP may change the dtype; the residual kernels take a tensor of the shortcut's type
            if ops.usable_nhwc(y, shortcut):
                y = y.contiguous()
                if ops.records(y, shortcut, self.gamma):
                    if self.gamma is not None:
                        return ops.block_residual_fn(y, shortcut, self.gamma)
                else:
                    return ops.block_residual(y, shortcut, self.gamma)
            x = y.permute(0, 3, 1, 2)
        else:
            x = x.permute(0, 2, 3, 1)
            x = self.mlp(self.norm(x))
            x = x.permute(0, 3, 1, 2)
        if self.gamma is not None:
            x = x.mul(self.gamma.reshape(1, -1, 1, 1))
        return self.drop_path(x) + shortcut


class WTConvNeXtStage(nn.Module):
    def __init__(self, in_chs, out_chs, kernel_size=5, stride=2, depth=2, ls_init_value=1e-6, conv_bias=True,
                 wt_levels=0, wtconv_class=None, norm_eps=1e-6, drop_path_rates=None):
        super().__init__()
        drop_path_rates = drop_path_rates or [0.] * depth
        self.grad_checkpointing = False
        if in_chs != out_chs or stride > 1:
            self.downsample = nn.Sequential(
                LayerNorm2d(in_chs, eps=norm_eps),
                nn.Conv2d(in_chs, out_chs, kernel_size=2 if stride > 1 else 1, stride=stride, bias=conv_bias))
        else:
            self.downsample = nn.Identity()
        self.blocks = nn.Sequential(*[
            WTConvNeXtBlock(out_chs, kernel_size=kernel_size, conv_bias=conv_bias, ls_init_value=ls_init_value,
                            wt_levels=wt_levels, wtconv_class=wtconv_class, norm_eps=norm_eps,
                            drop_path=drop_path_rates[i])
            for i in range(depth)])

    def forward(self, x):
        x = self.downsample(x)
        if self.grad_checkpointing and torch.is_grad_enabled():
            from torch.utils.checkpoint import checkpoint
            for blk in self.blocks:
                x = checkpoint(blk, x, use_reentrant=False)
            return x
        return self.blocks(x)


class _Head(nn.Module):
    """global average pool -> LayerNorm2d -> flatten -> Linear (the ConvNeXt head order)."""

    def __init__(self, in_features, num_classes, norm_eps=1e-6):
        super().__init__()
        self.norm = LayerNorm2d(in_features, eps=norm_eps)
        self.fc = nn.Linear(in_features, num_classes) if num_classes > 0 else nn.Identity()

    def reset(self, num_classes):
        self.fc = nn.Linear(self.norm.normalized_shape[0], num_classes) if num_classes > 0 else nn.Identity()

    def forward(self, x, pre_logits: bool = False):
        x = x.mean(dim=(2, 3), keepdim=True)
        x = self.norm(x).flatten(1)
        return x if pre_logits else self.fc(x)


def _init_weights(module, name="", head_init_scale=1.0):
    """trunc-normal(0.02) on every Conv2d / Linear weight, zero biases -- which, as in the
    reference, also re-initialises the nn.Conv2d holders inside WTConv2d; the classifier is
    scaled by `head_init_scale` (wtconvnext.py:483-493 of the reference)."""
    if isinstance(module, (nn.Conv2d, nn.Linear)):
        nn.init.trunc_normal_(module.weight, std=.02)
        if module.bias is not None:
            nn.init.zeros_(module.bias)
        if isinstance(module, nn.Linear) and name.startswith("head."):
            module.weight.data.mul_(head_init_scale)
            module.bias.data.mul_(head_init_scale)


class WTConvNeXt(nn.Module):
    def __init__(self, in_chans: int = 3, num_classes: int = 1000, depths: Tuple[int, ...] = (3, 3, 9, 3),
                 dims: Tuple[int, ...] = (96, 192, 384, 768), kernel_sizes=5, ls_init_value: Optional[float] = 1e-6,
                 patch_size: int = 4, conv_bias: bool = True, wt_levels: Tuple[int, ...] = (5, 4, 3, 2),
                 wtconv_class: Optional[type] = None, norm_eps: float = 1e-6, drop_path_rate: float = 0.,
                 head_init_scale: float = 1.):
        super().__init__()
        # stochastic depth grows linearly over all blocks (wtconvnext.py:309 of the reference)
        nblk = sum(depths)
        flat = [drop_path_rate * i / max(nblk - 1, 1) for i in range(nblk)]
        dp_rates, pos = [], 0
        for d in depths:
            dp_rates.append(flat[pos:pos + d])
            pos += d
        if isinstance(kernel_sizes, int):
            kernel_sizes = (kernel_sizes,) * 4
        self.num_classes = num_classes
        self.stem = nn.Sequential(
            nn.Conv2d(in_chans, dims[0], kernel_size=patch_size, stride=patch_size, bias=conv_bias),
            LayerNorm2d(dims[0], eps=norm_eps))
        stages, prev = [], dims[0]
        for i in range(4):
            stages.append(WTConvNeXtStage(prev, dims[i], kernel_size=kernel_sizes[i], stride=2 if i > 0 else 1,
                                          depth=depths[i], ls_init_value=ls_init_value, conv_bias=conv_bias,
                                          wt_levels=wt_levels[i], wtconv_class=wtconv_class, norm_eps=norm_eps,
                                          drop_path_rates=dp_rates[i]))
            prev = dims[i]
        self.stages = nn.Sequential(*stages)
        self.num_features = prev
        self.head = _Head(prev, num_classes, norm_eps=norm_eps)
        for name, module in self.named_modules():
            _init_weights(module, name, head_init_scale)

    def no_weight_decay(self):
        return {k for k, _ in self.named_parameters()
                if 'wavelet_scale' in k or 'wt_scales' in k or 'base_scale' in k}

    def get_classifier(self):
        return self.head.fc

    def reset_classifier(self, num_classes: int):
        self.num_classes = num_classes
        self.head.reset(num_classes)

    def set_grad_checkpointing(self, enable: bool = True):
        for s in self.stages:
            s.grad_checkpointing = enable

    def forward_features(self, x):
        return self.stages(self.stem(x))

    def forward_head(self, x, pre_logits: bool = False):
        return self.head(x, pre_logits=pre_logits)

    def forward(self, x):
        return self.forward_head(self.forward_features(x))


def wtconvnext_tiny(**kwargs) -> WTConvNeXt:
    return WTConvNeXt(**dict(dict(depths=(3, 3, 9, 3), dims=(96, 192, 384, 768)), **kwargs))


def wtconvnext_small(**kwargs) -> WTConvNeXt:
    return WTConvNeXt(**dict(dict(depths=(3, 3, 27, 3), dims=(96, 192, 384, 768)), **kwargs))


def wtconvnext_base(**kwargs) -> WTConvNeXt:
    return WTConvNeXt(**dict(dict(depths=(3, 3, 27, 3), dims=(128, 256, 512, 1024)), **kwargs))
