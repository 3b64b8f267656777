"""ConvNeXt-1D / ConvNeXt-1D++ harness around the MI355X oriented depthwise convolution.

This is the caller side of the hot path: the network of the reference's
``models/convnext.py`` (variants ``"1d"`` and ``"1dpp"``: Stem1D ``:132-191``, Block1D
``:255-319``, Block1DPP ``:322-399``, ConvNeXt ``:495-610``, kernel-size tables ``:479-492``,
angle assignment ``:60-77,111-114``), written against ``DepthwiseOrientedConv1d`` of this
package.  Module and parameter names are the reference's (``downsample_layers.N``,
``stages.i.j.dwconv{,1,2}``, ``norm``, ``pwconv1/2``, ``gamma``, ``head``), so a reference
checkpoint's state_dict loads with ``strict=True``.  It exists to measure images/s with random
weights; training recipes, data loading and timm registration are not part of it.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import fused
from .dwoconv1d import DepthwiseOrientedConv1d

# (block kernel sizes, stem kernel size) per variant -- models/convnext.py:485-492
_VARIANTS = {"1d": ((31,), 31), "1dpp": ((15, 31), 15)}
# per-stage block kernel sizes of the dense-prediction backbone (cropped for the coarse stages)
# -- semantic_segmentation/backbone/convnext.py:316-327
_BACKBONE_BLOCK_SIZES = {"1d": ((31,), (31,), (27,), (13,)),
                         "1dpp": ((15, 31), (15, 31), (15, 27), (13, 13))}


def channel_angles(channels, n_dir=8, layer_offset=0.0):
    """theta_c = pi * ((g/n_dir + layer_offset) mod 1) with g = (n_dir*(c+1) - 1) // channels:
    contiguous groups of about channels/n_dir channels share a direction
    (models/convnext.py:60-77,111-114)."""
    return [math.pi * ((((n_dir * (c + 1) - 1) // channels) / n_dir + layer_offset) % 1.0)
            for c in range(channels)]


class ConvWrapper(nn.Module):
    """Holds the operator as ``.conv``: the backbone's parameter naming
    (semantic_segmentation/backbone/convnext.py:74-80)."""

    def __init__(self, conv):
        super().__init__()
        self.conv = conv

    def forward(self, x):
        return self.conv(x)


def oriented_conv(channels, kernel_size, *, stride=1, padding=None, n_dir=8, layer_offset=0.0,
                  nhwc=False, resid=False, arbitrary_size=False, wrapped=False):
    """models/convnext.py:80-128 (get_convolution_1d); ``wrapped`` gives the backbone's form
    (semantic_segmentation/backbone/convnext.py:82-104: arbitrary sizes, inside a wrapper)."""
    conv = DepthwiseOrientedConv1d(
        channels, channels, kernel_size, groups=channels, stride=stride,
        padding=kernel_size // 2 if padding is None else padding, bias=True,
        angle=channel_angles(channels, n_dir, layer_offset), nhwc=nhwc, resid=resid,
        arbitrary_size=arbitrary_size or wrapped)
    return ConvWrapper(conv) if wrapped else conv


def _odd_layer_offset(index):
    """+90 degrees on layers at odd depth (models/convnext.py:68-72 with the cycle enabled,
    which it is for the 1d and 1dpp variants, :530)."""
    return (index % 2) / 2


class ChannelsFirstLayerNorm(nn.Module):
    """LayerNorm over dim 1 of an NCHW tensor (models/convnext.py:29-56, channels_first)."""

    def __init__(self, channels, eps=1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(channels))
        self.bias = nn.Parameter(torch.zeros(channels))
        self.eps = eps

    def forward(self, x):
        if fused.usable(x, x.shape[1], tiled=True):
            y = fused.nchw_layernorm_nhwc(x, self.weight, self.bias, self.eps)
        else:
            y = F.layer_norm(x.permute(0, 2, 3, 1), self.weight.shape, self.weight, self.bias,
                             self.eps)
        return y.permute(0, 3, 1, 2)


class StochasticDepth(nn.Module):
    """Drops the residual branch of whole samples with probability p while training."""

    def __init__(self, p):
        super().__init__()
        self.p = float(p)

    def forward(self, x):
        if not self.training or self.p == 0.0:
            return x
        keep = x.new_empty((x.shape[0],) + (1,) * (x.dim() - 1)).bernoulli_(1.0 - self.p)
        return x * keep / (1.0 - self.p)


class Stem1D(nn.Module):
    """3 -> dim1 pointwise, two stride-2 oriented convs (NHWC) with LayerNorm + GELU, dim1 -> dim2
    pointwise, LayerNorm; NCHW in, NCHW out at 1/4 resolution (models/convnext.py:132-191)."""

    def __init__(self, dim0, dim1, dim2, kernel_size, arbitrary_size=False, wrapped=False):
        super().__init__()
        self.pw1 = nn.Linear(dim0, dim1)
        self.pw2 = nn.Linear(dim1, dim2)
        pad = (kernel_size - 2) // 2  # shapes the parent Conv2d only; compute pads K // 2
        self.dw1 = oriented_conv(dim1, kernel_size, stride=2, padding=pad, nhwc=True,
                                 layer_offset=_odd_layer_offset(0), arbitrary_size=arbitrary_size,
                                 wrapped=wrapped)
        self.dw2 = oriented_conv(dim1, kernel_size, stride=2, padding=pad, nhwc=True,
                                 layer_offset=_odd_layer_offset(1), arbitrary_size=arbitrary_size,
                                 wrapped=wrapped)
        self.norm1 = nn.LayerNorm(dim1, eps=1e-6)
        self.norm2 = nn.LayerNorm(dim1, eps=1e-6)
        self.norm3 = nn.LayerNorm(dim2, eps=1e-6)

    def forward(self, x):
        x = x.permute(0, 2, 3, 1).contiguous()
        dw1 = self.dw1.conv if isinstance(self.dw1, ConvWrapper) else self.dw1
        if (fused.usable(x, self.pw1.out_features, tiled=True) and x.shape[-1] <= 4
                and self.pw1.out_features % 4 == 0
                and fused.usable(x, self.pw2.out_features, tiled=True)):
            # the same values with pw1 applied on the way into dw1 (its 64-channel output is
            # never written), and each LayerNorm (+ GELU) and the final transpose as one pass
            x = fused.pointwise_dwconv_nhwc(x, self.pw1, dw1)
            x = fused.layernorm_nhwc(x, self.norm1.weight, self.norm1.bias, self.norm1.eps,
                                     gelu=True)
            x = fused.layernorm_nhwc(self.dw2(x), self.norm2.weight, self.norm2.bias,
                                     self.norm2.eps, gelu=True)
            x = fused.layernorm_nhwc(self.pw2(x), self.norm3.weight, self.norm3.bias,
                                     self.norm3.eps)
            return fused.nhwc_scale_add_nchw(x)
        x = self.pw1(x)
        x = F.gelu(self.norm1(self.dw1(x)))
        x = F.gelu(self.norm2(self.dw2(x)))
        x = self.norm3(self.pw2(x))
        return x.permute(0, 3, 1, 2).contiguous()


class Block(nn.Module):
    """ConvNeXt-1D block (one oriented conv, models/convnext.py:255-319) or 1D++ block (a second
    oriented conv with a residual tap on the 4*dim hidden tensor in NHWC, :322-399)."""

    def __init__(self, dim, kernel_sizes, plus_plus, drop_path=0.0, layer_scale_init_value=1e-6,
                 layer_offset=0.0, n_dir=8, arbitrary_size=False, wrapped=False):
        super().__init__()
        self.norm = nn.LayerNorm(dim, eps=1e-6)
        self.pwconv1 = nn.Linear(dim, 4 * dim)
        self.pwconv2 = nn.Linear(4 * dim, dim)
        self.gamma = (nn.Parameter(layer_scale_init_value * torch.ones(dim))
                      if layer_scale_init_value > 0 else None)
        self.drop_path = StochasticDepth(drop_path) if drop_path > 0.0 else nn.Identity()
        first = oriented_conv(dim, kernel_sizes[0], n_dir=n_dir, layer_offset=layer_offset,
                              arbitrary_size=arbitrary_size, wrapped=wrapped)
        if plus_plus:
            self.dwconv1 = first
            self.dwconv2 = oriented_conv(4 * dim, kernel_sizes[1], n_dir=n_dir, nhwc=True,
                                         resid=True, layer_offset=layer_offset,
                                         arbitrary_size=arbitrary_size, wrapped=wrapped)
        else:
            self.dwconv = first
        self.plus_plus = plus_plus

    def forward(self, x):
        y = (self.dwconv1 if self.plus_plus else self.dwconv)(x)
        fuse = fused.usable(y, y.shape[1], tiled=True) and not self.training
        if fuse:  # permute + LayerNorm as one pass
            y = fused.nchw_layernorm_nhwc(y, self.norm.weight, self.norm.bias, self.norm.eps)
        else:
            y = self.norm(y.permute(0, 2, 3, 1).contiguous())
        y = F.gelu(self.pwconv1(y))
        if self.plus_plus:
            y = self.dwconv2(y)
        y = self.pwconv2(y)
        if fuse:  # layer scale + permute + residual as one pass (no stochastic depth in eval)
            return fused.nhwc_scale_add_nchw(y, self.gamma, x)
        if self.gamma is not None:
            y = self.gamma * y
        return x + self.drop_path(y.permute(0, 3, 1, 2).contiguous())


class ConvNeXt1D(nn.Module):
    """``variant`` "1d" or "1dpp"; ``out_stages=True`` returns the four stage outputs, each
    through its own LayerNorm, instead of logits (the dense-prediction backbone form of
    semantic_segmentation/backbone/convnext.py:395-399,433-443).  ``backbone=True`` is that
    backbone in full: stage outputs, kernel sizes cropped per stage (:316-327), any input size,
    and the operators held in wrappers (parameter names ``...dwconv.conv.weight``), so that
    checkpoints converted by ``backbone_weights.convert_to_backbone_state_dict`` load."""

    def __init__(self, in_chans=3, num_classes=1000, depths=(3, 3, 9, 3), dims=(96, 192, 384, 768),
                 drop_path_rate=0.0, layer_scale_init_value=1e-6, head_init_scale=1.0, variant="1d",
                 N=8, stem_dim1=64, arbitrary_size=False, out_stages=False, backbone=False):
        super().__init__()
        if variant not in _VARIANTS:
            raise ValueError("variant must be '1d' or '1dpp'")
        block_ks, stem_k = _VARIANTS[variant]
        stage_ks = _BACKBONE_BLOCK_SIZES[variant] if backbone else (block_ks,) * 4
        out_stages = out_stages or backbone
        self.out_stages = out_stages
        self.downsample_layers = nn.ModuleList(
            [Stem1D(in_chans, stem_dim1, dims[0], stem_k, arbitrary_size, wrapped=backbone)])
        for i in range(3):
            self.downsample_layers.append(nn.Sequential(
                ChannelsFirstLayerNorm(dims[i]), nn.Conv2d(dims[i], dims[i + 1], kernel_size=2, stride=2)))
        rates = torch.linspace(0, drop_path_rate, sum(depths)).tolist()
        self.stages = nn.ModuleList()
        done = 0
        for i, depth in enumerate(depths):
            self.stages.append(nn.Sequential(*[
                Block(dims[i], stage_ks[i], variant == "1dpp", rates[done + j],
                      layer_scale_init_value, _odd_layer_offset(j), N, arbitrary_size,
                      wrapped=backbone) for j in range(depth)]))
            done += depth
        if out_stages:
            for i in range(4):
                self.add_module("norm%d" % i, ChannelsFirstLayerNorm(dims[i]))
        else:
            self.norm = nn.LayerNorm(dims[-1], eps=1e-6)
            self.head = nn.Linear(dims[-1], num_classes)
        self.apply(self._init)
        if not out_stages:
            with torch.no_grad():
                self.head.weight.mul_(head_init_scale)
                self.head.bias.mul_(head_init_scale)

    @staticmethod
    def _init(m):
        # models/convnext.py:592-596: truncated normal(0.02) weights, zero biases, for every
        # Conv2d (the oriented convs included) and Linear
        if isinstance(m, (nn.Conv2d, nn.Linear)):
            nn.init.trunc_normal_(m.weight, std=0.02)
            if m.bias is not None:
                nn.init.zeros_(m.bias)

    def forward(self, x):
        outs = []
        for i in range(4):
            x = self.stages[i](self.downsample_layers[i](x))
            if self.out_stages:
                outs.append(getattr(self, "norm%d" % i)(x))
        if self.out_stages:
            return outs
        return self.head(self.norm(x.mean((-2, -1))))


def convnext_tiny_1d(variant="1d", **kw):
    return ConvNeXt1D(depths=(3, 3, 9, 3), dims=(96, 192, 384, 768), variant=variant, **kw)


def convnext_base_1d(variant="1d", **kw):
    return ConvNeXt1D(depths=(3, 3, 27, 3), dims=(128, 256, 512, 1024), variant=variant, **kw)
