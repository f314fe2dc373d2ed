"""FlashInternImage classifier: the in-tree caller of the DCNv4 operator, used by the end-to-end benchmark.

Own restatement of the reference model's architecture for the T/S/B/L classification variants
(classification/models/flash_intern_image.py:235-304 stem / downsample, :307-440 layer, :443-537 block,
:540-792 network; hyper-parameters classification/configs/flash_intern_image_{t,s,b,l}_*.yaml).  Module
nesting and attribute names follow the reference so its checkpoints' state-dict keys line up
(`patch_embed.conv1`, `levels.N.blocks.M.dcn.offset_mask`, `levels.N.downsample.norm.1`, `conv_head.1.0`, ...).
Not carried over: the InternImage-H/G extras (CLIP projector, attention pooling, level-2 post norms) that no
FlashInternImage config enables.
"""
import torch
from torch import nn

from ..functions import layer_norm_residual
from ..modules import DCNv4


class _ToChannelsFirst(nn.Module):
    def forward(self, x):
        return x.permute(0, 3, 1, 2)


class _ToChannelsLast(nn.Module):
    def forward(self, x):
        return x.permute(0, 2, 3, 1)


def _norm(dim, kind, in_format="channels_last", out_format="channels_last", eps=1e-6):
    """nn.Sequential whose child indices match the reference's build_norm_layer (:34-55)."""
    layers = []
    if kind == "BN":
        if in_format == "channels_last":
            layers.append(_ToChannelsFirst())
        layers.append(nn.BatchNorm2d(dim))
        if out_format == "channels_last":
            layers.append(_ToChannelsLast())
    elif kind == "LN":
        if in_format == "channels_first":
            layers.append(_ToChannelsLast())
        layers.append(nn.LayerNorm(dim, eps=eps))
        if out_format == "channels_first":
            layers.append(_ToChannelsFirst())
    else:
        raise NotImplementedError(f"norm layer {kind}")
    return nn.Sequential(*layers)


class DropPath(nn.Module):
    """Stochastic depth per sample; identity in eval mode."""

    def __init__(self, p=0.0):
        super().__init__()
        self.p = float(p)

    def forward(self, x):
        if self.p == 0.0 or not self.training:
            return x
        keep = 1.0 - self.p
        mask = x.new_empty((x.shape[0],) + (1,) * (x.dim() - 1)).bernoulli_(keep)
        return x * mask / keep


class StemLayer(nn.Module):
    def __init__(self, in_chans=3, out_chans=96, norm_layer="BN"):
        super().__init__()
        self.conv1 = nn.Conv2d(in_chans, out_chans // 2, kernel_size=3, stride=2, padding=1)
        self.norm1 = _norm(out_chans // 2, norm_layer, "channels_first", "channels_first")
        self.act = nn.GELU()
        self.conv2 = nn.Conv2d(out_chans // 2, out_chans, kernel_size=3, stride=2, padding=1)
        self.norm2 = _norm(out_chans, norm_layer, "channels_first", "channels_last")

    def forward(self, x):
        # channels-last memory from the first convolution on: the NHWC view the blocks work on is then dense, so
        # every kernel after the stem sees contiguous rows of channels (no strided elementwise kernels, no copies)
        x = x.contiguous(memory_format=torch.channels_last)
        return self.norm2(self.conv2(self.act(self.norm1(self.conv1(x))))).contiguous()


class DownsampleLayer(nn.Module):
    def __init__(self, channels, norm_layer="LN"):
        super().__init__()
        self.conv = nn.Conv2d(channels, 2 * channels, kernel_size=3, stride=2, padding=1, bias=False)
        self.norm = _norm(2 * channels, norm_layer, "channels_first", "channels_first")

    def forward(self, x, shape):
        H, W = shape
        N, _, C = x.shape
        x = self.norm(self.conv(x.view(N, H, W, C).permute(0, 3, 1, 2)))
        H, W = x.size(2), x.size(3)
        return x.flatten(2).permute(0, 2, 1), (H, W)


class MLPLayer(nn.Module):
    def __init__(self, in_features, hidden_features, mlp_fc2_bias=False, drop=0.0):
        super().__init__()
        self.fc1 = nn.Linear(in_features, hidden_features, bias=True)
        self.act = nn.GELU()
        self.fc2 = nn.Linear(hidden_features, in_features, bias=mlp_fc2_bias)
        self.drop = nn.Dropout(drop)

    def forward(self, x, shape=None):
        return self.drop(self.fc2(self.drop(self.act(self.fc1(x)))))


class InternImageLayer(nn.Module):
    def __init__(self, channels, groups, mlp_ratio=4.0, drop=0.0, drop_path=0.0, post_norm=False, layer_scale=None,
                 offset_scale=1.0, dcn_output_bias=False, mlp_fc2_bias=False, dw_kernel_size=None):
        super().__init__()
        self.post_norm = post_norm
        self.norm1 = _norm(channels, "LN")
        self.dcn = DCNv4(channels=channels, group=groups, offset_scale=offset_scale, dw_kernel_size=dw_kernel_size,
                         output_bias=dcn_output_bias)
        self.drop_path = DropPath(drop_path) if drop_path > 0.0 else nn.Identity()
        self.norm2 = _norm(channels, "LN")
        self.mlp = MLPLayer(channels, int(channels * mlp_ratio), mlp_fc2_bias=mlp_fc2_bias, drop=drop)
        self.layer_scale = layer_scale is not None
        if self.layer_scale:
            self.gamma1 = nn.Parameter(layer_scale * torch.ones(channels))
            self.gamma2 = nn.Parameter(layer_scale * torch.ones(channels))

    def _scaled_norm(self, norm, gamma, y, residual):
        """residual + drop_path(gamma * norm(y)); one kernel when stochastic depth is idle (always in eval mode)."""
        ln = norm[0] if len(norm) == 1 and isinstance(norm[0], nn.LayerNorm) else None
        if ln is None:
            return residual + self.drop_path((gamma * norm(y)) if gamma is not None else norm(y))
        if isinstance(self.drop_path, nn.Identity) or not self.training:
            return layer_norm_residual(y, ln, gamma, residual)
        return residual + self.drop_path(layer_norm_residual(y, ln, gamma))

    def forward(self, x, shape):
        g1, g2 = (self.gamma1, self.gamma2) if self.layer_scale else (None, None)
        if self.post_norm:
            x = self._scaled_norm(self.norm1, g1, self.dcn(x, shape), x)
            x = self._scaled_norm(self.norm2, g2, self.mlp(x, shape), x)
        else:
            y = self.dcn(layer_norm_residual(x, self.norm1[0]), shape)
            x = x + self.drop_path(y if g1 is None else g1 * y)
            y = self.mlp(layer_norm_residual(x, self.norm2[0]), shape)
            x = x + self.drop_path(y if g2 is None else g2 * y)
        return x


class InternImageBlock(nn.Module):
    def __init__(self, channels, depth, groups, downsample=True, drop_path=0.0, post_norm=False, norm_layer="LN", **layer_kw):
        super().__init__()
        self.post_norm = post_norm
        self.blocks = nn.ModuleList([
            InternImageLayer(channels, groups, drop_path=drop_path[i] if isinstance(drop_path, list) else drop_path,
                             post_norm=post_norm, **layer_kw) for i in range(depth)])
        if not post_norm:
            self.norm = _norm(channels, "LN")
        self.downsample = DownsampleLayer(channels, norm_layer) if downsample else None

    def forward(self, x, shape, return_wo_downsample=False):
        for blk in self.blocks:
            x = blk(x, shape)
        if not self.post_norm:
            x = self.norm(x)
        before = x
        if self.downsample is not None:
            x, shape = self.downsample(x, shape)
        return (x, before, shape) if return_wo_downsample else (x, shape)


class FlashInternImage(nn.Module):
    def __init__(self, core_op="DCNv4", channels=64, depths=(3, 4, 18, 5), groups=(3, 6, 12, 24), num_classes=1000,
                 mlp_ratio=4.0, drop_rate=0.0, drop_path_rate=0.2, drop_path_type="linear", norm_layer="LN",
                 layer_scale=None, offset_scale=0.5, post_norm=False, cls_scale=1.5, mlp_fc2_bias=False,
                 dcn_output_bias=False, dw_kernel_size=None, **kwargs):
        super().__init__()
        if core_op != "DCNv4":
            raise NotImplementedError(f"core_op {core_op}: only DCNv4 is available")
        unsupported = {k for k in ("use_clip_projector", "level2_post_norm", "res_post_norm", "center_feature_scale")
                       if kwargs.get(k)}
        if unsupported:
            raise NotImplementedError(f"InternImage-H/G options are not built: {sorted(unsupported)}")
        self.num_classes = num_classes
        self.depths = list(depths)
        self.num_levels = len(depths)
        self.channels = channels
        self.num_features = int(channels * 2 ** (self.num_levels - 1))

        self.patch_embed = StemLayer(3, channels, "BN")
        self.pos_drop = nn.Dropout(p=drop_rate)
        dpr = [x.item() for x in torch.linspace(0, drop_path_rate, sum(depths))]
        if drop_path_type == "uniform":
            dpr = [drop_path_rate] * len(dpr)
        self.levels = nn.ModuleList()
        for i in range(self.num_levels):
            self.levels.append(InternImageBlock(
                int(channels * 2 ** i), depths[i], groups[i], downsample=i < self.num_levels - 1,
                drop_path=dpr[sum(depths[:i]):sum(depths[:i + 1])], post_norm=post_norm, norm_layer=norm_layer,
                mlp_ratio=mlp_ratio, drop=drop_rate, layer_scale=layer_scale, offset_scale=offset_scale,
                dcn_output_bias=dcn_output_bias, mlp_fc2_bias=mlp_fc2_bias, dw_kernel_size=dw_kernel_size))
        head_dim = int(self.num_features * cls_scale)
        self.conv_head = nn.Sequential(nn.Conv2d(self.num_features, head_dim, kernel_size=1, bias=False),
                                       _norm(head_dim, "BN", "channels_first", "channels_first"), nn.GELU())
        self.head = nn.Linear(head_dim, num_classes) if num_classes > 0 else nn.Identity()
        self.avgpool = nn.AdaptiveAvgPool2d((1, 1))
        self.apply(self._init_weights)
        for m in self.modules():
            if isinstance(m, DCNv4):
                m._reset_parameters()

    @staticmethod
    def _init_weights(m):
        if isinstance(m, nn.Linear):
            nn.init.trunc_normal_(m.weight, std=0.02)
            if m.bias is not None:
                nn.init.constant_(m.bias, 0)
        elif isinstance(m, nn.LayerNorm):
            nn.init.constant_(m.bias, 0)
            nn.init.constant_(m.weight, 1.0)

    def forward_features_seq_out(self, x):
        """Per-level feature maps (N, C_l, H_l, W_l) before each downsample, as the dense-prediction backbones use."""
        x = self.patch_embed(x)
        N, H, W, C = x.shape
        x = x.view(N, H * W, C)
        shape, outs = (H, W), []
        for level in self.levels:
            h, w = shape
            x, before, shape = level(x, shape, return_wo_downsample=True)
            outs.append(before.reshape(N, h, w, -1).permute(0, 3, 1, 2))
        return outs

    def forward_features(self, x):
        x = self.patch_embed(x)
        N, H, W, C = x.shape
        x = self.pos_drop(x.view(N, H * W, C))
        shape = (H, W)
        for level in self.levels:
            x, shape = level(x, shape)
        h, w = shape
        x = self.conv_head(x.view(N, h, w, -1).permute(0, 3, 1, 2))
        return torch.flatten(self.avgpool(x), 1)

    def forward(self, x):
        return self.head(self.forward_features(x))


class FlashInternImageBackbone(FlashInternImage):
    """Dense-prediction backbone: the same stem and levels without the classification head; ``forward`` returns
    the NCHW feature map of every level in ``out_indices``, taken before that level's downsample, for inputs of
    any (non-square) size.  Follows detection/mmdet_custom/models/backbones/flash_intern_image.py:596-608,750-763
    (the segmentation backbone is the same code); checkpoint loading and layer-wise learning-rate tables belong to
    the mmdet/mmseg side and are not reproduced."""

    def __init__(self, out_indices=(0, 1, 2, 3), **kwargs):
        kwargs.setdefault("num_classes", 0)
        super().__init__(**kwargs)
        self.out_indices = tuple(out_indices)
        del self.conv_head, self.head, self.avgpool

    def forward_features(self, x):
        raise NotImplementedError("the backbone has no classification head; call forward()")

    def forward(self, x):
        x = self.patch_embed(x)
        N, H, W, C = x.shape
        x = x.view(N, H * W, C)
        shape, outs = (H, W), []
        for level_idx, level in enumerate(self.levels):
            h, w = shape
            x, before, shape = level(x, shape, return_wo_downsample=True)
            if level_idx in self.out_indices:
                outs.append(before.reshape(N, h, w, -1).permute(0, 3, 1, 2))
        return outs


# classification/configs/flash_intern_image_{t,s,b}_1k_224.yaml, flash_intern_image_l_22kto1k_384.yaml
_VARIANTS = {
    "t": dict(channels=64, depths=(4, 4, 18, 4), groups=(4, 8, 16, 32), offset_scale=1.0, drop_path_rate=0.1),
    "s": dict(channels=80, depths=(4, 4, 21, 4), groups=(5, 10, 20, 40), offset_scale=1.0, drop_path_rate=0.4,
              layer_scale=1e-5, post_norm=True, dw_kernel_size=3),
    "b": dict(channels=112, depths=(4, 4, 21, 4), groups=(7, 14, 28, 56), offset_scale=0.5, drop_path_rate=0.5,
              layer_scale=1e-5, post_norm=True, dw_kernel_size=3),
    "l": dict(channels=160, depths=(5, 5, 22, 5), groups=(10, 20, 40, 80), offset_scale=2.0, drop_path_rate=0.1,
              layer_scale=1e-5, post_norm=True, dw_kernel_size=3, dcn_output_bias=True, mlp_fc2_bias=True),
}


def flash_intern_image(variant="b", **overrides):
    """FlashInternImage-T/S/B/L with the reference configs' hyper-parameters (mlp_ratio 4, 1000 classes)."""
    cfg = dict(_VARIANTS[variant.lower()], mlp_ratio=4.0)
    cfg.update(overrides)
    return FlashInternImage(**cfg)
