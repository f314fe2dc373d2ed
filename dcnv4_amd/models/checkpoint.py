"""State-dict schema of the released FlashInternImage classification checkpoints, and a checker / loader
built on it.

The schema is written down from the reference's module definitions, independently of the model classes in
this package (classification/models/flash_intern_image.py: build_norm_layer :34-55, StemLayer :235-268,
DownsampleLayer :271-304, MLPLayer :307-345, InternImageLayer :348-440, InternImageBlock :443-537,
FlashInternImage :540-700; DCNv4_op/DCNv4/modules/dcnv4.py:67-93 for the operator's own parameters), so
comparing it with ``model.state_dict()`` checks both.  Checkpoints are the files the reference's README lists
(README.md:29-32, ``flash_intern_image_{t,s,b}_1k_224.pth``, ``flash_internimage_l_22kto1k_384.pth``): a dict
with the weights under ``"model"``.
"""
import math
from collections import OrderedDict

import torch

from .flash_intern_image import _VARIANTS


def _bn(prefix, dim):
    return [(f"{prefix}.weight", (dim,)), (f"{prefix}.bias", (dim,)), (f"{prefix}.running_mean", (dim,)),
            (f"{prefix}.running_var", (dim,)), (f"{prefix}.num_batches_tracked", ())]


def _ln(prefix, dim):
    return [(f"{prefix}.weight", (dim,)), (f"{prefix}.bias", (dim,))]


def _linear(prefix, out_f, in_f, bias=True):
    return [(f"{prefix}.weight", (out_f, in_f))] + ([(f"{prefix}.bias", (out_f,))] if bias else [])


def offset_mask_features(group, kernel_size=3, remove_center=False):
    """Out-features of a DCNv4 block's ``offset_mask`` projection: 3 numbers per sampling point and group,
    padded up to a multiple of 8 (DCNv4_op/DCNv4/modules/dcnv4.py:82)."""
    k = group * (kernel_size * kernel_size - int(remove_center))
    return int(math.ceil(k * 3 / 8) * 8)


def reference_schema(variant="b", num_classes=1000, mlp_ratio=4.0, cls_scale=1.5):
    """OrderedDict key -> shape of the reference's FlashInternImage-T/S/B/L state dict."""
    cfg = _VARIANTS[variant.lower()]
    C0, depths, groups = cfg["channels"], cfg["depths"], cfg["groups"]
    post_norm, layer_scale = cfg.get("post_norm", False), cfg.get("layer_scale") is not None
    dw, out_bias, fc2_bias = cfg.get("dw_kernel_size"), cfg.get("dcn_output_bias", False), cfg.get("mlp_fc2_bias", False)
    items = []
    # stem: conv 3x3 s2 -> BN (channels_first in and out: child 0) -> GELU -> conv 3x3 s2 -> BN (child 0, then to channels_last)
    items += [("patch_embed.conv1.weight", (C0 // 2, 3, 3, 3)), ("patch_embed.conv1.bias", (C0 // 2,))]
    items += _bn("patch_embed.norm1.0", C0 // 2)
    items += [("patch_embed.conv2.weight", (C0, C0 // 2, 3, 3)), ("patch_embed.conv2.bias", (C0,))]
    items += _bn("patch_embed.norm2.0", C0)
    for i, (depth, g) in enumerate(zip(depths, groups)):
        C = C0 * 2 ** i
        hidden = int(C * mlp_ratio)
        for j in range(depth):
            p = f"levels.{i}.blocks.{j}"
            if layer_scale:                                                    # a module's own parameters precede its children's
                items += [(f"{p}.gamma1", (C,)), (f"{p}.gamma2", (C,))]
            items += _ln(f"{p}.norm1.0", C)                                    # LN on channels_last: child 0
            if dw is not None:
                items += [(f"{p}.dcn.offset_mask_dw.weight", (C, 1, dw, dw)), (f"{p}.dcn.offset_mask_dw.bias", (C,))]
            items += _linear(f"{p}.dcn.offset_mask", offset_mask_features(g), C)
            items += _linear(f"{p}.dcn.value_proj", C, C)
            items += _linear(f"{p}.dcn.output_proj", C, C, bias=out_bias)
            items += _ln(f"{p}.norm2.0", C)
            items += _linear(f"{p}.mlp.fc1", hidden, C)
            items += _linear(f"{p}.mlp.fc2", C, hidden, bias=fc2_bias)
        if not post_norm:
            items += _ln(f"levels.{i}.norm.0", C)
        if i < len(depths) - 1:
            items += [(f"levels.{i}.downsample.conv.weight", (2 * C, C, 3, 3))]
            items += _ln(f"levels.{i}.downsample.norm.1", 2 * C)               # channels_first in: child 0 is the permute
    F = C0 * 2 ** (len(depths) - 1)
    head = int(F * cls_scale)
    items += [("conv_head.0.weight", (head, F, 1, 1))]
    items += _bn("conv_head.1.0", head)
    items += _linear("head", num_classes, head)
    return OrderedDict(items)


def check_state_dict(state_dict, schema):
    """Compares a state dict with a schema.  Returns a list of human-readable problems (empty = compatible)."""
    problems = []
    for key, shape in schema.items():
        if key not in state_dict:
            problems.append(f"missing key {key} {tuple(shape)}")
            continue
        got = tuple(state_dict[key].shape)
        if got != tuple(shape):
            hint = ""
            if key.endswith("dcn.offset_mask.weight") or key.endswith("dcn.offset_mask.bias"):
                hint = " (the projection's out-features are 3 per sampling point and group, padded up to a multiple of 8)"
            problems.append(f"shape of {key}: checkpoint {got}, model {tuple(shape)}{hint}")
    for key in state_dict:
        if key not in schema:
            problems.append(f"unexpected key {key} {tuple(state_dict[key].shape)}")
    return problems


def unwrap_checkpoint(obj):
    """The weights of a checkpoint file's content: the reference saves {"model": state_dict, ...}
    (classification/utils.py save_checkpoint), mm* trainers {"state_dict": ...} with a ``backbone.`` prefix,
    DistributedDataParallel adds ``module.``."""
    for k in ("model", "state_dict", "model_ema"):
        if isinstance(obj, dict) and k in obj and isinstance(obj[k], dict):
            obj = obj[k]
            break
    out = OrderedDict()
    for key, value in obj.items():
        for prefix in ("module.", "backbone."):
            if key.startswith(prefix):
                key = key[len(prefix):]
        out[key] = value
    return out


def load_checkpoint(model, path, strict=True):
    """Loads a released checkpoint into ``model`` after checking it against the model's own state dict.
    The file is read with ``weights_only=True`` (nothing in it is executed).  Returns the list of problems
    (raises RuntimeError when ``strict`` and the list is not empty)."""
    state = unwrap_checkpoint(torch.load(path, map_location="cpu", weights_only=True))
    schema = OrderedDict((k, tuple(v.shape)) for k, v in model.state_dict().items())
    problems = check_state_dict(state, schema)
    if problems and strict:
        raise RuntimeError("checkpoint does not fit the model:\n  " + "\n  ".join(problems[:20]))
    model.load_state_dict(state, strict=strict)
    return problems
