"""TEST INFRASTRUCTURE ONLY: torch ``grid_sample`` formulation of the two operators.

An independent second statement of the same mathematics as oracle/sampling_oracle.c:
the operators are written as ``F.grid_sample(bilinear, zeros, align_corners=False)``
on normalised coordinates, so autograd supplies every gradient.  It serves two
purposes: it pins the C oracle (two formulations that only agree if both index
maps are right) and it is the pure-PyTorch CPU baseline the benchmark times.

``dcnv4_core_torch`` follows the semantics of the reference's
classification/ops_dcnv3/functions/dcnv3_func.py:109-220 (reference points :109-137,
dilation grid with x-major point order :140-162, centre removal :165-170, core
:172-220) with two differences that DCNv4 makes: offsets and the un-normalised
modulation come packed in one ``offset_mask`` tensor
(DCNv4_op/src/cuda/dcnv4_im2col_cuda.cuh:163-171,220-224), and the H / W paddings are
applied to the axes they are named after (the reference core swaps them in its
``F.pad`` call at :183-185, which is only harmless when pad_h == pad_w).

``msda_core_torch`` is the textbook Deformable-DETR multi-scale core that the
reference's scripts import as ``ms_deform_attn_core_pytorch``
(DCNv4_op/scripts/test_flash_deform_attn_backward.py:113-116) but do not ship, fed
from the packed ``sampling_loc_attn`` layout of
DCNv4_op/src/cuda/flash_deform_im2col_cuda.cuh:145-149.
"""
import torch
import torch.nn.functional as F


def unpack_offset_mask(offset_mask, group, points):
    """(B,Ho,Wo,P_pad) -> offsets (B,Ho,Wo,G,K,2) as (x,y) pairs, mask (B,Ho,Wo,G,K)."""
    B, Ho, Wo, _ = offset_mask.shape
    body = offset_mask[..., : group * points * 3].reshape(B, Ho, Wo, group, points * 3)
    return body[..., : points * 2].reshape(B, Ho, Wo, group, points, 2), body[..., points * 2:]


def pack_offset_mask(offset, mask):
    """Inverse of :func:`unpack_offset_mask`; pads the last dim up to a multiple of 8 with zeros
    (DCNv4_op/DCNv4/modules/dcnv4.py:82, DCNv4_op/scripts/test_dcnv4.py:84,104-107)."""
    B, Ho, Wo, G, K, _ = offset.shape
    om = torch.cat([offset.reshape(B, Ho, Wo, G, K * 2), mask], dim=-1).reshape(B, Ho, Wo, G * K * 3)
    pad = (-om.shape[-1]) % 8
    return F.pad(om, (0, pad)) if pad else om


def dcnv4_core_torch(value, offset_mask, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w,
                     dilation_h, dilation_w, group, group_channels, offset_scale,
                     remove_center=0, softmax=False):
    B, H, W, C = value.shape
    _, Ho, Wo, _ = offset_mask.shape
    dt, dev = value.dtype, value.device
    Hp, Wp = H + 2 * pad_h, W + 2 * pad_w
    padded = F.pad(value, (0, 0, pad_w, pad_w, pad_h, pad_h))

    # kernel taps, x index outer / y index inner
    taps = [(i, j) for i in range(kernel_w) for j in range(kernel_h)
            if not (remove_center and i == kernel_w // 2 and j == kernel_h // 2)]
    K = len(taps)
    tap_x = torch.tensor([i * dilation_w - (dilation_w * (kernel_w - 1)) // 2 for i, _ in taps], dtype=dt, device=dev)
    tap_y = torch.tensor([j * dilation_h - (dilation_h * (kernel_h - 1)) // 2 for _, j in taps], dtype=dt, device=dev)

    offset, mask = unpack_offset_mask(offset_mask, group, K)
    if softmax:
        mask = mask.softmax(-1)
    ref_x = (dilation_w * (kernel_w - 1)) // 2 + 0.5 + torch.arange(Wo, dtype=dt, device=dev) * stride_w
    ref_y = (dilation_h * (kernel_h - 1)) // 2 + 0.5 + torch.arange(Ho, dtype=dt, device=dev) * stride_h
    # padded-image pixel-centre coordinates, then normalise to [-1, 1]
    px = ref_x.view(1, 1, Wo, 1, 1) + (tap_x.view(1, 1, 1, 1, K) + offset[..., 0]) * offset_scale
    py = ref_y.view(1, Ho, 1, 1, 1) + (tap_y.view(1, 1, 1, 1, K) + offset[..., 1]) * offset_scale
    grid = torch.stack([2 * px / Wp - 1, 2 * py / Hp - 1], dim=-1)          # B,Ho,Wo,G,K,2
    grid = grid.permute(0, 3, 1, 2, 4, 5).reshape(B * group, Ho * Wo, K, 2)
    img = padded.reshape(B, Hp * Wp, group, group_channels).permute(0, 2, 3, 1).reshape(
        B * group, group_channels, Hp, Wp)
    sampled = F.grid_sample(img, grid, mode="bilinear", padding_mode="zeros", align_corners=False)
    m = mask.permute(0, 3, 1, 2, 4).reshape(B * group, 1, Ho * Wo, K)
    out = (sampled * m).sum(-1).reshape(B, group * group_channels, Ho * Wo)
    return out.transpose(1, 2).reshape(B, Ho, Wo, C).contiguous()


def msda_core_torch(value, spatial_shapes, level_start_index, sampling_loc_attn, K):
    B, N, G, D = value.shape
    L = len(spatial_shapes)
    Q = sampling_loc_attn.shape[1]
    LK = L * K
    loc = sampling_loc_attn[..., : 2 * LK].reshape(B, Q, G, L, K, 2)
    attn = sampling_loc_attn[..., 2 * LK:].softmax(-1).reshape(B, Q, G, L, K)
    out = 0
    for l in range(L):
        Hl, Wl = int(spatial_shapes[l][0]), int(spatial_shapes[l][1])
        s = int(level_start_index[l])
        img = value[:, s:s + Hl * Wl].permute(0, 2, 3, 1).reshape(B * G, D, Hl, Wl)
        grid = (2 * loc[:, :, :, l] - 1).permute(0, 2, 1, 3, 4).reshape(B * G, Q, K, 2)
        sampled = F.grid_sample(img, grid, mode="bilinear", padding_mode="zeros", align_corners=False)
        w = attn[:, :, :, l].permute(0, 2, 1, 3).reshape(B * G, 1, Q, K)
        out = out + (sampled * w).sum(-1)
    return out.reshape(B, G * D, Q).transpose(1, 2).contiguous()
