"""Seeded synthetic inputs shared by the oracle tests, the GPU parity tests and the benchmark.

Recipes follow the distributions the reference's manual scripts use
(DCNv4_op/scripts/test_dcnv4_bwd.py:104-126, test_flash_deform_attn.py:104-111): value and
modulation normal, offsets uniform in pixels, attention locations uniform in [0,1].
Everything is generated on the CPU in fp32 from one torch.Generator so that the CPU oracle and
the GPU kernels see identical bits after the same dtype cast.
"""
import math

import torch


def dcn_out_hw(H, W, kh, kw, sh, sw, ph, pw, dh, dw):
    return ((H + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1,
            (W + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1)


def make_dcnv4_inputs(B, H, W, G, D, kh=3, kw=3, sh=1, sw=1, ph=1, pw=1, dh=1, dw=1,
                      remove_center=0, offset_range=2.0, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    K = kh * kw - int(bool(remove_center))
    Ho, Wo = dcn_out_hw(H, W, kh, kw, sh, sw, ph, pw, dh, dw)
    value = torch.randn(B, H, W, G * D, generator=g)
    offset = (torch.rand(B, Ho, Wo, G, K * 2, generator=g) * 2 - 1) * offset_range
    mask = torch.randn(B, Ho, Wo, G, K, generator=g)
    om = torch.cat([offset, mask], -1).reshape(B, Ho, Wo, G * K * 3)
    P_pad = int(math.ceil(G * K * 3 / 8) * 8)
    packed = torch.zeros(B, Ho, Wo, P_pad)
    packed[..., : G * K * 3] = om
    grad_out = torch.randn(B, Ho, Wo, G * D, generator=g)
    return value.to(dtype), packed.to(dtype), grad_out.to(dtype)


def level_start_index(shapes):
    starts, s = [], 0
    for h, w in shapes:
        starts.append(s)
        s += h * w
    return starts, s


def make_fda_inputs(B, shapes, G, D, K, Q=None, seed=0, dtype=torch.float32, loc_lo=0.0, loc_hi=1.0):
    g = torch.Generator().manual_seed(seed)
    starts, N = level_start_index(shapes)
    L = len(shapes)
    Q = N if Q is None else Q
    value = torch.randn(B, N, G, D, generator=g)
    loc = torch.rand(B, Q, G, L * K * 2, generator=g) * (loc_hi - loc_lo) + loc_lo
    logits = torch.randn(B, Q, G, L * K, generator=g)
    sla = torch.cat([loc, logits], -1)
    grad_out = torch.randn(B, Q, G * D, generator=g)
    return (value.to(dtype), torch.tensor(shapes, dtype=torch.int64),
            torch.tensor(starts, dtype=torch.int64), sla.to(dtype), grad_out.to(dtype))
