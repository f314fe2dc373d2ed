"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle on identical bits.

Tolerances (stated by the task for this path): forward rtol 1e-4 / atol 1e-5 in fp32 and 1e-2 in
fp16; gradients 1e-3 relative in fp32 (atomic summation order differs run to run).  The oracle is
always fed the dtype-quantised inputs widened exactly to float64.
"""
import zlib

import numpy as np
import pytest
import torch

from tests import cabi
from tests.inputs import make_dcnv4_inputs, make_fda_inputs

pytestmark = pytest.mark.gpu

FWD_TOL = {torch.float32: (1e-4, 1e-5), torch.float16: (1e-2, 1e-3), torch.bfloat16: (2e-2, 2e-2)}
GRAD_TOL = {torch.float32: (1e-3, 1e-4), torch.float16: (1e-2, 1e-2), torch.bfloat16: (4e-2, 8e-2)}

# B, H, W, G, D, (kh, kw, sh, sw, ph, pw, dh, dw), remove_center, offset_scale, offset_range
DCN_CASES = {
    "cfg1_56x56_c64_g4": (2, 56, 56, 4, 16, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 2.0),
    "stage_28x28_c128_g8": (3, 28, 28, 8, 16, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 3.0),
    "stage_7x7_c512_g32": (5, 7, 7, 32, 16, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 3.0),
    "wide_g80": (1, 9, 11, 80, 16, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 4.0),
    "g7_c112_scale_half": (2, 14, 14, 7, 16, (3, 3, 1, 1, 1, 1, 1, 1), 0, 0.5, 3.0),
    "remove_center": (2, 12, 10, 4, 16, (3, 3, 1, 1, 1, 1, 1, 1), 1, 1.3, 2.5),
    "stride2": (2, 15, 17, 3, 16, (3, 3, 2, 2, 1, 1, 1, 1), 0, 2.0, 2.0),
    "dilation2_pad2": (1, 13, 12, 2, 32, (3, 3, 1, 1, 2, 2, 2, 2), 0, 1.0, 1.5),
    "kernel_1x3_mixed_pad": (1, 9, 8, 2, 8, (1, 3, 1, 1, 0, 1, 1, 1), 0, 0.7, 2.0),
    "kernel_5x5": (1, 10, 10, 2, 16, (5, 5, 1, 1, 2, 2, 1, 1), 0, 1.0, 2.0),
    "kernel_3x1_stride_2x1": (1, 10, 9, 2, 4, (3, 1, 2, 1, 2, 0, 2, 1), 0, 1.0, 2.0),
    "d1_scalar_lanes": (1, 6, 7, 5, 1, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 2.0),
    "d6_three_lane_cluster": (2, 6, 5, 3, 6, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 2.0),
    "d48_six_lane_cluster": (1, 8, 8, 2, 48, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 2.0),
    "d64": (1, 8, 9, 2, 64, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 2.0),
    # groups of 64 channels as in a third of the reference's tuned keys (DCNv4_op/DCNv4/functions/table.py:452-461), several tiles
    "d64_g4_20x18": (2, 20, 18, 4, 64, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 3.0),
    # four lanes of 32 channels per (cell, group) in the tiled grad_value kernel, the last one partly idle
    "d104_four_lanes_per_slot": (1, 9, 7, 2, 104, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 2.0),
    # the widest group the fp32 backward takes: 64 gather lanes, eight lanes of 32 channels per (cell, group)
    "d256_eight_lanes_per_slot": (1, 5, 6, 1, 256, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 2.0),
    # 49 taps: strips of a few pixels
    "kernel_7x7_g3": (1, 12, 11, 3, 16, (7, 7, 1, 1, 3, 3, 1, 1), 0, 1.0, 1.5),
    "far_offsets_mostly_outside": (1, 5, 5, 4, 16, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 9.0),
    "single_pixel": (1, 1, 1, 1, 16, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 1.0),
    # 32-wide grad_value tiles, one group per workgroup: a one-pixel remainder tile in both directions
    "edge_33x33_g2": (1, 33, 33, 2, 16, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 3.0),
    # ... a tile two rows high, whose corners above and below land outside the accumulators
    "wide_short_2x40_g3": (2, 2, 40, 3, 16, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 3.0),
    # ... and a tall image only 8 pixels wide (narrow tiles keep the general accumulation)
    "tall_narrow_40x8_g2": (1, 40, 8, 2, 16, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 3.0),
    # 16-wide tiles with four groups per workgroup and a last chunk of one group
    "g5_16x12": (2, 16, 12, 5, 16, (3, 3, 1, 1, 1, 1, 1, 1), 1, 1.0, 3.0),
}


def _dcn_inputs(case, dtype, seed=0):
    B, H, W, G, D, geom, rc, scale, rng = case
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, *geom, remove_center=rc, offset_range=rng, seed=seed, dtype=dtype)
    return v, om, go, (geom, G, D, scale, rc)


def _oracle_args(geom, G, D, scale, rc):
    return (*geom, G, D, scale, rc)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("name", list(DCN_CASES))
def test_dcnv4_forward_and_backward_match_oracle(oracle, name, dtype):
    v, om, go, (geom, G, D, scale, rc) = _dcn_inputs(DCN_CASES[name], dtype, seed=zlib.crc32(name.encode()) % 1000)
    print(f"case {name} dtype {dtype}", flush=True)
    want = oracle.dcnv4_forward(cabi.f64(v), cabi.f64(om), *_oracle_args(geom, G, D, scale, rc), coord_f32=True)
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *_oracle_args(geom, G, D, scale, rc), coord_f32=True)
    vd, omd, god = v.cuda(), om.cuda(), go.cuda()
    out = cabi.dcnv4_forward(vd, omd, geom, G, D, scale, rc)
    gv, gom = cabi.dcnv4_backward(vd, omd, god, geom, G, D, scale, rc)
    torch.cuda.synchronize()
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    cabi.assert_close(gv, wgv, *GRAD_TOL[dtype], what="grad_value")
    cabi.assert_close(gom, wgom, *GRAD_TOL[dtype], what="grad_offset_mask")
    used = G * 3 * (geom[0] * geom[1] - rc)
    assert (gom[..., used:] == 0).all(), "padded tail of grad_offset_mask must be exactly zero"


# The library picks between kernel families by shape; these launch options force the other branches:
# the global-memory gather kernels, (tiny reach) the per-point global fetches of the LDS-tiled
# gathers, and smaller grad_value tiles with several groups per workgroup.
KERNEL_PATHS = {
    "direct_gather": dict(gather="direct"),
    "reach1": dict(reach=1),
    "reach0": dict(reach=0),
    "reach9": dict(reach=9),
    "tile16": dict(tile=16),                                   # grad_value on 16x16 tiles, four groups each
    "tile8_reach1": dict(tile=8, reach=1),
    "gv512": dict(gv_threads=512),                             # grad_value workgroups of 512 / 1024 lanes
    "gv1024": dict(gv_threads=1024),
    "gather_tile4": dict(gather_tile=4),                       # smaller output tiles of the LDS-tiled gathers (more groups each)
    "gather_tile8": dict(gather_tile=8),
    "gather_tile8_reach2": dict(gather_tile=8, reach=2),
    "gather_tile4_gv512": dict(gather_tile=4, gv_threads=512),
    # images that are one grad_value tile: both backward kernels as one launch with two workgroup roles, or as two launches
    "dual_on": dict(dual="on", gv_threads=512),
    "dual_off": dict(dual="off"),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("path", list(KERNEL_PATHS))
@pytest.mark.parametrize("name", ["cfg1_56x56_c64_g4", "g7_c112_scale_half", "remove_center", "stride2", "dilation2_pad2",
                                  "kernel_5x5", "far_offsets_mostly_outside", "wide_g80", "d64_g4_20x18", "stage_7x7_c512_g32",
                                  "stage_28x28_c128_g8"])
def test_dcnv4_every_kernel_path_matches_oracle(oracle, name, path, dtype):
    from dcnv4_amd import ext
    v, om, go, (geom, G, D, scale, rc) = _dcn_inputs(DCN_CASES[name], dtype, seed=zlib.crc32((name + path).encode()) % 1000)
    print(f"case {name} path {path} dtype {dtype}", flush=True)
    args = _oracle_args(geom, G, D, scale, rc)
    want = oracle.dcnv4_forward(cabi.f64(v), cabi.f64(om), *args, coord_f32=True)
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *args, coord_f32=True)
    with ext.launch_options(**KERNEL_PATHS[path]):
        out = cabi.dcnv4_forward(v.cuda(), om.cuda(), geom, G, D, scale, rc)
        gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), geom, G, D, scale, rc)
    torch.cuda.synchronize()
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    cabi.assert_close(gv, wgv, *GRAD_TOL[dtype], what="grad_value")
    cabi.assert_close(gom, wgom, *GRAD_TOL[dtype], what="grad_offset_mask")
    used = G * 3 * (geom[0] * geom[1] - rc)
    assert (gom[..., used:] == 0).all(), "padded tail of grad_offset_mask must be exactly zero"


SOFTMAX_PATHS = {
    "library_choice": {},                       # the LDS-tiled gathers (their run-time-shape instantiations)
    "direct_gather": dict(gather="direct"),
    "reach0": dict(reach=0),                    # every sampling point through the tiled gathers' global-memory path
    "gather_tile4_reach1": dict(gather_tile=4, reach=1),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("path", list(SOFTMAX_PATHS))
@pytest.mark.parametrize("name", ["remove_center", "cfg1_56x56_c64_g4", "stride2", "dilation2_pad2", "kernel_5x5", "g5_16x12",
                                  "far_offsets_mostly_outside", "d64_g4_20x18", "stage_7x7_c512_g32"])
def test_dcnv4_softmax_flag_matches_oracle(oracle, name, path, dtype):
    """The reference's latent softmax over a group's modulation scalars (dcnv4_im2col_cuda.cuh:173-193,
    dcnv4_col2im_cuda.cuh:352-365), through both gather families."""
    from dcnv4_amd import ext
    v, om, go, (geom, G, D, scale, rc) = _dcn_inputs(DCN_CASES[name], dtype, seed=5)
    print(f"softmax case {name} path {path} dtype {dtype}", flush=True)
    args = _oracle_args(geom, G, D, scale, rc)
    want = oracle.dcnv4_forward(cabi.f64(v), cabi.f64(om), *args, softmax=True, coord_f32=True)
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *args, softmax=True, coord_f32=True)
    with ext.launch_options(**SOFTMAX_PATHS[path]):
        out = cabi.dcnv4_forward(v.cuda(), om.cuda(), geom, G, D, scale, rc, softmax=1)
        gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), geom, G, D, scale, rc, softmax=1)
    torch.cuda.synchronize()
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    cabi.assert_close(gv, wgv, *GRAD_TOL[dtype], what="grad_value")
    cabi.assert_close(gom, wgom, *GRAD_TOL[dtype], what="grad_offset_mask")
    used = G * 3 * (geom[0] * geom[1] - rc)
    assert (gom[..., used:] == 0).all(), "padded tail of grad_offset_mask must be exactly zero"


def test_dcnv4_unpadded_offset_mask_rows(oracle):
    # P_pad = G*K*3 = 54, not a multiple of 8: rows are not 16-byte aligned, scalar staging path
    B, H, W, G, D = 2, 6, 7, 2, 16
    geom = (3, 3, 1, 1, 1, 1, 1, 1)
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, seed=3, dtype=torch.float16)
    om = om[..., :54].contiguous()
    args = (*geom, G, D, 1.0, 0)
    want = oracle.dcnv4_forward(cabi.f64(v), cabi.f64(om), *args, coord_f32=True)
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *args, coord_f32=True)
    out = cabi.dcnv4_forward(v.cuda(), om.cuda(), geom, G, D, 1.0)
    gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), geom, G, D, 1.0)
    cabi.assert_close(out, want, *FWD_TOL[torch.float16], what="output")
    cabi.assert_close(gv, wgv, *GRAD_TOL[torch.float16], what="grad_value")
    cabi.assert_close(gom, wgom, *GRAD_TOL[torch.float16], what="grad_offset_mask")


@pytest.mark.parametrize("d_stride,block_thread", [(1, 64), (2, 128), (4, 512), (8, 1024), (16, 32)])
def test_dcnv4_launch_hints_do_not_change_results(oracle, d_stride, block_thread):
    v, om, go, (geom, G, D, scale, rc) = _dcn_inputs(DCN_CASES["g7_c112_scale_half"], torch.float16, seed=9)
    args = _oracle_args(geom, G, D, scale, rc)
    want = oracle.dcnv4_forward(cabi.f64(v), cabi.f64(om), *args, coord_f32=True)
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *args, coord_f32=True)
    out = cabi.dcnv4_forward(v.cuda(), om.cuda(), geom, G, D, scale, rc, d_stride=d_stride, block_thread=block_thread)
    gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), geom, G, D, scale, rc, d_stride=d_stride,
                                  block_thread=block_thread)
    cabi.assert_close(out, want, *FWD_TOL[torch.float16], what="output")
    cabi.assert_close(gv, wgv, *GRAD_TOL[torch.float16], what="grad_value")
    cabi.assert_close(gom, wgom, *GRAD_TOL[torch.float16], what="grad_offset_mask")


def test_dcnv4_zero_offsets_unit_mask_is_box_sum_on_gpu():
    B, H, W, G, D, K = 2, 20, 24, 4, 16, 9
    v, om, _ = make_dcnv4_inputs(B, H, W, G, D, seed=1)
    om.zero_()
    body = om[..., : G * K * 3].reshape(B, H, W, G, K * 3)
    body[..., 2 * K:] = 1.0
    out = cabi.dcnv4_forward(v.cuda(), om.cuda(), (3, 3, 1, 1, 1, 1, 1, 1), G, D, 1.0)
    box = torch.nn.functional.avg_pool2d(v.permute(0, 3, 1, 2).double(), 3, 1, 1) * 9
    cabi.assert_close(out, box.permute(0, 2, 3, 1).numpy(), 1e-5, 1e-5, what="box sum")


def test_dcnv4_infinite_and_nan_offsets_are_dropped_not_propagated():
    B, H, W, G, D, K = 1, 6, 6, 1, 16, 9
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, seed=2)
    om[..., 0] = float("inf")
    om[..., 3] = float("nan")
    om[..., 4] = -1e30
    out = cabi.dcnv4_forward(v.cuda(), om.cuda(), (3, 3, 1, 1, 1, 1, 1, 1), G, D, 1.0)
    gv, _ = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), (3, 3, 1, 1, 1, 1, 1, 1), G, D, 1.0)
    assert torch.isfinite(out).all() and torch.isfinite(gv).all()


# B, shapes, G, D, K, Q, (loc_lo, loc_hi)
FDA_CASES = {
    "detr_small_4lvl_k4": (2, [(16, 16), (8, 8), (4, 4), (2, 2)], 8, 32, 4, None, (0.0, 1.0)),
    "k8_one_level": (1, [(20, 30)], 8, 32, 8, 77, (-0.1, 1.1)),
    "five_levels": (1, [(8, 12), (6, 6), (4, 5), (2, 2), (1, 3)], 2, 16, 4, 50, (-0.3, 1.3)),
    "k3_generic_points": (2, [(7, 5), (3, 4)], 3, 8, 3, 19, (0.0, 1.0)),
    "d6_heads5": (1, [(6, 6), (3, 3)], 5, 6, 4, 11, (0.0, 1.0)),
    "d64_two_levels": (1, [(9, 9), (5, 5)], 4, 64, 4, 33, (0.0, 1.0)),
    "one_query": (1, [(4, 4)], 1, 32, 4, 1, (0.0, 1.0)),
    # a decoder's few queries against an encoder's pyramid: with fp32 tensors the backward takes the atomic scatter by itself
    "decoder_few_queries": (2, [(20, 30), (10, 15)], 4, 32, 4, 12, (0.0, 1.0)),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("name", list(FDA_CASES))
def test_flash_deform_attn_forward_and_backward_match_oracle(oracle, name, dtype):
    B, shapes, G, D, K, Q, (lo, hi) = FDA_CASES[name]
    print(f"case {name} dtype {dtype}", flush=True)
    v, shp, st, sla, go = make_fda_inputs(B, shapes, G, D, K, Q, seed=zlib.crc32(name.encode()) % 1000, dtype=dtype, loc_lo=lo, loc_hi=hi)
    want = oracle.flash_deform_attn_forward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), K, coord_f32=True)
    wgv, wgs = oracle.flash_deform_attn_backward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), cabi.f64(go), K, coord_f32=True)
    vd, sd, gd, shd, std = v.cuda(), sla.cuda(), go.cuda(), shp.cuda(), st.cuda()
    out = cabi.fda_forward(vd, shd, std, sd, K)
    gv, gs = cabi.fda_backward(vd, shd, std, sd, gd, K)
    torch.cuda.synchronize()
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    cabi.assert_close(gv, wgv, *GRAD_TOL[dtype], what="grad_value")
    cabi.assert_close(gs, wgs, *GRAD_TOL[dtype], what="grad_sampling_loc_attn")


FDA_PATH_CASES = {
    # head width 24 pads to 32 accumulator channels in the tiled grad_value kernel
    "d24_three_levels": (2, [(12, 20), (6, 10), (3, 5)], 3, 24, 4, 90, (-0.2, 1.2)),
    # heads wider than 32 channels: the tiled grad_value kernel runs once per window of 32 channels over the same
    # records and lists - two whole windows, a window of 8 behind one of 32, four windows
    "d64_three_levels": (2, [(14, 18), (7, 9), (4, 5)], 3, 64, 4, 120, (-0.1, 1.1)),
    "d40_two_windows": (1, [(10, 12), (5, 6)], 2, 40, 8, 70, (0.0, 1.0)),
    "d128_four_windows": (1, [(9, 8), (5, 4)], 2, 128, 4, 60, (0.0, 1.0)),
    # 6000 queries x 8 points on a 3x3 level: every tile collects far more points than one batch, the list is flushed repeatedly
    "crowded_small_level": (1, [(3, 3), (20, 17)], 2, 16, 8, 6000, (0.0, 1.0)),
    # a level wider than the 16-bit fields of a key: the scan recomputes those positions
    "level_wider_than_a_key": (1, [(1, 65530), (2, 3)], 1, 8, 4, 300, (0.0, 1.0)),
    # a level of more 8x8 tiles (8320) than the binning kernel counts: the binned kernels stand back and the atomic
    # fallback kernel adds everything
    "level_of_more_tiles_than_binned": (1, [(1024, 520), (4, 4)], 1, 8, 4, 300, (0.0, 1.0)),
    # ... with 12000 points on a few cells of it: the fallback has to sum them in fp32 whatever the tensor dtype
    "level_of_more_tiles_than_binned_crowded": (1, [(1024, 520), (4, 4)], 1, 8, 4, 3000, (0.5, 0.503)),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("scatter", ["tiled", "atomic"])
@pytest.mark.parametrize("name", ["detr_small_4lvl_k4", "five_levels", "k8_one_level"] + list(FDA_PATH_CASES))
def test_flash_deform_attn_backward_paths_match_oracle(oracle, name, scatter, dtype):
    from dcnv4_amd import ext
    if name == "level_wider_than_a_key" and dtype != torch.float32:
        pytest.skip("location gradients scale with the level width (65530) and overflow the 16-bit types")
    B, shapes, G, D, K, Q, (lo, hi) = {**FDA_CASES, **FDA_PATH_CASES}[name]
    print(f"case {name} scatter {scatter} dtype {dtype}", flush=True)
    v, shp, st, sla, go = make_fda_inputs(B, shapes, G, D, K, Q, seed=zlib.crc32((name + scatter).encode()) % 1000, dtype=dtype,
                                          loc_lo=lo, loc_hi=hi)
    wgv, wgs = oracle.flash_deform_attn_backward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), cabi.f64(go), K, coord_f32=True)
    with ext.launch_options(scatter=scatter):
        gv, gs = cabi.fda_backward(v.cuda(), shp.cuda(), st.cuda(), sla.cuda(), go.cuda(), K)
    torch.cuda.synchronize()
    rtol, atol = GRAD_TOL[dtype]
    if name in ("crowded_small_level", "level_of_more_tiles_than_binned_crowded"):       # thousands of terms per cell: the tolerance scales with the sum's magnitude
        atol = atol * float(np.abs(wgv).max())
    cabi.assert_close(gv, wgv, rtol, atol, what="grad_value")
    cabi.assert_close(gs, wgs, *GRAD_TOL[dtype], what="grad_sampling_loc_attn")


def test_flash_deform_attn_backward_repeats_and_handles_non_finite_grad_out(oracle):
    B, shapes, G, D, K, Q, (lo, hi) = FDA_CASES["detr_small_4lvl_k4"]
    v, shp, st, sla, go = make_fda_inputs(B, shapes, G, D, K, Q, seed=4, dtype=torch.float16, loc_lo=lo, loc_hi=hi)
    args = (v.cuda(), shp.cuda(), st.cuda(), sla.cuda())
    first = cabi.fda_backward(*args, go.cuda(), K)
    for _ in range(3):
        # grad_sampling_loc_attn has a fixed summation order; grad_value sums in fp32 in the order the hardware ranked the
        # terms and rounds once: repeats differ by at most one unit of fp16, rarely
        again = cabi.fda_backward(*args, go.cuda(), K)
        assert torch.equal(first[1], again[1])
        diff = (first[0].float() - again[0].float()).abs()
        assert (diff <= 2e-3 * first[0].float().abs() + 1e-6).all() and (diff > 0).float().mean().item() < 0.01
    # NaN / Inf in grad_out propagate exactly like in the oracle (sums are floating point throughout), and every
    # finite element keeps the gradient tolerance
    go32 = go.float()
    go32[0, 3, 5] = float("nan")
    go32[1, 7, 40] = float("inf")
    wgv, _ = oracle.flash_deform_attn_backward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), cabi.f64(go32.half()), K, coord_f32=True)
    gv, _ = cabi.fda_backward(*args, go32.half().cuda(), K)
    gv = cabi.f64(gv)
    assert np.array_equal(np.isnan(gv), np.isnan(wgv))
    assert np.array_equal(np.isposinf(gv), np.isposinf(wgv)) and np.array_equal(np.isneginf(gv), np.isneginf(wgv))
    ok = np.isfinite(wgv)
    np.testing.assert_allclose(gv[ok], wgv[ok], rtol=1e-2, atol=1e-2)


def test_c_abi_rejects_bad_arguments():
    from dcnv4_amd import _lib
    v = torch.zeros(2, 4, 4, 16, device="cuda")
    om = torch.zeros(2, 4, 4, 32, device="cuda")
    geom = (3, 3, 1, 1, 1, 1, 1, 1)
    with pytest.raises(ValueError, match="d_stride"):
        cabi.dcnv4_forward(v, om, geom, 1, 16, 1.0, d_stride=3)
    with pytest.raises(RuntimeError, match="im2col_step"):
        cabi.dcnv4_forward(torch.zeros(3, 4, 4, 16, device="cuda"), torch.zeros(3, 4, 4, 32, device="cuda"), geom, 1, 16,
                           1.0, im2col_step=2)
    with pytest.raises(RuntimeError, match="smaller than"):
        cabi.dcnv4_forward(v, om[..., :24].contiguous(), geom, 1, 16, 1.0)
    with pytest.raises(ValueError, match="taps"):
        cabi.dcnv4_forward(v, om, (9, 9, 1, 1, 4, 4, 1, 1), 1, 16, 1.0)
    with pytest.raises(RuntimeError, match="aligned"):
        cabi.dcnv4_forward(v.view(-1)[1:17].view(1, 1, 1, 16), torch.zeros(1, 1, 1, 32, device="cuda"), geom, 1, 16, 1.0)
    L = _lib.load()
    rc = L.dcnv4_gfx950_backward(v.data_ptr(), om.data_ptr(), v.data_ptr(), v.data_ptr(), om.data_ptr(), None, 0,
                                 _lib.DTYPE_F16, 2, 4, 4, 1, 16, *geom, 1.0, 64, 0, 32, 0, 0, 0, None)
    assert rc == _lib.ERR_RUNTIME and b"workspace" in L.dcnv4_gfx950_last_error()
    shp = torch.tensor([[2, 2]] * 17, device="cuda")
    with pytest.raises(ValueError, match="scales"):
        cabi.fda_forward(torch.zeros(1, 68, 1, 16, device="cuda"), shp, torch.zeros(17, dtype=torch.int64, device="cuda"),
                         torch.zeros(1, 1, 1, 17 * 3, device="cuda"), 1)


# ---------------------------------------------------------------- depthwise convolution (offset_mask_dw layer)
# N, H, W, C, k, pad
DW_CASES = {
    "stage1_56x56_c64": (2, 56, 56, 64, 3, 1),
    "stage4_7x7_c512": (3, 7, 7, 512, 3, 1),
    "c112_non_square": (2, 13, 29, 112, 3, 1),
    "c2560_many_vectors": (1, 5, 6, 2560, 3, 1),
    "odd_channels": (2, 9, 8, 7, 3, 1),
    "channels_multiple_of_2": (1, 10, 11, 6, 3, 1),
    "no_padding": (1, 8, 9, 16, 3, 0),
    "full_padding": (1, 6, 7, 16, 3, 2),
    "kernel_5": (2, 11, 10, 24, 5, 2),
    "kernel_7": (1, 12, 9, 16, 7, 3),
    "kernel_1": (2, 6, 6, 32, 1, 0),
    "single_pixel": (1, 1, 1, 8, 3, 1),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("name", list(DW_CASES))
def test_depthwise_conv_matches_oracle(name, dtype):
    from oracle import depthwise
    N, H, W, C, k, pad = DW_CASES[name]
    g = torch.Generator().manual_seed(5)
    x = torch.randn(N, H, W, C, generator=g).to(dtype)
    w = (torch.randn(C, k, k, generator=g) / k).to(dtype)
    b = torch.randn(C, generator=g).to(dtype)
    go = torch.randn(N, H + 2 * pad - k + 1, W + 2 * pad - k + 1, C, generator=g).to(dtype)
    print(f"depthwise case {name} {dtype}", flush=True)
    want = depthwise.depthwise_forward(cabi.f64(x), cabi.f64(w), cabi.f64(b), pad)
    wgx, wgw, wgb = depthwise.depthwise_backward(cabi.f64(x), cabi.f64(w), cabi.f64(go), pad)
    xd, wd, bd, god = x.cuda(), w.cuda(), b.cuda(), go.cuda()
    out = cabi.depthwise_forward(xd, wd, bd, pad)
    out_nb = cabi.depthwise_forward(xd, wd, None, pad)
    gx, gw, gb = cabi.depthwise_backward(xd, wd, god, pad)
    torch.cuda.synchronize()
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    cabi.assert_close(out_nb, want - cabi.f64(b), *FWD_TOL[dtype], what="output without bias")
    cabi.assert_close(gx, wgx, *GRAD_TOL[dtype], what="grad_input")
    # sums over N*Ho*Wo products: tolerance relative to the size of the sum of magnitudes
    n_terms = go.numel() // C
    scale = float(n_terms) ** 0.5
    rtol, atol = GRAD_TOL[dtype]
    cabi.assert_close(gw, wgw, rtol, atol * scale, what="grad_weight")
    cabi.assert_close(gb, wgb, rtol, atol * scale, what="grad_bias")
    # skipping outputs leaves them alone and gives the same values for the others
    gx2, gw2, gb2 = cabi.depthwise_backward(xd, wd, god, pad, with_bias=False)
    assert gb2 is None and torch.equal(gx2, gx) and torch.equal(gw2, gw)


def test_depthwise_conv_rejects_unsupported_kernels():
    x = torch.zeros(1, 4, 4, 8, device="cuda")
    with pytest.raises(ValueError, match="kernel size"):
        cabi.depthwise_forward(x, torch.zeros(8, 2, 2, device="cuda"), None, 0)
    with pytest.raises(ValueError, match="padding"):
        cabi.depthwise_forward(x, torch.zeros(8, 3, 3, device="cuda"), None, 3)


# ---------------------------------------------------------------- layer norm + layer scale + residual
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("rows,C", [(2 * 56 * 56, 112), (300, 224), (77, 448), (33, 896), (5, 8), (9, 64), (3, 4096), (1, 2048),
                                    (130, 1024), (7, 40)])
def test_layer_norm_residual_matches_oracle(rows, C, dtype):
    from oracle import layer_norm
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    if C % vec or C // vec > 512:
        pytest.skip("channel count is not a whole number of 16-byte vectors for this dtype, or more than 512 of them")
    g = torch.Generator().manual_seed(9)
    y = (torch.randn(rows, C, generator=g) * 2 + 0.5).to(dtype)
    res = torch.randn(rows, C, generator=g).to(dtype)
    w = (1 + 0.3 * torch.randn(C, generator=g)).to(dtype)
    b = (0.2 * torch.randn(C, generator=g)).to(dtype)
    gamma = torch.randn(C, generator=g).to(dtype)
    print(f"layer norm case rows {rows} C {C} {dtype}", flush=True)
    for use_res, use_gamma in ((True, True), (False, True), (True, False), (False, False)):
        want = layer_norm.layer_norm_residual(cabi.f64(y), cabi.f64(w), cabi.f64(b), 1e-6, cabi.f64(gamma) if use_gamma else None,
                                              cabi.f64(res) if use_res else None)
        got = cabi.layer_norm_residual(y.cuda(), res.cuda() if use_res else None, w.cuda(), b.cuda(),
                                       gamma.cuda() if use_gamma else None, 1e-6)
        rtol, atol = FWD_TOL[dtype]
        cabi.assert_close(got, want, rtol, max(atol, 1e-4), what=f"residual={use_res} gamma={use_gamma}")


def test_layer_norm_residual_rejects_unsupported_widths():
    y = torch.zeros(4, 12, device="cuda", dtype=torch.float16)
    w = torch.ones(12, device="cuda", dtype=torch.float16)
    with pytest.raises(ValueError, match="multiple of 8"):
        cabi.layer_norm_residual(y, None, w, w, None, 1e-6)
    y = torch.zeros(2, 8192, device="cuda", dtype=torch.float16)
    w = torch.ones(8192, device="cuda", dtype=torch.float16)
    with pytest.raises(ValueError, match="too long"):
        cabi.layer_norm_residual(y, None, w, w, None, 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=["fp32", "fp16"])
def test_flash_deform_attn_head_major_order_matches_oracle_and_row_order(oracle, dtype):
    """A value image larger than half an L2 slice whose heads each fit one: the library then gives every workgroup one
    head and orders workgroups [image][head][queries].  Same arithmetic per (query, head), so the same bits as the
    row order, and parity with the oracle."""
    B, shapes, G, D, K, Q = 2, [(64, 64), (32, 32)], 8, 32, 4, 150
    v, shp, st, sla, go = make_fda_inputs(B, shapes, G, D, K, Q, seed=21, dtype=dtype, loc_lo=-0.05, loc_hi=1.05)
    assert v[0].numel() * v.element_size() > (2 << 20)
    args = (v.cuda(), shp.cuda(), st.cuda(), sla.cuda())
    print(f"head-major case {dtype}", flush=True)
    out = cabi.fda_forward(*args, K)
    gv, gs = cabi.fda_backward(*args, go.cuda(), K)
    from dcnv4_amd import ext
    with ext.launch_options(fda_order="rows"):
        out_rows = cabi.fda_forward(*args, K)
        gv_rows, gs_rows = cabi.fda_backward(*args, go.cuda(), K)
    assert torch.equal(out, out_rows) and torch.equal(gs, gs_rows)
    assert (gv.float() - gv_rows.float()).abs().max().item() <= 2e-3 * gv.float().abs().max().item()      # fp32 sums in hardware order
    want = oracle.flash_deform_attn_forward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), K, coord_f32=True)
    wgv, wgs = oracle.flash_deform_attn_backward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), cabi.f64(go), K, coord_f32=True)
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    cabi.assert_close(gv, wgv, *GRAD_TOL[dtype], what="grad_value")
    cabi.assert_close(gs, wgs, *GRAD_TOL[dtype], what="grad_sampling_loc_attn")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("name,B,shapes,G,D,K,Q,lo,hi", [
    ("pyramid_two_levels_staged", 2, [(64, 64), (32, 32), (16, 16), (8, 8)], 8, 32, 4, 700, -0.05, 1.05),
    ("all_levels_staged", 1, [(12, 20), (6, 10), (3, 5)], 3, 24, 4, 2100, -0.2, 1.2),
    ("nothing_fits", 1, [(200, 160)], 2, 32, 8, 300, 0.0, 1.0),
    ("k3_d8_five_levels", 2, [(9, 7), (5, 5), (4, 3), (2, 2), (1, 1)], 5, 8, 3, 1030, -0.3, 1.3),
])
def test_flash_deform_attn_forward_with_small_levels_staged_in_lds(oracle, name, B, shapes, G, D, K, Q, lo, hi, dtype):
    """The forward that copies the smallest levels of one head's value slice into LDS, forced on: parity with the
    oracle, and the same bits as the kernel that gathers everything from memory (same arithmetic per (query, head))."""
    from dcnv4_amd import ext
    v, shp, st, sla, _ = make_fda_inputs(B, shapes, G, D, K, Q, seed=zlib.crc32(name.encode()) % 1000, dtype=dtype, loc_lo=lo, loc_hi=hi)
    args = (v.cuda(), shp.cuda(), st.cuda(), sla.cuda())
    print(f"staged forward case {name} {dtype}", flush=True)
    with ext.launch_options(fda_order="heads", fda_stage="on"):
        out = cabi.fda_forward(*args, K)
    with ext.launch_options(fda_order="heads", fda_stage="off"):
        plain = cabi.fda_forward(*args, K)
    torch.cuda.synchronize()
    want = oracle.flash_deform_attn_forward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), K, coord_f32=True)
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    assert torch.equal(out, plain)
