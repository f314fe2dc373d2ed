"""GPU parity at the benchmark's own sub-workloads, at the input recipes of the reference's manual scripts, and on
inputs chosen to expose accumulation error: heavy-tailed gradients, sampling points that pile up on one input pixel,
offsets far beyond any staged window.  Everything goes through the C ABI and is checked against the CPU oracle on
identical bits.

Heavy-tailed cases use a per-element bound instead of one absolute tolerance: an element of grad_value is a sum of
terms, and an implementation that accumulates in fp32 and rounds once is off by about one rounding of the result
plus fp32 noise on the sum of the terms' magnitudes.  That sum of magnitudes is itself a backward pass (all
bilinear weights are non-negative): the oracle run on |grad_out| and |modulation|.
"""
import math
import zlib

import numpy as np
import pytest
import torch

from tests import cabi
from tests.inputs import level_start_index, make_dcnv4_inputs, make_fda_inputs

pytestmark = pytest.mark.gpu

FWD_TOL = {torch.float32: (1e-4, 1e-5), torch.float16: (1e-2, 1e-3), torch.bfloat16: (2e-2, 2e-2)}
GRAD_TOL = {torch.float32: (1e-3, 1e-4), torch.float16: (1e-2, 1e-2), torch.bfloat16: (4e-2, 8e-2)}
GEOM3 = (3, 3, 1, 1, 1, 1, 1, 1)

# name: B, H, W, G, D, offset_scale, offset_range, dtypes  (3x3, stride 1, pad 1: every benchmark configuration)
WORKLOADS = {
    # FlashInternImage-T stage 3 (batch 64 in the benchmark)
    "T_stage3_14x14_g16": (4, 14, 14, 16, 16, 1.0, 3.0, (torch.float32, torch.float16)),
    # dense prediction, FlashInternImage-L widths (batch 2 in the benchmark), offsets U(-4, 4)
    "L_dense2_128x128_g20": (1, 128, 128, 20, 16, 1.0, 4.0, (torch.float16,)),
    "L_dense3_64x64_g40": (1, 64, 64, 40, 16, 1.0, 4.0, (torch.float16,)),
    "L_dense4_32x32_g80": (1, 32, 32, 80, 16, 1.0, 4.0, (torch.float16,)),
    # FlashInternImage-B stages 2-4 (batch 128 in the benchmark), the model's offset_scale
    "B_stage2_28x28_g14": (2, 28, 28, 14, 16, 0.5, 3.0, (torch.float16,)),
    "B_stage3_14x14_g28": (2, 14, 14, 28, 16, 0.5, 3.0, (torch.float16,)),
    "B_stage4_7x7_g56": (3, 7, 7, 56, 16, 0.5, 3.0, (torch.float16,)),
}


def _check_dcn(oracle, v, om, go, G, D, scale, dtype, geom=GEOM3, rc=0, grad_tol=None):
    args = (*geom, G, D, scale, rc)
    want = oracle.dcnv4_forward(cabi.f64(v), cabi.f64(om), *args, coord_f32=True)
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *args, coord_f32=True)
    out = cabi.dcnv4_forward(v.cuda(), om.cuda(), geom, G, D, scale, rc)
    gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), geom, G, D, scale, rc)
    torch.cuda.synchronize()
    grad_tol = grad_tol or GRAD_TOL[dtype]
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    cabi.assert_close(gv, wgv, *grad_tol, what="grad_value")
    cabi.assert_close(gom, wgom, *grad_tol, what="grad_offset_mask")


@pytest.mark.parametrize("name,dtype", [(n, d) for n, c in WORKLOADS.items() for d in c[-1]],
                         ids=[f"{n}-{str(d).split('.')[-1]}" for n, c in WORKLOADS.items() for d in c[-1]])
def test_dcnv4_benchmark_sub_workloads_match_oracle(oracle, name, dtype):
    B, H, W, G, D, scale, rng, _ = WORKLOADS[name]
    print(f"workload {name} {dtype}", flush=True)
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, offset_range=rng, seed=zlib.crc32(name.encode()) % 1000, dtype=dtype)
    _check_dcn(oracle, v, om, go, G, D, scale, dtype)


def _pack_offset_mask(offset, mask):
    """offset (B,Ho,Wo,G,2K), mask (B,Ho,Wo,G,K) -> packed rows padded to a multiple of 8, as the reference's scripts
    build them (DCNv4_op/scripts/test_dcnv4.py:84,104-107)."""
    B, Ho, Wo, G, K2 = offset.shape
    om = torch.cat([offset, mask], -1).reshape(B, Ho, Wo, G * (K2 // 2) * 3)
    pad = int(math.ceil(om.shape[-1] / 8) * 8) - om.shape[-1]
    return torch.cat([om, torch.zeros(B, Ho, Wo, pad)], -1)


def test_dcnv4_reference_forward_script_recipe(oracle):
    """DCNv4_op/scripts/test_dcnv4.py:25-26,44,76-80: 56x56, 4 groups of 32 channels, offset_scale 2, offsets
    U(-10, 10) (displacements up to 20 pixels), value U(0, 1), modulation U(0, 1) + 1e-5, seed 3, fp16; two images of
    the script's 64.  Tolerance of the script (rtol 1e-2, atol 1e-3) for the output."""
    g = torch.Generator().manual_seed(3)
    B, H, W, G, D, K = 2, 56, 56, 4, 32, 9
    v = torch.rand(B, H, W, G * D, generator=g).half()
    offset = ((torch.rand(B, H, W, G, K * 2, generator=g) * 2 - 1) * 10).half().float()
    mask = (torch.rand(B, H, W, G, K, generator=g) + 1e-5).half().float()
    om = _pack_offset_mask(offset, mask).half()
    go = torch.randn(B, H, W, G * D, generator=g).half()
    print("reference recipe test_dcnv4.py", flush=True)
    _check_dcn(oracle, v, om, go, G, D, 2.0, torch.float16)


def test_dcnv4_reference_backward_script_recipe(oracle):
    """DCNv4_op/scripts/test_dcnv4_bwd.py:102-106,131: value U(0, 10), offsets U(-2, 2), modulation U(0, 1) + 1e-5,
    upstream gradient of sum()/10 (a constant 0.1), fp16, 56x56, 4 groups of 32 channels, offset_scale 2."""
    g = torch.Generator().manual_seed(3)
    B, H, W, G, D, K = 2, 56, 56, 4, 32, 9
    v = (torch.rand(B, H, W, G * D, generator=g) * 10).half()
    offset = ((torch.rand(B, H, W, G, K * 2, generator=g) * 2 - 1) * 2).half().float()
    mask = (torch.rand(B, H, W, G, K, generator=g) + 1e-5).half().float()
    om = _pack_offset_mask(offset, mask).half()
    go = torch.full((B, H, W, G * D), 0.1).half()
    print("reference recipe test_dcnv4_bwd.py", flush=True)
    # values up to 10 and nine taps: outputs and gradients of the order of 50; the script's relative tolerance
    _check_dcn(oracle, v, om, go, G, D, 2.0, torch.float16, grad_tol=(1e-2, 5e-2))


def test_flash_deform_attn_reference_script_recipe(oracle):
    """DCNv4_op/scripts/test_flash_deform_attn.py:104-111: one image, 8 heads of 32 channels, levels 100x152 ... 13x19,
    15200 queries, 8 points per level, value U(0, 0.01), locations U(0, 1), logits U(0, 1) + 1e-5, fp16."""
    g = torch.Generator().manual_seed(3)
    shapes = [(100, 152), (50, 76), (25, 38), (13, 19)]
    starts, N = level_start_index(shapes)
    B, G, D, L, K, Q = 1, 8, 32, 4, 8, 15200
    v = (torch.rand(B, N, G, D, generator=g) * 0.01).half()
    loc = torch.rand(B, Q, G, L * K * 2, generator=g)
    logits = torch.rand(B, Q, G, L * K, generator=g) + 1e-5
    sla = torch.cat([loc, logits], -1).half()
    go = torch.randn(B, Q, G * D, generator=g).half()
    shp, st = torch.tensor(shapes, dtype=torch.int64), torch.tensor(starts, dtype=torch.int64)
    print("reference recipe test_flash_deform_attn.py", flush=True)
    want = oracle.flash_deform_attn_forward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), K, coord_f32=True)
    wgv, wgs = oracle.flash_deform_attn_backward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), cabi.f64(go), K, coord_f32=True)
    out = cabi.fda_forward(v.cuda(), shp.cuda(), st.cuda(), sla.cuda(), K)
    gv, gs = cabi.fda_backward(v.cuda(), shp.cuda(), st.cuda(), sla.cuda(), go.cuda(), K)
    torch.cuda.synchronize()
    cabi.assert_close(out, want, 1e-2, 1e-3 * 0.01, what="output")      # outputs are of the order of 0.005
    # a cell of the coarsest level collects ~1500 terms; the tolerance follows the size of the sums
    cabi.assert_close(gv, wgv, 1e-2, 1e-2 * float(np.abs(wgv).std()), what="grad_value")
    cabi.assert_close(gs, wgs, 1e-2, 1e-2 * float(np.abs(wgs).std()) + 1e-4, what="grad_sampling_loc_attn")


# ---------------------------------------------------------------- accumulation accuracy
def _magnitude_sum_dcn(oracle, v, om, go, G, D, scale, K=9):
    """Sum of |term| over the terms of every grad_value element: the backward of |grad_out| under |modulation|."""
    om_abs = cabi.f64(om).copy()
    body = om_abs[..., : G * K * 3].reshape(*om_abs.shape[:3], G, K * 3)
    body[..., 2 * K:] = np.abs(body[..., 2 * K:])
    mag, _ = oracle.dcnv4_backward(cabi.f64(v), om_abs, np.abs(cabi.f64(go)), *GEOM3, G, D, scale, 0, coord_f32=True)
    return mag


def _magnitude_sum_dcn_geom(oracle, v, om, go, geom, G, D, scale, K=9):
    om_abs = cabi.f64(om).copy()
    body = om_abs[..., : G * K * 3].reshape(*om_abs.shape[:3], G, K * 3)
    body[..., 2 * K:] = np.abs(body[..., 2 * K:])
    mag, _ = oracle.dcnv4_backward(cabi.f64(v), om_abs, np.abs(cabi.f64(go)), *geom, G, D, scale, 0, coord_f32=True)
    return mag


def _assert_accumulated_like_fp32(got, want, mag, dtype, what):
    """|got - want| <= one generous rounding of the result in the tensor dtype + 2^-14 of the sum of magnitudes."""
    eps = {torch.float32: 2.0 ** -20, torch.float16: 2.0 ** -9, torch.bfloat16: 2.0 ** -6}[dtype]
    tiny = {torch.float32: 1e-37, torch.float16: 2.0 ** -23, torch.bfloat16: 1e-37}[dtype]     # fp16 subnormal spacing
    got = cabi.f64(got)
    assert np.isfinite(got).all(), f"{what}: non-finite values"
    tol = eps * np.abs(want) + 2.0 ** -14 * mag + tiny
    err = np.abs(got - want)
    bad = err > tol
    if bad.any():
        i = np.unravel_index(np.argmax(err / tol), err.shape)
        raise AssertionError(f"{what}: {bad.sum()} / {bad.size} elements off; worst at {i}: got {got[i]!r} want {want[i]!r} "
                             f"magnitude sum {mag[i]!r} (err {err[i]:.3e}, allowed {tol[i]:.3e})")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=["fp16", "bf16", "fp32"])
@pytest.mark.parametrize("tile", ["32x32_one_group", "16x16_four_groups"])
def test_dcnv4_grad_value_keeps_fp32_accuracy_on_heavy_tailed_gradients(oracle, dtype, tile):
    """grad_out N(0, 1) with 0.1 % of the elements scaled by 2^12 and one image region scaled by 2^-12 (what loss
    scaling and dead regions produce), one modulation scalar 30 times the others: elements far below the largest
    term must keep their precision, as they do when gradients are summed in fp32 and rounded once
    (DCNv4_op/src/cuda/dcnv4_cuda.cu:133-139,169-171)."""
    B, H, W, G, D = (2, 40, 40, 2, 16) if tile == "32x32_one_group" else (2, 16, 16, 5, 16)
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, offset_range=3.0, seed=11, dtype=torch.float32)
    g = torch.Generator().manual_seed(12)
    spikes = torch.rand(go.shape, generator=g) < 1e-3
    go[spikes] *= 4096.0
    go[:, : H // 2, : W // 2] *= 2.0 ** -12
    om[0, H // 3, W // 3, 2 * 9] = 30.0              # first modulation scalar of group 0
    v, om, go = v.to(dtype), om.to(dtype), go.to(dtype)
    print(f"heavy-tailed dcnv4 {tile} {dtype}", flush=True)
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *GEOM3, G, D, 1.0, 0, coord_f32=True)
    mag = _magnitude_sum_dcn(oracle, v, om, go, G, D, 1.0)
    gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), GEOM3, G, D, 1.0)
    torch.cuda.synchronize()
    _assert_accumulated_like_fp32(gv, wgv, mag, dtype, "grad_value")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=["fp16", "bf16", "fp32"])
def test_dcnv4_grad_value_when_most_sampling_points_hit_one_pixel(oracle, dtype):
    """Offsets that send every tap of every output pixel of a 32x32 image exactly onto pixel (10, 20), with constant
    grad_out and modulation: one cell collects 9216 equal terms of full weight.  Any accumulator narrower than the
    sum wraps."""
    B, H, W, G, D, K = 1, 32, 32, 1, 16, 9
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, seed=5, dtype=torch.float32)
    body = om[..., : G * K * 3].reshape(B, H, W, G, K * 3)
    ys, xs = torch.meshgrid(torch.arange(H, dtype=torch.float32), torch.arange(W, dtype=torch.float32), indexing="ij")
    k = 0
    for i in range(3):          # x index outer, y index inner: the packing's tap order
        for j in range(3):
            body[0, :, :, 0, 2 * k] = 20.0 - (xs - 1 + i)        # tap position = p0 - 1 + (i, j) + offset, offset_scale 1
            body[0, :, :, 0, 2 * k + 1] = 10.0 - (ys - 1 + j)
            k += 1
    body[..., 2 * K:] = 1.0
    go.fill_(1.0)
    v, om, go = v.to(dtype), om.to(dtype), go.to(dtype)
    print(f"concentrated dcnv4 {dtype}", flush=True)
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *GEOM3, G, D, 1.0, 0, coord_f32=True)
    assert wgv.max() == 9216.0
    gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), GEOM3, G, D, 1.0)
    torch.cuda.synchronize()
    rtol = {torch.float32: 1e-4, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dtype]
    cabi.assert_close(gv, wgv, rtol, 1e-3, what="grad_value")
    cabi.assert_close(gom, wgom, *GRAD_TOL[dtype], what="grad_offset_mask")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
def test_dcnv4_far_offsets_at_image_scale_keep_the_stated_tolerance(oracle, dtype):
    """Offsets U(-10, 10) at offset_scale 2 on a 56x56 image: nearly every sampling point lies outside any window a
    tile stages, so forward and backward run their per-point global-memory paths.  Gradients must still be summed
    in fp32 (the reference never accumulates in a 16-bit type)."""
    B, H, W, G, D = 1, 56, 56, 2, 16
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, offset_range=10.0, seed=17, dtype=dtype)
    print(f"far offsets {dtype}", flush=True)
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *GEOM3, G, D, 2.0, 0, coord_f32=True)
    mag = _magnitude_sum_dcn(oracle, v, om, go, G, D, 2.0)
    want = oracle.dcnv4_forward(cabi.f64(v), cabi.f64(om), *GEOM3, G, D, 2.0, 0, coord_f32=True)
    out = cabi.dcnv4_forward(v.cuda(), om.cuda(), GEOM3, G, D, 2.0)
    gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), GEOM3, G, D, 2.0)
    torch.cuda.synchronize()
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    _assert_accumulated_like_fp32(gv, wgv, mag, dtype, "grad_value")
    cabi.assert_close(gom, wgom, *GRAD_TOL[dtype], what="grad_offset_mask")


@pytest.mark.parametrize("gather", ["tiled", "direct"])
@pytest.mark.parametrize("geom", [GEOM3, (3, 3, 2, 2, 1, 1, 1, 1)], ids=["stride1", "stride2"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=["fp16", "bf16", "fp32"])
def test_dcnv4_backward_with_a_few_outlier_offsets(oracle, dtype, geom, gather):
    """Offsets U(-2, 2) on a 72x40 image (six grad_value tiles) except for a handful of sampling points sent 20 to 70
    pixels away - into other tiles, onto the image's far corner, outside the image: the backward keeps the reach of
    the bulk for all tiles and lets only the tiles such a point lands in look further; every gradient must come out
    as if nothing were special, summed in fp32."""
    from dcnv4_amd import ext
    B, H, W, G, D, K = 2, 72, 40, 2, 16, 9
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, *geom, offset_range=2.0, seed=31, dtype=torch.float32)
    Ho, Wo = om.shape[1:3]
    body = om[..., : G * K * 3].reshape(B, Ho, Wo, G, K * 3)
    far = [  # image, output row, output column, group, tap, x offset, y offset
        (0, 2, 1, 0, 4, 30.0, 50.0), (0, Ho - 1, Wo - 1, 1, 0, -35.0, -66.0), (1, Ho // 2, 2, 0, 8, 33.25, -0.5),
        (1, 1, Wo // 2, 1, 3, 0.5, 60.75), (0, 3, 3, 1, 7, 300.0, 5.0), (1, Ho - 2, 1, 0, 2, 25.5, -40.5), (0, Ho // 2, Wo // 2, 0, 5, -17.5, 21.0)]
    for b, r, c, g, k, dx, dy in far:
        body[b, r, c, g, 2 * k], body[b, r, c, g, 2 * k + 1] = dx, dy
    v, om, go = v.to(dtype), om.to(dtype), go.to(dtype)
    print(f"outlier offsets {dtype} {geom} {gather}", flush=True)
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *geom, G, D, 1.0, 0, coord_f32=True)
    mag = _magnitude_sum_dcn_geom(oracle, v, om, go, geom, G, D, 1.0)
    with ext.launch_options(gather=gather):
        gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), geom, G, D, 1.0)
    torch.cuda.synchronize()
    _assert_accumulated_like_fp32(gv, wgv, mag, dtype, "grad_value")
    cabi.assert_close(gom, wgom, *GRAD_TOL[dtype], what="grad_offset_mask")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=["fp16", "bf16", "fp32"])
def test_flash_deform_attn_grad_value_keeps_fp32_accuracy_on_heavy_tailed_gradients(oracle, dtype):
    B, shapes, G, D, K, Q = 2, [(24, 24), (12, 12)], 4, 32, 4, 700
    v, shp, st, sla, go = make_fda_inputs(B, shapes, G, D, K, Q, seed=23, dtype=torch.float32)
    g = torch.Generator().manual_seed(24)
    go[torch.rand(go.shape, generator=g) < 1e-3] *= 4096.0
    go[:, : Q // 2] *= 2.0 ** -12
    v, sla, go = v.to(dtype), sla.to(dtype), go.to(dtype)
    print(f"heavy-tailed attention {dtype}", flush=True)
    wgv, _ = oracle.flash_deform_attn_backward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), cabi.f64(go), K, coord_f32=True)
    mag, _ = oracle.flash_deform_attn_backward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), np.abs(cabi.f64(go)), K, coord_f32=True)
    gv, _ = cabi.fda_backward(v.cuda(), shp.cuda(), st.cuda(), sla.cuda(), go.cuda(), K)
    torch.cuda.synchronize()
    _assert_accumulated_like_fp32(gv, wgv, mag, dtype, "grad_value")


def test_flash_deform_attn_value_rows_no_level_covers_get_zero_gradient(oracle):
    """spatial_size larger than the levels cover, and a gap between two levels: the reference returns
    zeros_like(value) there (DCNv4_op/src/cuda/flash_deform_attn_cuda.cu:118)."""
    shapes, G, D, K, Q = [(6, 5), (3, 4)], 2, 16, 4, 40
    v, shp, st, sla, go = make_fda_inputs(1, shapes, G, D, K, Q, seed=31, dtype=torch.float16)
    N = 30 + 12
    wgv, _ = oracle.flash_deform_attn_backward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), cabi.f64(go), K, coord_f32=True)
    gap, tail = 7, 9
    big = torch.randn(1, N + gap + tail, G, D).half()
    big[:, :30] = v[:, :30]
    big[:, 30 + gap: 30 + gap + 12] = v[:, 30:]
    starts = torch.tensor([0, 30 + gap], dtype=torch.int64)
    from dcnv4_amd import ext
    for scatter in ("tiled", "atomic"):
        with ext.launch_options(scatter=scatter):
            gv, _ = cabi.fda_backward(big.cuda(), shp.cuda(), starts.cuda(), sla.cuda(), go.cuda(), K)
        torch.cuda.synchronize()
        gv = gv.cpu()
        assert (gv[:, 30: 30 + gap] == 0).all() and (gv[:, 30 + gap + 12:] == 0).all(), scatter
        covered = torch.cat([gv[:, :30], gv[:, 30 + gap: 30 + gap + 12]], 1)
        cabi.assert_close(covered, wgv, *GRAD_TOL[torch.float16], what=f"grad_value ({scatter})")
