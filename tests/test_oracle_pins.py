"""Pins for the CPU oracle (oracle/sampling_oracle.c).

The reference ships no golden vectors for this path (its scripts under DCNv4_op/scripts only
compare two GPU ops live), so the oracle is pinned by what the mathematics fixes:
  * agreement in fp64 with an independent torch grid_sample formulation, over strides,
    dilations, paddings, offset_scale, remove_center, non-square kernels and images;
  * closed forms (box sum, integer shifts, single-tap attention, uniform attention);
  * exact zeros outside the image, linearity, padded-tail invariants;
  * central finite differences of the oracle's own forward for every gradient, and torch
    autograd through the grid_sample formulation.
Each check is chosen so that a swapped x/y, a wrong tap order, a dropped offset_scale factor or
a wrong sign in a bilinear derivative fails it.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import torch_core
from tests.inputs import make_dcnv4_inputs, make_fda_inputs

DCN_CASES = [
    # B, H, W, G, D, kh, kw, sh, sw, ph, pw, dh, dw, remove_center, offset_scale, offset_range
    (2, 7, 9, 2, 4, 3, 3, 1, 1, 1, 1, 1, 1, 0, 1.0, 2.0),
    (1, 8, 6, 3, 2, 3, 3, 2, 2, 1, 1, 1, 1, 0, 0.5, 3.0),
    (2, 9, 10, 2, 3, 3, 3, 1, 1, 2, 2, 2, 2, 0, 2.0, 1.5),
    (1, 6, 7, 4, 2, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1.3, 2.5),
    (1, 7, 8, 2, 2, 3, 3, 1, 2, 0, 1, 1, 1, 1, 1.0, 4.0),
    (1, 9, 8, 1, 5, 1, 3, 1, 1, 0, 1, 1, 1, 0, 0.7, 2.0),   # kh != kw, pad_h != pad_w
    (1, 10, 9, 2, 2, 3, 1, 2, 1, 2, 0, 2, 1, 0, 1.0, 2.0),  # kh != kw the other way, mixed stride/dilation
    (1, 5, 5, 7, 1, 3, 3, 1, 1, 1, 1, 1, 1, 0, 1.0, 8.0),   # offsets mostly far outside
]


def _dcn_args(case):
    B, H, W, G, D, kh, kw, sh, sw, ph, pw, dh, dw, rc, scale, rng = case
    return (kh, kw, sh, sw, ph, pw, dh, dw, G, D, scale, rc)


@pytest.mark.parametrize("case", DCN_CASES)
@pytest.mark.parametrize("softmax", [False, True])
def test_dcnv4_c_oracle_matches_grid_sample_formulation(oracle, case, softmax):
    B, H, W, G, D, kh, kw, sh, sw, ph, pw, dh, dw, rc, scale, rng = case
    value, om, go = make_dcnv4_inputs(B, H, W, G, D, kh, kw, sh, sw, ph, pw, dh, dw, rc, rng,
                                      seed=11, dtype=torch.float64)
    args = _dcn_args(case)
    v = value.clone().requires_grad_(True)
    o = om.clone().requires_grad_(True)
    ref = torch_core.dcnv4_core_torch(v, o, *args, softmax=softmax)
    ref.backward(go)
    out = oracle.dcnv4_forward(value.numpy(), om.numpy(), *args, softmax=softmax)
    gv, gom = oracle.dcnv4_backward(value.numpy(), om.numpy(), go.numpy(), *args, softmax=softmax)
    np.testing.assert_allclose(out, ref.detach().numpy(), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(gv, v.grad.numpy(), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(gom, o.grad.numpy(), rtol=1e-10, atol=1e-11)
    used = G * 3 * (kh * kw - rc)
    assert np.all(gom[..., used:] == 0.0)          # padded tail keeps exact zeros


def test_dcnv4_zero_offsets_unit_mask_is_box_sum(oracle):
    B, H, W, G, D = 2, 9, 11, 3, 4
    value, om, _ = make_dcnv4_inputs(B, H, W, G, D, seed=3, dtype=torch.float64)
    K = 9
    om.zero_()
    body = om[..., : G * K * 3].reshape(B, H, W, G, K * 3)
    body[..., 2 * K:] = 1.0
    out = oracle.dcnv4_forward(value.numpy(), om.numpy(), 3, 3, 1, 1, 1, 1, 1, 1, G, D, 1.0)
    box = F.avg_pool2d(value.permute(0, 3, 1, 2), 3, 1, 1, count_include_pad=True) * 9
    np.testing.assert_allclose(out, box.permute(0, 2, 3, 1).numpy(), rtol=1e-12, atol=1e-12)


def test_dcnv4_integer_offsets_are_shifted_copies_in_x_major_tap_order(oracle):
    # one-hot mask on tap k with an integer offset (ox, oy) must copy value[y+ty+oy, x+tx+ox]
    # where tap k = (tx index outer, ty index inner): a y-major order or swapped x/y fails.
    B, H, W, G, D, K = 1, 8, 10, 1, 3, 9
    value, om, _ = make_dcnv4_inputs(B, H, W, G, D, seed=5, dtype=torch.float64)
    for k, (ox, oy) in [(1, (2, -1)), (3, (0, 0)), (5, (-2, 1)), (8, (1, 3))]:
        om.zero_()
        om[..., 2 * k] = ox
        om[..., 2 * k + 1] = oy
        om[..., 2 * K + k] = 1.0
        out = oracle.dcnv4_forward(value.numpy(), om.numpy(), 3, 3, 1, 1, 1, 1, 1, 1, G, D, 1.0)
        tx, ty = k // 3 - 1, k % 3 - 1
        expect = np.zeros_like(out)
        for y in range(H):
            for x in range(W):
                yy, xx = y + ty + oy, x + tx + ox
                if 0 <= yy < H and 0 <= xx < W:
                    expect[0, y, x] = value[0, yy, xx].numpy()
        np.testing.assert_array_equal(out, expect)


def test_dcnv4_offset_scale_multiplies_tap_and_offset(oracle):
    # offset_scale 2 with a one-hot mask on the (+1,+1) tap and offset (0.5, 0) samples 3 px right
    B, H, W, G, D, K = 1, 8, 8, 1, 2, 9
    value, om, _ = make_dcnv4_inputs(B, H, W, G, D, seed=6, dtype=torch.float64)
    om.zero_()
    k = 8
    om[..., 2 * k] = 0.5
    om[..., 2 * K + k] = 1.0
    out = oracle.dcnv4_forward(value.numpy(), om.numpy(), 3, 3, 1, 1, 1, 1, 1, 1, G, D, 2.0)
    np.testing.assert_array_equal(out[0, 2, 1], value[0, 4, 4].numpy())   # x: 1 + 2*(1+0.5), y: 2 + 2*1


def test_dcnv4_out_of_range_taps_give_exact_zeros(oracle):
    B, H, W, G, D, K = 1, 5, 6, 2, 4, 9
    value, om, go = make_dcnv4_inputs(B, H, W, G, D, seed=7, dtype=torch.float64)
    body = om[..., : G * K * 3].reshape(B, H, W, G, K * 3)
    body[..., : 2 * K] = 100.0
    om[..., : G * K * 3] = body.reshape(B, H, W, -1)
    args = (3, 3, 1, 1, 1, 1, 1, 1, G, D, 1.0, 0)
    assert np.all(oracle.dcnv4_forward(value.numpy(), om.numpy(), *args) == 0.0)
    gv, gom = oracle.dcnv4_backward(value.numpy(), om.numpy(), go.numpy(), *args)
    assert np.all(gv == 0.0) and np.all(gom == 0.0)


def test_dcnv4_is_linear_in_value_and_mask(oracle):
    B, H, W, G, D, K = 1, 6, 7, 2, 3, 9
    args = (3, 3, 1, 1, 1, 1, 1, 1, G, D, 1.0, 0)
    v1, om, _ = make_dcnv4_inputs(B, H, W, G, D, seed=8, dtype=torch.float64)
    v2, om2, _ = make_dcnv4_inputs(B, H, W, G, D, seed=9, dtype=torch.float64)
    f = lambda v, o: oracle.dcnv4_forward(v.numpy(), o.numpy(), *args)
    np.testing.assert_allclose(f(2.0 * v1 - 3.0 * v2, om), 2.0 * f(v1, om) - 3.0 * f(v2, om), rtol=1e-12, atol=1e-12)
    oma, omb = om.clone(), om.clone()      # same offsets, different masks
    ma = oma[..., : G * K * 3].reshape(B, H, W, G, K * 3)
    mb = om2[..., : G * K * 3].reshape(B, H, W, G, K * 3)
    mixed = ma.clone()
    mixed[..., 2 * K:] = ma[..., 2 * K:] + mb[..., 2 * K:]
    only_b = ma.clone()
    only_b[..., 2 * K:] = mb[..., 2 * K:]
    omb[..., : G * K * 3] = only_b.reshape(B, H, W, -1)
    omm = om.clone()
    omm[..., : G * K * 3] = mixed.reshape(B, H, W, -1)
    np.testing.assert_allclose(f(v1, omm), f(v1, oma) + f(v1, omb), rtol=1e-12, atol=1e-12)


def _central_differences(fn, x, go, idx, eps=1e-6):
    out = []
    flat = x.reshape(-1)
    for i in idx:
        old = flat[i]
        flat[i] = old + eps
        hi = fn()
        flat[i] = old - eps
        lo = fn()
        flat[i] = old
        out.append(float(((hi - lo) * go).sum() / (2 * eps)))
    return np.array(out)


@pytest.mark.parametrize("softmax", [False, True])
def test_dcnv4_backward_matches_finite_differences(oracle, softmax):
    B, H, W, G, D = 1, 5, 6, 2, 3
    args = (3, 3, 1, 1, 1, 1, 1, 1, G, D, 1.7, 0)
    value, om, go = make_dcnv4_inputs(B, H, W, G, D, offset_range=1.5, seed=21, dtype=torch.float64)
    v, o, g = value.numpy().copy(), om.numpy().copy(), go.numpy()
    gv, gom = oracle.dcnv4_backward(v, o, g, *args, softmax=softmax)
    rng = np.random.default_rng(0)
    fwd = lambda: oracle.dcnv4_forward(v, o, *args, softmax=softmax)
    iv = rng.choice(v.size, 40, replace=False)
    np.testing.assert_allclose(gv.reshape(-1)[iv], _central_differences(fwd, v, g, iv), rtol=1e-6, atol=1e-7)
    used = np.arange(o.size).reshape(o.shape)[..., : G * 27].reshape(-1)
    io = rng.choice(used, 80, replace=False)
    np.testing.assert_allclose(gom.reshape(-1)[io], _central_differences(fwd, o, g, io), rtol=1e-5, atol=1e-6)


def test_dcnv4_grad_mask_is_inner_product_with_each_tap_sample(oracle):
    # grad_mask[k] = <grad_out, sample_k>; sample_k is the forward with a one-hot mask on k
    B, H, W, G, D, K = 1, 4, 5, 1, 3, 9
    args = (3, 3, 1, 1, 1, 1, 1, 1, G, D, 1.0, 0)
    value, om, go = make_dcnv4_inputs(B, H, W, G, D, seed=22, dtype=torch.float64)
    _, gom = oracle.dcnv4_backward(value.numpy(), om.numpy(), go.numpy(), *args)
    for k in range(K):
        one = om.clone()
        one[..., 2 * K: 3 * K] = 0.0
        one[..., 2 * K + k] = 1.0
        sample = oracle.dcnv4_forward(value.numpy(), one.numpy(), *args)
        np.testing.assert_allclose(gom[..., 2 * K + k], (sample * go.numpy()).sum(-1), rtol=1e-12, atol=1e-12)


FDA_CASES = [
    # B, shapes, G, D, K, Q, loc range
    (2, [(6, 5), (3, 4)], 2, 4, 4, 7, (0.0, 1.0)),
    (1, [(5, 7)], 3, 2, 8, 9, (-0.2, 1.2)),
    (1, [(8, 8), (4, 4), (2, 2), (1, 1)], 2, 3, 4, None, (0.0, 1.0)),
    (1, [(4, 6), (3, 3), (2, 5), (2, 2), (1, 3)], 1, 5, 4, 6, (-0.5, 1.5)),
]


@pytest.mark.parametrize("case", FDA_CASES)
def test_fda_c_oracle_matches_grid_sample_formulation(oracle, case):
    B, shapes, G, D, K, Q, (lo, hi) = case
    value, shp, start, sla, go = make_fda_inputs(B, shapes, G, D, K, Q, seed=31, dtype=torch.float64,
                                                 loc_lo=lo, loc_hi=hi)
    v = value.clone().requires_grad_(True)
    s = sla.clone().requires_grad_(True)
    ref = torch_core.msda_core_torch(v, shapes, start.tolist(), s, K)
    ref.backward(go)
    out = oracle.flash_deform_attn_forward(value.numpy(), shp.numpy(), start.numpy(), sla.numpy(), K)
    gv, gs = oracle.flash_deform_attn_backward(value.numpy(), shp.numpy(), start.numpy(), sla.numpy(),
                                               go.numpy(), K)
    np.testing.assert_allclose(out, ref.detach().numpy(), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(gv, v.grad.numpy(), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(gs, s.grad.numpy(), rtol=1e-10, atol=1e-11)


def test_fda_pixel_centre_locations_with_uniform_logits_average_the_pixels(oracle):
    # location ((x+0.5)/W, (y+0.5)/H) hits pixel (y,x) exactly; equal logits => plain mean of taps
    H, W, G, D, K = 4, 5, 2, 3, 4
    value, shp, start, sla, _ = make_fda_inputs(1, [(H, W)], G, D, K, Q=3, seed=32, dtype=torch.float64)
    pix = [(0, 0), (3, 4), (2, 1), (1, 3)]
    for k, (y, x) in enumerate(pix):
        sla[..., 2 * k] = (x + 0.5) / W
        sla[..., 2 * k + 1] = (y + 0.5) / H
    sla[..., 2 * K:] = 0.25
    out = oracle.flash_deform_attn_forward(value.numpy(), shp.numpy(), start.numpy(), sla.numpy(), K)
    expect = sum(value[0, y * W + x] for y, x in pix) / 4          # (G, D)
    np.testing.assert_allclose(out[0, 0], expect.reshape(-1).numpy(), rtol=1e-12, atol=1e-12)


def test_fda_level_start_index_selects_the_level(oracle):
    # a dominant logit on a tap of level 1 must read from value[start_1 + ...]
    shapes, G, D, K = [(3, 3), (2, 2)], 1, 2, 4
    value, shp, start, sla, _ = make_fda_inputs(1, shapes, G, D, K, Q=1, seed=33, dtype=torch.float64)
    sla[..., 2 * 2 * K:] = -1e3
    t = 1 * K + 2
    sla[..., 2 * 2 * K + t] = 0.0
    sla[..., 2 * t] = 1.5 / 2
    sla[..., 2 * t + 1] = 0.5 / 2
    out = oracle.flash_deform_attn_forward(value.numpy(), shp.numpy(), start.numpy(), sla.numpy(), K)
    np.testing.assert_allclose(out[0, 0], value[0, 9 + 0 * 2 + 1, 0].numpy(), rtol=1e-12)


def test_fda_backward_matches_finite_differences(oracle):
    shapes, G, D, K = [(5, 4), (3, 2)], 2, 3, 4
    value, shp, start, sla, go = make_fda_inputs(1, shapes, G, D, K, Q=5, seed=34, dtype=torch.float64,
                                                 loc_lo=-0.1, loc_hi=1.1)
    v, s, g = value.numpy().copy(), sla.numpy().copy(), go.numpy()
    gv, gs = oracle.flash_deform_attn_backward(v, shp.numpy(), start.numpy(), s, g, K)
    fwd = lambda: oracle.flash_deform_attn_forward(v, shp.numpy(), start.numpy(), s, K)
    rng = np.random.default_rng(1)
    iv = rng.choice(v.size, 40, replace=False)
    np.testing.assert_allclose(gv.reshape(-1)[iv], _central_differences(fwd, v, g, iv), rtol=1e-6, atol=1e-7)
    io = rng.choice(s.size, 80, replace=False)
    np.testing.assert_allclose(gs.reshape(-1)[io], _central_differences(fwd, s, g, io), rtol=1e-5, atol=1e-6)


def test_fda_logit_gradients_sum_to_zero_and_vanish_for_out_of_range_locations(oracle):
    shapes, G, D, K = [(4, 4), (2, 2)], 2, 2, 4
    value, shp, start, sla, go = make_fda_inputs(1, shapes, G, D, K, Q=6, seed=35, dtype=torch.float64)
    _, gs = oracle.flash_deform_attn_backward(value.numpy(), shp.numpy(), start.numpy(), sla.numpy(), go.numpy(), K)
    np.testing.assert_allclose(gs[..., 16:].sum(-1), 0.0, atol=1e-12)     # softmax Jacobian has zero row sums
    sla[..., :16] = 7.0
    gv, gs = oracle.flash_deform_attn_backward(value.numpy(), shp.numpy(), start.numpy(), sla.numpy(), go.numpy(), K)
    assert np.all(gv == 0.0) and np.all(gs == 0.0)


def test_fp32_coordinate_mode_tracks_the_float64_mode(oracle):
    # same inputs, coordinates rounded to fp32 vs kept in double: only ulp-level coordinate noise may differ
    B, H, W, G, D = 1, 20, 24, 2, 4
    args = (3, 3, 1, 1, 1, 1, 1, 1, G, D, 1.3, 0)
    value, om, go = make_dcnv4_inputs(B, H, W, G, D, seed=41)          # fp32-representable inputs
    v, o, g = value.double().numpy(), om.double().numpy(), go.double().numpy()
    a = oracle.dcnv4_forward(v, o, *args)
    b = oracle.dcnv4_forward(v, o, *args, coord_f32=True)
    assert np.abs(a - b).max() < 2e-4 and np.abs(a - b).max() > 0.0
    ga, gb = oracle.dcnv4_backward(v, o, g, *args), oracle.dcnv4_backward(v, o, g, *args, coord_f32=True)
    assert np.abs(ga[0] - gb[0]).max() < 2e-4 and np.abs(ga[1] - gb[1]).max() < 2e-3
    value, shp, start, sla, go = make_fda_inputs(1, [(30, 40), (7, 9)], 2, 4, 4, Q=50, seed=42)
    v, s, g = value.double().numpy(), sla.double().numpy(), go.double().numpy()
    a = oracle.flash_deform_attn_forward(v, shp.numpy(), start.numpy(), s, 4)
    b = oracle.flash_deform_attn_forward(v, shp.numpy(), start.numpy(), s, 4, coord_f32=True)
    assert np.abs(a - b).max() < 2e-4
    ga = oracle.flash_deform_attn_backward(v, shp.numpy(), start.numpy(), s, g, 4)
    gb = oracle.flash_deform_attn_backward(v, shp.numpy(), start.numpy(), s, g, 4, coord_f32=True)
    assert np.abs(ga[0] - gb[0]).max() < 2e-4 and np.abs(ga[1] - gb[1]).max() < 5e-3


# ---------------------------------------------------------------- depthwise convolution oracle (oracle/depthwise.py)
DW_CASES = [
    # N, H, W, C, k, pad
    (2, 7, 9, 6, 3, 1),
    (1, 5, 6, 4, 3, 0),
    (1, 6, 5, 3, 3, 2),
    (2, 8, 7, 5, 5, 2),
    (1, 9, 9, 2, 7, 3),
    (1, 4, 4, 8, 1, 0),
]


@pytest.mark.parametrize("case", DW_CASES)
def test_depthwise_oracle_matches_torch_conv2d_and_autograd(case):
    """The reference's layer IS nn.Conv2d(groups=C) between two permutes (modules/dcnv4.py:67-75,121-123)."""
    from oracle import depthwise
    N, H, W, C, k, pad = case
    g = torch.Generator().manual_seed(11)
    x = torch.randn(N, H, W, C, dtype=torch.float64, generator=g, requires_grad=True)
    w = torch.randn(C, 1, k, k, dtype=torch.float64, generator=g, requires_grad=True)
    b = torch.randn(C, dtype=torch.float64, generator=g, requires_grad=True)
    out = F.conv2d(x.permute(0, 3, 1, 2), w, b, stride=1, padding=pad, groups=C).permute(0, 2, 3, 1)
    go = torch.randn(out.shape, dtype=torch.float64, generator=g)
    out.backward(go)
    got = depthwise.depthwise_forward(x.detach().numpy(), w.detach().numpy(), b.detach().numpy(), pad)
    np.testing.assert_allclose(got, out.detach().numpy(), rtol=1e-12, atol=1e-12)
    gx, gw, gb = depthwise.depthwise_backward(x.detach().numpy(), w.detach().numpy(), go.numpy(), pad)
    np.testing.assert_allclose(gx, x.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(gw, w.grad.numpy().reshape(C, k, k), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(gb, b.grad.numpy(), rtol=1e-12, atol=1e-12)


def test_depthwise_one_hot_kernel_is_a_shifted_copy_and_ones_kernel_a_box_sum():
    """Pins the tap orientation (i = row, j = column) and the sign of the padding shift."""
    from oracle import depthwise
    rng = np.random.default_rng(3)
    x = rng.standard_normal((1, 6, 7, 2))
    w = np.zeros((2, 3, 3))
    w[0, 0, 2] = 1.0            # channel 0 reads the pixel one row up, one column right
    w[1, 2, 1] = 1.0            # channel 1 reads the pixel one row down
    out = depthwise.depthwise_forward(x, w, None, 1)
    want0 = np.zeros((6, 7)); want0[1:, :-1] = x[0, :-1, 1:, 0]
    want1 = np.zeros((6, 7)); want1[:-1, :] = x[0, 1:, :, 1]
    np.testing.assert_array_equal(out[0, :, :, 0], want0)
    np.testing.assert_array_equal(out[0, :, :, 1], want1)
    box = depthwise.depthwise_forward(x, np.ones((2, 3, 3)), np.array([0.5, -1.0]), 1)
    assert np.isclose(box[0, 2, 3, 0], x[0, 1:4, 2:5, 0].sum() + 0.5)
    assert np.isclose(box[0, 0, 0, 1], x[0, 0:2, 0:2, 1].sum() - 1.0)      # corner: zeros outside


def test_layer_norm_oracle_matches_torch_and_normalises_rows():
    from oracle import layer_norm
    g = torch.Generator().manual_seed(21)
    y = torch.randn(5, 7, 24, dtype=torch.float64, generator=g) * 3 + 1.5
    w, b, gamma = (torch.randn(24, dtype=torch.float64, generator=g) for _ in range(3))
    res = torch.randn(5, 7, 24, dtype=torch.float64, generator=g)
    want = res + gamma * F.layer_norm(y, (24,), w, b, 1e-6)
    got = layer_norm.layer_norm_residual(y.numpy(), w.numpy(), b.numpy(), 1e-6, gamma.numpy(), res.numpy())
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-12, atol=1e-12)
    plain = layer_norm.layer_norm_residual(y.numpy(), np.ones(24), np.zeros(24), 0.0)
    np.testing.assert_allclose(plain.mean(-1), 0.0, atol=1e-12)
    np.testing.assert_allclose((plain ** 2).mean(-1), 1.0, rtol=1e-12)          # biased variance
    shifted = layer_norm.layer_norm_residual(y.numpy() + 100.0, np.ones(24), np.zeros(24), 0.0)
    np.testing.assert_allclose(shifted, plain, atol=1e-9)


@pytest.mark.parametrize("use_gamma", [True, False])
def test_layer_norm_backward_oracle_matches_autograd_and_finite_differences(use_gamma):
    from oracle import layer_norm
    g = torch.Generator().manual_seed(22)
    y = (torch.randn(4, 6, 24, dtype=torch.float64, generator=g) * 2 + 0.7).requires_grad_(True)
    w, b, gamma = (torch.randn(24, dtype=torch.float64, generator=g).requires_grad_(True) for _ in range(3))
    res = torch.randn(4, 6, 24, dtype=torch.float64, generator=g).requires_grad_(True)
    go = torch.randn(4, 6, 24, dtype=torch.float64, generator=g)
    z = F.layer_norm(y, (24,), w, b, 1e-6)
    out = res + (gamma * z if use_gamma else z)
    leaves = [y, w, b, res] + ([gamma] if use_gamma else [])
    want = torch.autograd.grad(out, leaves, go)
    gy, gw, gb, gg = layer_norm.layer_norm_residual_backward(go.numpy(), y.detach().numpy(), w.detach().numpy(), b.detach().numpy(),
                                                             1e-6, gamma.detach().numpy() if use_gamma else None)
    np.testing.assert_allclose(gy, want[0].numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(gw, want[1].numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(gb, want[2].numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_array_equal(want[3].numpy(), go.numpy())          # the residual's gradient is grad_out itself
    if use_gamma:
        np.testing.assert_allclose(gg, want[4].numpy(), rtol=1e-10, atol=1e-11)
    else:
        assert gg is None
    # central differences of the oracle's own forward along a random direction of y
    d = torch.randn(4, 6, 24, dtype=torch.float64, generator=g).numpy()
    f = lambda t: (layer_norm.layer_norm_residual(t, w.detach().numpy(), b.detach().numpy(), 1e-6,
                                                  gamma.detach().numpy() if use_gamma else None) * go.numpy()).sum()
    h = 1e-6
    num = (f(y.detach().numpy() + h * d) - f(y.detach().numpy() - h * d)) / (2 * h)
    assert abs(num - (gy * d).sum()) < 1e-6 * max(1.0, abs(num))
    # rows of grad_y are orthogonal to the constant vector and to the normalised row (the two directions LayerNorm ignores)
    assert np.abs(gy.sum(-1)).max() < 1e-10


def test_center_feature_oracle_matches_the_reference_expression_autograd_and_limits():
    """The expression of DCNv4_op/DCNv4/modules/dcnv4.py:17-26,142-147 written with the reference's own torch calls."""
    from oracle import center_feature
    g = torch.Generator().manual_seed(23)
    y = torch.randn(2, 3, 4, 32, dtype=torch.float64, generator=g).requires_grad_(True)
    x = torch.randn(2, 3, 4, 32, dtype=torch.float64, generator=g).requires_grad_(True)
    w = (0.4 * torch.randn(2, 32, dtype=torch.float64, generator=g)).requires_grad_(True)
    b = torch.randn(2, dtype=torch.float64, generator=g).requires_grad_(True)
    go = torch.randn(2, 3, 4, 32, dtype=torch.float64, generator=g)
    s = F.linear(y, weight=w, bias=b).sigmoid()
    s = s[..., None].repeat(1, 1, 1, 1, 32 // 2).flatten(-2)
    want = y * (1 - s) + x * s
    np_ = lambda t: t.detach().numpy()
    got = center_feature.blend_forward(np_(y), np_(x), np_(w), np_(b))
    np.testing.assert_allclose(got, np_(want), rtol=1e-12, atol=1e-12)
    wy, wx, ww, wb = torch.autograd.grad(want, [y, x, w, b], go)
    gy, gx, gw, gb, gl = center_feature.blend_backward(go.numpy(), np_(y), np_(x), np_(w), np_(b))
    for a, e in ((gy, wy), (gx, wx), (gw, ww), (gb, wb)):
        np.testing.assert_allclose(a, e.numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(gl.reshape(-1, 2).sum(0), gb, rtol=1e-12)
    # limits: a very negative bias closes the gate (out = y), a very positive one opens it (out = x)
    np.testing.assert_allclose(center_feature.blend_forward(np_(y), np_(x), np_(w), np.full(2, -80.0)), np_(y), atol=1e-12)
    np.testing.assert_allclose(center_feature.blend_forward(np_(y), np_(x), np_(w), np.full(2, 80.0)), np_(x), atol=1e-12)
    # one-hot weight on a channel of group 1 only: group 0's gate is sigmoid(b0) everywhere
    w1 = np.zeros((2, 32)); w1[1, 20] = 1.0
    out = center_feature.blend_forward(np_(y), np_(x), w1, np.array([0.3, 0.0]))
    s0 = 1 / (1 + np.exp(-0.3))
    np.testing.assert_allclose(out[..., :16], np_(y)[..., :16] * (1 - s0) + np_(x)[..., :16] * s0, rtol=1e-12)
