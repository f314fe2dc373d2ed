"""Seeded random shapes through the C ABI against the CPU oracle: the shape planners (tile sizes, group chunks, window
reach and padding, workgroup sizes, level staging) see combinations no hand-picked case names.  Same tolerances as
tests/test_gpu_parity.py."""
import random

import pytest
import torch

from tests import cabi
from tests.inputs import make_dcnv4_inputs, make_fda_inputs
from tests.test_gpu_parity import FWD_TOL, GRAD_TOL

pytestmark = pytest.mark.gpu


def _random_dcn_case(rnd):
    while True:
        k = rnd.choice([(3, 3), (3, 3), (3, 3), (1, 3), (5, 5), (3, 1)])
        s = rnd.choice([(1, 1), (1, 1), (1, 1), (2, 2), (2, 1)])
        d = rnd.choice([(1, 1), (1, 1), (2, 2)])
        pad = (rnd.randint(0, k[0] // 2 * d[0] + 1), rnd.randint(0, k[1] // 2 * d[1] + 1))
        H, W = rnd.randint(1, 90), rnd.randint(1, 90)
        if H + 2 * pad[0] < d[0] * (k[0] - 1) + 1 or W + 2 * pad[1] < d[1] * (k[1] - 1) + 1:
            continue
        G = rnd.choice([1, 2, 3, 4, 5, 7, 8, 10, 14, 16])
        D = rnd.choice([8, 16, 16, 16, 32, 32, 24, 64])
        B = rnd.randint(1, 3)
        if B * H * W * G * D > 2e6:
            continue
        rc = rnd.choice([0, 0, 1]) if k == (3, 3) else 0
        return B, H, W, G, D, (*k, *s, *pad, *d), rc, rnd.choice([1.0, 0.5, 2.0]), rnd.choice([1.0, 3.0, 6.0])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("seed", range(16))
def test_dcnv4_random_shapes_match_oracle(oracle, seed, dtype):
    B, H, W, G, D, geom, rc, scale, rng = _random_dcn_case(random.Random(1000 + seed))
    print(f"case B={B} {H}x{W} G={G} D={D} geom={geom} remove_center={rc} scale={scale} range={rng} dtype {dtype}", flush=True)
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, *geom, remove_center=rc, offset_range=rng, seed=seed, dtype=dtype)
    args = (*geom, G, D, scale, rc)
    want = oracle.dcnv4_forward(cabi.f64(v), cabi.f64(om), *args, coord_f32=True)
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *args, coord_f32=True)
    out = cabi.dcnv4_forward(v.cuda(), om.cuda(), geom, G, D, scale, rc)
    gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), geom, G, D, scale, rc)
    torch.cuda.synchronize()
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    cabi.assert_close(gv, wgv, *GRAD_TOL[dtype], what="grad_value")
    cabi.assert_close(gom, wgom, *GRAD_TOL[dtype], what="grad_offset_mask")
    if seed % 2 == 0:       # every other shape also with the softmax over a group's modulation scalars
        want = oracle.dcnv4_forward(cabi.f64(v), cabi.f64(om), *args, softmax=True, coord_f32=True)
        wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *args, softmax=True, coord_f32=True)
        out = cabi.dcnv4_forward(v.cuda(), om.cuda(), geom, G, D, scale, rc, softmax=1)
        gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), geom, G, D, scale, rc, softmax=1)
        torch.cuda.synchronize()
        cabi.assert_close(out, want, *FWD_TOL[dtype], what="output, softmax")
        cabi.assert_close(gv, wgv, *GRAD_TOL[dtype], what="grad_value, softmax")
        cabi.assert_close(gom, wgom, *GRAD_TOL[dtype], what="grad_offset_mask, softmax")


def _random_fda_case(rnd):
    while True:
        L = rnd.randint(1, 5)
        h0, w0 = rnd.randint(2, 48), rnd.randint(2, 48)
        shapes = [(max(1, h0 >> l), max(1, w0 >> l)) for l in range(L)]
        K = rnd.choice([4, 4, 8, 2, 3])
        if L * K > 32:
            continue
        G, D = rnd.choice([1, 2, 4, 8, 8, 3]), rnd.choice([8, 16, 32, 32, 32, 64, 24, 40, 96, 128])
        Q = rnd.choice([None, None, rnd.randint(1, 3000)])
        return rnd.randint(1, 3), shapes, G, D, K, Q, rnd.choice([(0.0, 1.0), (-0.2, 1.2), (0.3, 0.7)])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("options", [dict(), dict(fda_order="heads", fda_stage="on"), dict(scatter="atomic")],
                         ids=["library_choice", "staged_levels", "atomic_scatter"])
@pytest.mark.parametrize("seed", range(8))
def test_flash_deform_attn_random_shapes_match_oracle(oracle, seed, options, dtype):
    from dcnv4_amd import ext
    B, shapes, G, D, K, Q, (lo, hi) = _random_fda_case(random.Random(2000 + seed))
    print(f"case B={B} levels={shapes} G={G} D={D} K={K} Q={Q} loc=({lo},{hi}) options={options} dtype {dtype}", flush=True)
    v, shp, st, sla, go = make_fda_inputs(B, shapes, G, D, K, Q, seed=seed, dtype=dtype, loc_lo=lo, loc_hi=hi)
    want = oracle.flash_deform_attn_forward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), K, coord_f32=True)
    wgv, wgs = oracle.flash_deform_attn_backward(cabi.f64(v), shp.numpy(), st.numpy(), cabi.f64(sla), cabi.f64(go), K, coord_f32=True)
    vd, sd, gd, shd, std = v.cuda(), sla.cuda(), go.cuda(), shp.cuda(), st.cuda()
    with ext.launch_options(**options):
        out = cabi.fda_forward(vd, shd, std, sd, K)
        gv, gs = cabi.fda_backward(vd, shd, std, sd, gd, K)
    torch.cuda.synchronize()
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    cabi.assert_close(gv, wgv, *GRAD_TOL[dtype], what="grad_value")
    cabi.assert_close(gs, wgs, *GRAD_TOL[dtype], what="grad_sampling_loc_attn")
