"""GPU parity of the layer-level kernels around the two operators, through the C ABI, against the CPU oracles: the
block tail's backward, the centre-feature blend, and flash deformable attention on un-packed rows."""
import zlib

import numpy as np
import pytest
import torch

from tests import cabi
from tests.inputs import make_fda_inputs
from tests.test_gpu_parity import FDA_CASES, FWD_TOL, GRAD_TOL

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def oracle():
    from oracle import c_oracle
    return c_oracle


# ---------------------------------------------------------------- block tail, backward
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("rows,C", [(2 * 56 * 56, 112), (3000, 64), (300, 224), (77, 448), (33, 896), (5, 8), (3, 4096), (1, 2048),
                                    (130, 1024), (7, 40), (4099, 1280)])
def test_layer_norm_residual_backward_matches_oracle(rows, C, dtype):
    from oracle import layer_norm
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    if C % vec or C // vec > 512:
        pytest.skip("channel count is not a whole number of 16-byte vectors for this dtype, or more than 512 of them")
    g = torch.Generator().manual_seed(rows + C)
    y = (torch.randn(rows, C, generator=g) * 2 + 0.5).to(dtype)
    go = torch.randn(rows, C, generator=g).to(dtype)
    w = (1 + 0.3 * torch.randn(C, generator=g)).to(dtype)
    b = (0.2 * torch.randn(C, generator=g)).to(dtype)
    gamma = torch.randn(C, generator=g).to(dtype)
    print(f"layer norm backward rows {rows} C {C} {dtype}", flush=True)
    for use_gamma in (True, False):
        wy, ww, wb, wg = layer_norm.layer_norm_residual_backward(cabi.f64(go), cabi.f64(y), cabi.f64(w), cabi.f64(b), 1e-6,
                                                                 cabi.f64(gamma) if use_gamma else None)
        gy, gw, gb, gg = cabi.layer_norm_residual_backward(go.cuda(), y.cuda(), w.cuda(), b.cuda(), gamma.cuda() if use_gamma else None, 1e-6)
        rtol, atol = GRAD_TOL[dtype]
        cabi.assert_close(gy, wy, rtol, atol, what=f"grad_input gamma={use_gamma}")
        # column sums over `rows` terms: the absolute tolerance follows the size of the sum
        for got, want, what in ((gw, ww, "grad_weight"), (gb, wb, "grad_bias")) + (((gg, wg, "grad_gamma"),) if use_gamma else ()):
            cabi.assert_close(got, want, rtol, atol * max(1.0, float(np.abs(want).max())), what=f"{what} gamma={use_gamma}")
        assert (gg is None) == (not use_gamma)
    # parameter gradients not asked for: grad_input unchanged
    gy2, gw2, gb2, gg2 = cabi.layer_norm_residual_backward(go.cuda(), y.cuda(), w.cuda(), b.cuda(), None, 1e-6, want_params=False)
    assert gw2 is None and gb2 is None and gg2 is None and torch.equal(gy2, gy)
    # same bits on a second call (fixed summation order)
    again = cabi.layer_norm_residual_backward(go.cuda(), y.cuda(), w.cuda(), b.cuda(), None, 1e-6)
    assert torch.equal(again[1], gw) and torch.equal(again[2], gb)


def test_layer_norm_function_gradients_match_autograd_of_the_torch_expression():
    from dcnv4_amd.functions import layer_norm_residual
    torch.manual_seed(3)
    norm = torch.nn.LayerNorm(112, eps=1e-6).cuda()
    with torch.no_grad():
        norm.weight.normal_(1, 0.2)
        norm.bias.normal_(0, 0.2)
    gamma = torch.randn(112, device="cuda", requires_grad=True)
    y = torch.randn(4, 9, 9, 112, device="cuda", requires_grad=True)
    x = torch.randn(4, 9, 9, 112, device="cuda", requires_grad=True)
    go = torch.randn(4, 9, 9, 112, device="cuda")
    out = layer_norm_residual(y, norm, gamma, x)
    got = torch.autograd.grad(out, [y, x, gamma, norm.weight, norm.bias], go)
    want = torch.autograd.grad(x + gamma * norm(y), [y, x, gamma, norm.weight, norm.bias], go)
    for a, e in zip(got, want):
        assert torch.allclose(a, e, rtol=1e-4, atol=1e-4 * float(e.abs().max()))


# ---------------------------------------------------------------- centre-feature blend
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("rows,C,G", [(2 * 56 * 56, 64, 4), (500, 112, 7), (300, 128, 8), (77, 512, 32), (33, 1280, 80), (5, 16, 1),
                                      (9, 64, 2), (3, 4096, 8), (130, 448, 28)])
def test_center_feature_blend_matches_oracle(rows, C, G, dtype):
    from oracle import center_feature
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    if (C // G) % vec or C // vec > 512:
        pytest.skip("group width is not a whole number of 16-byte vectors for this dtype")
    g = torch.Generator().manual_seed(rows + C + G)
    y = torch.randn(rows, C, generator=g).to(dtype)
    x = torch.randn(rows, C, generator=g).to(dtype)
    go = torch.randn(rows, C, generator=g).to(dtype)
    w = (torch.randn(G, C, generator=g) * (2.0 / C ** 0.5)).to(dtype)
    b = (0.5 * torch.randn(G, generator=g)).to(dtype)
    print(f"centre-feature blend rows {rows} C {C} G {G} {dtype}", flush=True)
    want = center_feature.blend_forward(cabi.f64(y), cabi.f64(x), cabi.f64(w), cabi.f64(b))
    wy, wx, _, _, wl = center_feature.blend_backward(cabi.f64(go), cabi.f64(y), cabi.f64(x), cabi.f64(w), cabi.f64(b))
    out = cabi.center_feature_blend_forward(y.cuda(), x.cuda(), w.cuda(), b.cuda())
    gy, gx, gl = cabi.center_feature_blend_backward(go.cuda(), y.cuda(), x.cuda(), w.cuda(), b.cuda())
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    rtol, atol = GRAD_TOL[dtype]
    cabi.assert_close(gy, wy, rtol, atol, what="grad_sampled")
    cabi.assert_close(gx, wx, rtol, atol, what="grad_projected")
    cabi.assert_close(gl, wl, 1e-3, 1e-4 * max(1.0, float(np.abs(wl).max())), what="grad_gate_logits")


def test_center_feature_blend_rejects_group_widths_that_split_a_vector():
    y = torch.zeros(4, 24, device="cuda", dtype=torch.float16)
    w = torch.zeros(6, 24, device="cuda", dtype=torch.float16)
    b = torch.zeros(6, device="cuda", dtype=torch.float16)
    with pytest.raises(ValueError, match="group width"):
        cabi.center_feature_blend_forward(y, y, w, b)
    with pytest.raises(ValueError, match="equal groups"):
        cabi.center_feature_blend_forward(y, y, torch.zeros(5, 24, device="cuda", dtype=torch.float16), b[:5].contiguous())


def test_center_feature_function_gradients_match_autograd_of_the_reference_expression():
    from dcnv4_amd.functions import CenterFeatureBlendFunction
    torch.manual_seed(5)
    y, x = (torch.randn(2, 7, 5, 64, device="cuda", requires_grad=True) for _ in range(2))
    w = (0.3 * torch.randn(4, 64, device="cuda")).requires_grad_(True)
    b = torch.randn(4, device="cuda", requires_grad=True)
    go = torch.randn(2, 7, 5, 64, device="cuda")
    got = torch.autograd.grad(CenterFeatureBlendFunction.apply(y, x, w, b), [y, x, w, b], go)
    s = torch.nn.functional.linear(y, w, b).sigmoid()
    s = s[..., None].repeat(1, 1, 1, 1, 16).flatten(-2)
    want = torch.autograd.grad(y * (1 - s) + x * s, [y, x, w, b], go)
    for a, e in zip(got, want):
        assert torch.allclose(a, e, rtol=1e-4, atol=1e-4 * max(1.0, float(e.abs().max())))


def test_center_feature_function_takes_parameters_that_are_views_into_a_flat_buffer():
    """Flattened / fused parameter storage: weight and bias start 8 bytes into a 16-byte unit, where the
    reference's F.linear works (DCNv4_op/DCNv4/modules/dcnv4.py:17-26)."""
    from dcnv4_amd.functions import CenterFeatureBlendFunction
    torch.manual_seed(6)
    flat = torch.randn(2 + 4 * 64 + 4, device="cuda")
    w, b = flat[2:2 + 256].view(4, 64), flat[258:262]
    assert w.data_ptr() % 16 == 8 and b.data_ptr() % 16 == 8
    y, x = torch.randn(3, 5, 64, device="cuda"), torch.randn(3, 5, 64, device="cuda")
    got = CenterFeatureBlendFunction.apply(y, x, w, b)
    s = torch.nn.functional.linear(y, w, b).sigmoid()[..., None].repeat(1, 1, 1, 16).flatten(-2)
    assert torch.allclose(got, y * (1 - s) + x * s, rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------- attention on un-packed rows
@pytest.mark.parametrize("loc_fp32", [True, False], ids=["loc_fp32", "loc_like_value"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("name", ["detr_small_4lvl_k4", "k8_one_level", "five_levels", "k3_generic_points", "d6_heads5", "one_query",
                                  "d64_two_levels", "decoder_few_queries"])
def test_flash_deform_attn_split_rows_match_oracle_on_fp16_rounded_locations(oracle, name, dtype, loc_fp32):
    """The oracle sees what the reference's module would have packed: locations rounded to fp16, then the logits
    (DCNv4_op/DCNv4/modules/flash_deform_attn.py:132-133)."""
    B, shapes, G, D, K, Q, (lo, hi) = FDA_CASES[name]
    print(f"split case {name} dtype {dtype} loc_fp32 {loc_fp32}", flush=True)
    v, shp, st, sla, go = make_fda_inputs(B, shapes, G, D, K, Q, seed=zlib.crc32(name.encode()) % 1000, dtype=torch.float32,
                                          loc_lo=lo, loc_hi=hi)
    LK = len(shapes) * K
    loc = sla[..., : 2 * LK].contiguous().to(torch.float32 if loc_fp32 else dtype)
    logits = sla[..., 2 * LK:].contiguous().to(dtype)
    v, go = v.to(dtype), go.to(dtype)
    packed = np.concatenate([cabi.f64(loc.half()), cabi.f64(logits)], -1)
    want = oracle.flash_deform_attn_forward(cabi.f64(v), shp.numpy(), st.numpy(), packed, K, coord_f32=True)
    wgv, wgs = oracle.flash_deform_attn_backward(cabi.f64(v), shp.numpy(), st.numpy(), packed, cabi.f64(go), K, coord_f32=True)
    args = (v.cuda(), shp.cuda(), st.cuda(), loc.cuda(), logits.cuda())
    out = cabi.fda_forward_split(*args, K)
    gv, gloc, glog = cabi.fda_backward_split(*args, go.cuda(), K)
    torch.cuda.synchronize()
    assert gloc.dtype == loc.dtype and glog.dtype == dtype
    cabi.assert_close(out, want, *FWD_TOL[dtype], what="output")
    cabi.assert_close(gv, wgv, *GRAD_TOL[dtype], what="grad_value")
    cabi.assert_close(gloc, wgs[..., : 2 * LK], *GRAD_TOL[dtype], what="grad_sampling_locations")
    cabi.assert_close(glog, wgs[..., 2 * LK:], *GRAD_TOL[dtype], what="grad_attention_logits")
    # and the packed entry point on the packed tensor gives the same bits for fp16-representable rows
    if not loc_fp32 and dtype == torch.float16:
        sla16 = torch.cat([loc, logits], -1).cuda()
        assert torch.equal(cabi.fda_forward(v.cuda(), shp.cuda(), st.cuda(), sla16, K), out)


def test_flash_deform_attn_split_head_major_order(oracle):
    """A value image large enough for the one-head-per-workgroup order, rows un-packed."""
    B, shapes, G, D, K = 1, [(96, 128), (48, 64)], 8, 32, 4
    v, shp, st, sla, go = make_fda_inputs(B, shapes, G, D, K, 700, seed=8, dtype=torch.float32)
    LK = 2 * K
    loc, logits = sla[..., : 2 * LK].contiguous(), sla[..., 2 * LK:].contiguous().half()
    v, go = v.half(), go.half()
    packed = np.concatenate([cabi.f64(loc.half()), cabi.f64(logits)], -1)
    want = oracle.flash_deform_attn_forward(cabi.f64(v), shp.numpy(), st.numpy(), packed, K, coord_f32=True)
    wgv, wgs = oracle.flash_deform_attn_backward(cabi.f64(v), shp.numpy(), st.numpy(), packed, cabi.f64(go), K, coord_f32=True)
    args = (v.cuda(), shp.cuda(), st.cuda(), loc.cuda(), logits.cuda())
    out = cabi.fda_forward_split(*args, K)
    gv, gloc, glog = cabi.fda_backward_split(*args, go.cuda(), K)
    cabi.assert_close(out, want, *FWD_TOL[torch.float16], what="output")
    cabi.assert_close(gv, wgv, *GRAD_TOL[torch.float16], what="grad_value")
    cabi.assert_close(gloc, wgs[..., : 2 * LK], 1e-2, 1e-2 * float(np.abs(wgs[..., : 2 * LK]).max()), what="grad_sampling_locations")
    cabi.assert_close(glog, wgs[..., 2 * LK:], *GRAD_TOL[torch.float16], what="grad_attention_logits")


def test_flash_deform_attn_split_function_equals_the_reference_modules_half_and_cat_graph():
    """fp32 locations through the split Function against the graph the reference's module builds with torch ops -
    `.half()`, `cat`, the packed Function (DCNv4_op/DCNv4/modules/flash_deform_attn.py:132-133): autograd hands the
    locations' gradient back through an fp16 tensor, so it is an fp16-rounded value in an fp32 tensor, bit for bit.
    Gradients beyond the fp16 range (they would be infinities on both sides) are not covered: parity unpinned there."""
    from dcnv4_amd.functions import FlashDeformAttnFunction, FlashDeformAttnSplitFunction
    B, shapes, G, D, K = 2, [(20, 24), (10, 12), (5, 6)], 4, 32, 4
    v, shp, st, sla, go = make_fda_inputs(B, shapes, G, D, K, 150, seed=21, dtype=torch.float32)
    LK = len(shapes) * K
    v, go = v.cuda().half(), (300.0 * go).cuda().half()
    shp, st = shp.cuda(), st.cuda()
    loc = sla[..., : 2 * LK].contiguous().cuda().requires_grad_(True)              # fp32
    logits = sla[..., 2 * LK:].contiguous().cuda().half().requires_grad_(True)
    out = FlashDeformAttnSplitFunction.apply(v, shp, st, loc, logits, 64, K)
    g_loc, g_logits = torch.autograd.grad(out, [loc, logits], go)
    loc2, logits2 = loc.detach().clone().requires_grad_(True), logits.detach().clone().requires_grad_(True)
    out2 = FlashDeformAttnFunction.apply(v, shp, st, torch.cat([loc2.half(), logits2], -1), 64, K)
    w_loc, w_logits = torch.autograd.grad(out2, [loc2, logits2], go)
    assert g_loc.dtype == torch.float32 and w_loc.dtype == torch.float32
    assert torch.equal(out, out2)
    assert torch.equal(g_loc, w_loc), f"largest difference {(g_loc - w_loc).abs().max().item()}"
    assert torch.equal(g_logits, w_logits)
    assert torch.equal(g_loc, g_loc.half().float())          # every value is fp16-representable


def test_flash_deform_attn_split_rejects_mismatched_location_dtype():
    v = torch.zeros(1, 16, 2, 16, device="cuda")
    shp = torch.tensor([[4, 4]], device="cuda")
    st = torch.tensor([0], device="cuda")
    with pytest.raises(RuntimeError, match="fp32 or of the value's dtype"):
        cabi.fda_forward_split(v, shp, st, torch.zeros(1, 3, 2, 8, device="cuda", dtype=torch.float16),
                               torch.zeros(1, 3, 2, 4, device="cuda"), 4)


def test_stream_copy_copies_and_rejects_odd_sizes():
    from dcnv4_amd import ext
    src = torch.randn(1 << 20, device="cuda")
    dst = torch.zeros_like(src)
    ext.stream_copy(src, dst)
    assert torch.equal(src, dst)
    small = torch.arange(12, device="cuda", dtype=torch.float32)         # 48 bytes: three vectors, less than one workgroup
    out = torch.zeros_like(small)
    ext.stream_copy(small, out)
    assert torch.equal(small, out)
    with pytest.raises(ValueError, match="multiple of 16"):
        ext.stream_copy(torch.zeros(3, device="cuda"), torch.zeros(3, device="cuda"))


def test_lds_read_probe_orders_its_patterns():
    """The measurement aid behind the LDS-pattern figures: all lanes on one 16-byte slot must cost several times what
    16 lanes on 16 different slots cost, and a random gather lies in between."""
    from dcnv4_amd import ext
    best = min(ext.lds_read_probe(1, 2000) for _ in range(3))
    gather = min(ext.lds_read_probe(3, 2000) for _ in range(3))
    worst = min(ext.lds_read_probe(4, 2000) for _ in range(3))
    print(f"LDS probe: spread {best:.2f}, gather {gather:.2f}, one slot {worst:.2f} ticks per read", flush=True)
    assert 0 < best < gather < worst and worst > 3 * best
    with pytest.raises(ValueError, match="pattern"):
        ext.lds_read_probe(9)
