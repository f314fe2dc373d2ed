"""GPU tests of the Python surface (autograd Functions, nn.Modules) and of size-independent
properties at the benchmark's full sizes, where the CPU oracle would take too long:
adjoint identities (the operator is linear in value and in the modulation), bit-reproducibility,
batch chunking, non-finite gradients, HIP-graph replay."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import torch_core
from tests import cabi
from tests.inputs import make_dcnv4_inputs, make_fda_inputs

pytestmark = pytest.mark.gpu
GEOM = (3, 3, 1, 1, 1, 1, 1, 1)


def _rel_err(a, b):
    a, b = a.double(), b.double()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


class DepthwiseOnCpu:
    """The reference's formulation of the offset_mask_dw layer (modules/dcnv4.py:121-123) for CPU re-evaluation."""

    @staticmethod
    def apply(inp, weight, bias, pad):
        return F.conv2d(inp.permute(0, 3, 1, 2), weight, bias, stride=1, padding=pad, groups=inp.shape[-1]).permute(0, 2, 3, 1)


def test_dcnv4_function_autograd_matches_grid_sample_autograd():
    import dcnv4_amd
    B, H, W, G, D = 2, 12, 10, 4, 16
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, seed=4)
    vd, omd = v.cuda().requires_grad_(True), om.cuda().requires_grad_(True)
    out = dcnv4_amd.DCNv4Function.apply(vd, omd, *GEOM, G, D, 1.0, 256, 0)
    out.backward(go.cuda())
    v64, om64 = v.double().requires_grad_(True), om.double().requires_grad_(True)
    ref = torch_core.dcnv4_core_torch(v64, om64, *GEOM, G, D, 1.0)
    ref.backward(go.double())
    assert out.shape == ref.shape and out.dtype == torch.float32
    assert _rel_err(out.cpu(), ref.detach()) < 1e-4
    assert _rel_err(vd.grad.cpu(), v64.grad) < 1e-3
    assert _rel_err(omd.grad.cpu(), om64.grad) < 1e-3
    assert vd.grad.dtype == torch.float32 and omd.grad.shape == om.shape


def test_flash_deform_attn_function_autograd_matches_grid_sample_autograd():
    import dcnv4_amd
    shapes = [(10, 12), (5, 6), (3, 3)]
    v, shp, st, sla, go = make_fda_inputs(2, shapes, 4, 32, 4, Q=60, seed=6)
    vd, sd = v.cuda().requires_grad_(True), sla.cuda().requires_grad_(True)
    out = dcnv4_amd.FlashDeformAttnFunction.apply(vd, shp.cuda(), st.cuda(), sd, 64, 4)
    out.backward(go.cuda())
    v64, s64 = v.double().requires_grad_(True), sla.double().requires_grad_(True)
    ref = torch_core.msda_core_torch(v64, shapes, st.tolist(), s64, 4)
    ref.backward(go.double())
    assert out.shape == (2, 60, 128)
    assert _rel_err(out.cpu(), ref.detach()) < 1e-4
    assert _rel_err(vd.grad.cpu(), v64.grad) < 1e-3
    assert _rel_err(sd.grad.cpu(), s64.grad) < 1e-3


@pytest.mark.parametrize("kwargs", [dict(), dict(dw_kernel_size=3, center_feature_scale=True, remove_center=True, offset_scale=0.5),
                                    dict(without_pointwise=True, output_bias=False)])
def test_dcnv4_module_matches_a_reference_built_from_torch_ops(kwargs):
    import dcnv4_amd
    torch.manual_seed(0)
    C, G, H, W, N = 64, 4, 9, 7, 2
    m = dcnv4_amd.DCNv4(channels=C, group=G, **kwargs)
    with torch.no_grad():       # the module initialises offsets to zero; give them something to do
        m.offset_mask.weight.normal_(0, 0.3)
        m.offset_mask.bias.normal_(0, 0.5)
        if m.center_feature_scale:
            m.center_feature_scale_proj_weight.normal_(0, 0.2)
    x = torch.randn(N, H * W, C)

    def reference(mod, inp):
        xx = inp if mod.without_pointwise else mod.value_proj(inp)
        xx = xx.reshape(N, H, W, -1)
        src = inp
        if mod.dw_kernel_size is not None:
            src = mod.offset_mask_dw(inp.view(N, H, W, C).permute(0, 3, 1, 2)).permute(0, 2, 3, 1).reshape(N, H * W, C)
        om = mod.offset_mask(src).reshape(N, H, W, -1)
        y = torch_core.dcnv4_core_torch(xx, om, mod.kernel_size, mod.kernel_size, mod.stride, mod.stride, mod.pad, mod.pad,
                                        mod.dilation, mod.dilation, mod.group, mod.group_channels, mod.offset_scale,
                                        mod.remove_center)
        if mod.center_feature_scale:
            s = F.linear(y, mod.center_feature_scale_proj_weight, mod.center_feature_scale_proj_bias).sigmoid()
            s = s[..., None].repeat(1, 1, 1, 1, mod.channels // mod.group).flatten(-2)
            y = y * (1 - s) + xx * s
        y = y.view(N, H * W, -1)
        return y if mod.without_pointwise else mod.output_proj(y)

    want = reference(m, x)
    xg = x.clone().requires_grad_(True)
    reference(m, xg).sum().backward()
    md = m.cuda()
    xd = x.cuda().requires_grad_(True)
    got = md(xd, shape=(H, W), level_idx=0)
    got.sum().backward()
    assert _rel_err(got.detach().cpu(), want.detach()) < 2e-4
    assert _rel_err(xd.grad.cpu(), xg.grad) < 2e-3


def test_flash_deform_attn_module_matches_a_reference_built_from_torch_ops():
    import dcnv4_amd
    torch.manual_seed(1)
    shapes = [(8, 8), (4, 4)]
    m = dcnv4_amd.FlashDeformAttn(d_model=64, n_levels=2, n_heads=4, n_points=4)
    with torch.no_grad():
        m.attention_weights.weight.normal_(0, 0.2)
        m.sampling_offsets.weight.normal_(0, 0.05)
    N, Lq, S = 2, 30, 80
    q, feat = torch.randn(N, Lq, 64), torch.randn(N, S, 64)
    ref_pts = torch.rand(N, Lq, 2, 2)
    shp = torch.tensor(shapes)
    starts = torch.tensor([0, 64])
    pad = torch.zeros(N, S, dtype=torch.bool)
    pad[0, -5:] = True
    value = m.value_proj(feat).masked_fill(pad[..., None], 0.0).view(N, S, 4, 16)
    off = m.sampling_offsets(q).view(N, Lq, 4, 2, 4, 2)
    logits = m.attention_weights(q).view(N, Lq, 4, 8)
    norm = torch.stack([shp[..., 1], shp[..., 0]], -1)
    loc = ref_pts[:, :, None, :, None, :] + off / norm[None, None, None, :, None, :]
    sla = torch.cat([loc.flatten(-3).half().float(), logits], -1)       # locations pass through fp16 in the module
    want = m.output_proj(torch_core.msda_core_torch(value, shapes, [0, 64], sla, 4))
    md = m.cuda()
    got = md(q.cuda(), ref_pts.cuda(), feat.cuda(), shp.cuda(), starts.cuda(), pad.cuda())
    assert _rel_err(got.detach().cpu(), want.detach()) < 2e-4


def test_backward_repeats_to_the_rounding_of_fp32_sums():
    """grad_offset_mask has a fixed summation order: same bits every time.  grad_value sums each cell's terms in fp32
    in the order the hardware ranked them (like the reference's atomics): repeats agree to fp32 rounding, far inside
    one unit of the fp16 result."""
    B, H, W, G, D = 4, 28, 28, 8, 16
    v, om, go = (t.cuda() for t in make_dcnv4_inputs(B, H, W, G, D, offset_range=3.0, seed=8, dtype=torch.float32))
    first = cabi.dcnv4_backward(v, om, go, GEOM, G, D, 1.0)
    for _ in range(3):
        again = cabi.dcnv4_backward(v, om, go, GEOM, G, D, 1.0)
        assert torch.equal(first[1], again[1])
        assert (first[0] - again[0]).abs().max().item() <= 2e-5 and _rel_err(first[0], again[0]) < 1e-6


def test_nan_in_grad_output_propagates_like_the_oracle(oracle):
    B, H, W, G, D = 1, 10, 10, 2, 16
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, seed=9)
    go[0, 4, 5, 3] = float("nan")
    go[0, 2, 2, 20] = float("inf")
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *GEOM, G, D, 1.0, coord_f32=True)
    gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), GEOM, G, D, 1.0)
    gv, gom = cabi.f64(gv), cabi.f64(gom)
    assert np.array_equal(np.isfinite(gv), np.isfinite(wgv)) and np.array_equal(np.isnan(gv), np.isnan(wgv))
    ok = np.isfinite(wgv)
    np.testing.assert_allclose(gv[ok], wgv[ok], rtol=1e-3, atol=1e-4)
    assert np.array_equal(np.isfinite(gom), np.isfinite(wgom))


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.float16, 3e-3)], ids=["fp32", "fp16"])
def test_dcnv4_adjoint_identities_at_full_benchmark_size(dtype, tol):
    # out is linear in value and in the modulation scalars, so with g = grad_out:
    #   <g, out> = <grad_value, value> = <grad_mask, mask>          (B=64, 56x56, C=64, G=4)
    torch.manual_seed(3)
    B, H, W, G, D, K = 64, 56, 56, 4, 16, 9
    dev = "cuda"
    v = torch.randn(B, H, W, G * D, device=dev).to(dtype)
    body = torch.cat([(torch.rand(B, H, W, G, 2 * K, device=dev) * 6 - 3), torch.randn(B, H, W, G, K, device=dev)], -1)
    om = torch.zeros(B, H, W, 112, device=dev)
    om[..., :108] = body.reshape(B, H, W, 108)
    om = om.to(dtype)
    g = torch.randn(B, H, W, G * D, device=dev).to(dtype)
    out = cabi.dcnv4_forward(v, om, GEOM, G, D, 1.0)
    gv, gom = cabi.dcnv4_backward(v, om, g, GEOM, G, D, 1.0)
    lhs = (g.double() * out.double()).sum()
    by_value = (gv.double() * v.double()).sum()
    mask = om[..., :108].reshape(B, H, W, G, 27)[..., 18:].double()
    gmask = gom[..., :108].reshape(B, H, W, G, 27)[..., 18:].double()
    by_mask = (gmask * mask).sum()
    scale = (g.double().abs() * out.double().abs()).sum()
    assert abs(float(lhs - by_value)) / float(scale) < tol
    assert abs(float(lhs - by_mask)) / float(scale) < tol
    assert (gom[..., 108:] == 0).all()


@pytest.mark.parametrize("B,H,W,G,off,dtype,tol", [
    (2, 256, 256, 10, 4.0, torch.float16, 3e-3),      # dense-prediction stage 1 (1024x1024 image, FlashInternImage-L width)
    (128, 56, 56, 7, 3.0, torch.float16, 3e-3),       # FlashInternImage-B stage 1 at batch 128
    (64, 7, 7, 32, 3.0, torch.float32, 2e-5),         # smallest classification stage: most groups per pixel
], ids=["dense_256x256_g10", "b_stage1_batch128", "t_stage4_fp32"])
def test_dcnv4_adjoint_identities_at_the_other_benchmark_shapes(B, H, W, G, off, dtype, tol):
    torch.manual_seed(6)
    D, K, dev = 16, 9, "cuda"
    P = G * K * 3
    P_pad = (P + 7) // 8 * 8
    v = torch.randn(B, H, W, G * D, device=dev).to(dtype)
    body = torch.cat([(torch.rand(B, H, W, G, 2 * K, device=dev) * 2 - 1) * off, torch.randn(B, H, W, G, K, device=dev)], -1)
    om = torch.zeros(B, H, W, P_pad, device=dev)
    om[..., :P] = body.reshape(B, H, W, P)
    om = om.to(dtype)
    g = torch.randn(B, H, W, G * D, device=dev).to(dtype)
    out = cabi.dcnv4_forward(v, om, GEOM, G, D, 1.0)
    gv, gom = cabi.dcnv4_backward(v, om, g, GEOM, G, D, 1.0)
    lhs = (g.double() * out.double()).sum()
    by_value = (gv.double() * v.double()).sum()
    mask = om[..., :P].reshape(B, H, W, G, 3 * K)[..., 2 * K:].double()
    gmask = gom[..., :P].reshape(B, H, W, G, 3 * K)[..., 2 * K:].double()
    scale = (g.double().abs() * out.double().abs()).sum()
    assert abs(float(lhs - by_value)) / float(scale) < tol
    assert abs(float(lhs - (gmask * mask).sum())) / float(scale) < tol
    assert (gom[..., P:] == 0).all()


def test_dcnv4_benchmark_stage_shape_matches_the_oracle_element_by_element(oracle):
    """56x56, C=64, G=4 with the benchmark's offset range, a quarter of its batch: every element against the oracle."""
    B, H, W, G, D = 16, 56, 56, 4, 16
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, offset_range=3.0, seed=21, dtype=torch.float16)
    want = oracle.dcnv4_forward(cabi.f64(v), cabi.f64(om), *GEOM, G, D, 1.0, coord_f32=True)
    wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *GEOM, G, D, 1.0, coord_f32=True)
    out = cabi.dcnv4_forward(v.cuda(), om.cuda(), GEOM, G, D, 1.0)
    gv, gom = cabi.dcnv4_backward(v.cuda(), om.cuda(), go.cuda(), GEOM, G, D, 1.0)
    cabi.assert_close(out, want, 1e-2, 1e-3, what="output")
    cabi.assert_close(gv, wgv, 1e-2, 1e-2, what="grad_value")
    cabi.assert_close(gom, wgom, 1e-2, 1e-2, what="grad_offset_mask")


def test_flash_deform_attn_adjoint_identity_at_full_benchmark_size():
    torch.manual_seed(4)
    shapes = [(128, 128), (64, 64), (32, 32), (16, 16)]
    B, G, D, L, K = 4, 8, 32, 4, 4
    N = sum(h * w for h, w in shapes)
    dev = "cuda"
    shp = torch.tensor(shapes, device=dev)
    sizes = [h * w for h, w in shapes]
    st = torch.tensor([sum(sizes[:i]) for i in range(L)], device=dev)
    v = torch.randn(B, N, G, D, device=dev)
    sla = torch.cat([torch.rand(B, N, G, L * K * 2, device=dev), torch.randn(B, N, G, L * K, device=dev)], -1)
    g = torch.randn(B, N, G * D, device=dev)
    out = cabi.fda_forward(v, shp, st, sla, K)
    gv, gs = cabi.fda_backward(v, shp, st, sla, g, K)
    lhs = (g.double() * out.double()).sum()
    rhs = (gv.double() * v.double()).sum()
    scale = (g.double().abs() * out.double().abs()).sum()
    assert abs(float(lhs - rhs)) / float(scale) < 2e-5
    # softmax Jacobian rows sum to zero
    assert float(gs[..., 2 * L * K:].double().sum(-1).abs().max()) < 1e-3


def test_batches_beyond_the_32_bit_addressing_span_are_chunked_consistently():
    # value of 2.7 GB: more than one launch can address with 32-bit buffer offsets
    torch.manual_seed(5)
    B, H, W, G, D, K = 20, 512, 512, 8, 16, 9
    dev = "cuda"
    v = torch.randn(B, H, W, G * D, device=dev)
    om = torch.zeros(B, H, W, 216, device=dev)
    om[..., : 2 * K * G] = torch.rand(B, H, W, 2 * K * G, device=dev) * 4 - 2      # not the packing order: any values do
    om[..., 2 * K * G:] = torch.randn(B, H, W, K * G, device=dev)
    out = cabi.dcnv4_forward(v, om, GEOM, G, D, 1.0)
    for lo, hi in [(0, 3), (9, 12), (17, 20)]:
        part = cabi.dcnv4_forward(v[lo:hi].contiguous(), om[lo:hi].contiguous(), GEOM, G, D, 1.0)
        assert torch.equal(out[lo:hi], part)
    del out
    g = torch.randn(B, H, W, G * D, device=dev)
    gv, gom = cabi.dcnv4_backward(v, om, g, GEOM, G, D, 1.0)
    pv, pom = cabi.dcnv4_backward(v[9:12].contiguous(), om[9:12].contiguous(), g[9:12].contiguous(), GEOM, G, D, 1.0)
    assert torch.equal(gom[9:12], pom)
    assert _rel_err(gv[9:12], pv) < 1e-6       # fp32 sums in hardware order


def test_forward_and_backward_replay_correctly_from_a_hip_graph():
    B, H, W, G, D = 4, 20, 20, 4, 16
    v, om, go = (t.cuda() for t in make_dcnv4_inputs(B, H, W, G, D, seed=10, dtype=torch.float16))
    import dcnv4_amd
    from dcnv4_amd import ext
    eager_out = ext.dcnv4_forward(v, om, *GEOM, G, D, 1.0, 64, 0, 0, 0, False)
    eager_gv, eager_gom = ext.dcnv4_backward(v, om, *GEOM, G, D, 1.0, 64, go, 0, 0, 0, False)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # warm up on the capture stream (allocator, lazy init)
        ext.dcnv4_forward(v, om, *GEOM, G, D, 1.0, 64, 0, 0, 0, False)
        ext.dcnv4_backward(v, om, *GEOM, G, D, 1.0, 64, go, 0, 0, 0, False)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out = ext.dcnv4_forward(v, om, *GEOM, G, D, 1.0, 64, 0, 0, 0, False)
        g_gv, g_gom = ext.dcnv4_backward(v, om, *GEOM, G, D, 1.0, 64, go, 0, 0, 0, False)
    for _ in range(3):
        g_out.fill_(7.0)
        g_gv.fill_(7.0)
        g_gom.fill_(7.0)
        (v.float() @ torch.ones(64, 8, device="cuda")).sum().item()      # unrelated eager work + sync between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_out, eager_out) and torch.equal(g_gom, eager_gom)
        # grad_value: fp32 sums in hardware order, rounded once to fp16: at most one unit apart, and rarely
        diff = (g_gv.float() - eager_gv.float()).abs()
        assert (diff <= 2e-3 * eager_gv.float().abs() + 1e-6).all() and (diff > 0).float().mean().item() < 0.01


def test_small_flash_intern_image_matches_the_same_network_on_the_torch_core(monkeypatch):
    """A two-level FlashInternImage (DCNv4 layers on the HIP kernels) against the same weights evaluated on the
    CPU with the operator swapped for the grid_sample formulation."""
    from dcnv4_amd.models import FlashInternImage
    from dcnv4_amd.modules import dcnv4 as dcnv4_module

    torch.manual_seed(2)
    kw = dict(channels=32, depths=(2, 2), groups=(2, 4), offset_scale=1.0, drop_path_rate=0.0, layer_scale=1e-1,
              post_norm=True, dw_kernel_size=3, num_classes=10)
    model = FlashInternImage(**kw).eval()
    with torch.no_grad():
        for m in model.modules():
            if isinstance(m, dcnv4_module.DCNv4):
                m.offset_mask.weight.normal_(0, 0.2)
                m.offset_mask.bias.normal_(0, 0.5)
    x = torch.randn(2, 3, 64, 64)

    class CoreOnCpu:
        @staticmethod
        def apply(inp, om, kh, kw_, sh, sw, ph, pw, dh, dw, group, group_channels, offset_scale, im2col_step, remove_center):
            return torch_core.dcnv4_core_torch(inp, om, kh, kw_, sh, sw, ph, pw, dh, dw, group, group_channels,
                                               offset_scale, remove_center)

    with torch.no_grad():
        got = model.cuda()(x.cuda()).cpu()
        feats = [f.cpu() for f in model.forward_features_seq_out(x.cuda())]
    # one training-style backward on the GPU (every autograd Function of the library in place) ...
    import copy
    state = copy.deepcopy(model.state_dict())           # the training pass moves the batch-norm statistics
    model.train()
    weights = torch.randn(2, 10)
    (model(x.cuda()) * weights.cuda()).sum().backward()
    gpu_grads = {k: p.grad.detach().cpu().clone() for k, p in model.named_parameters() if p.grad is not None}
    model.zero_grad()
    model.load_state_dict(state)
    model.cpu().eval()
    # ... against the same network on the CPU with the operators swapped for torch formulations
    monkeypatch.setattr(dcnv4_module, "DCNv4Function", CoreOnCpu)
    monkeypatch.setattr(dcnv4_module, "DepthwiseConvNHWCFunction", DepthwiseOnCpu)
    with torch.no_grad():
        want = model(x)
    model.train()
    (model(x) * weights).sum().backward()
    assert got.shape == (2, 10) and [tuple(f.shape) for f in feats] == [(2, 32, 16, 16), (2, 64, 8, 8)]
    assert _rel_err(got, want) < 1e-3
    checked = 0
    scale = max(float(p.grad.abs().max()) for p in model.parameters() if p.grad is not None)
    for k, p in model.named_parameters():
        if p.grad is None:
            continue
        assert k in gpu_grads, k
        if float(p.grad.abs().max()) < 1e-5 * scale:         # e.g. a bias in front of a batch norm: zero up to rounding
            assert float(gpu_grads[k].abs().max()) < 1e-4 * scale, k
            continue
        assert _rel_err(gpu_grads[k], p.grad) < 5e-3, k
        checked += 1
    assert checked > 60


def test_dense_prediction_backbone_returns_per_level_maps_for_a_non_square_input(monkeypatch):
    """FlashInternImageBackbone (detection / segmentation use): list of NCHW maps for the requested levels, on a
    non-square input, equal to the same weights evaluated with the operator on the CPU grid_sample formulation."""
    from dcnv4_amd.models import FlashInternImageBackbone
    from dcnv4_amd.modules import dcnv4 as dcnv4_module

    torch.manual_seed(5)
    model = FlashInternImageBackbone(out_indices=(1, 2, 3), channels=16, depths=(1, 1, 1, 1), groups=(1, 2, 4, 8),
                                     offset_scale=1.0, drop_path_rate=0.0, layer_scale=1e-1, post_norm=True,
                                     dw_kernel_size=3).eval()
    assert not any(k.startswith(("conv_head", "head")) for k in model.state_dict())
    with torch.no_grad():
        for m in model.modules():
            if isinstance(m, dcnv4_module.DCNv4):
                m.offset_mask.weight.normal_(0, 0.2)
                m.offset_mask.bias.normal_(0, 0.5)
    x = torch.randn(2, 3, 64, 96)

    class CoreOnCpu:
        @staticmethod
        def apply(inp, om, kh, kw_, sh, sw, ph, pw, dh, dw, group, group_channels, offset_scale, im2col_step, remove_center):
            return torch_core.dcnv4_core_torch(inp, om, kh, kw_, sh, sw, ph, pw, dh, dw, group, group_channels,
                                               offset_scale, remove_center)

    with torch.no_grad():
        got = [f.cpu() for f in model.cuda()(x.cuda())]
        model.cpu()
        monkeypatch.setattr(dcnv4_module, "DCNv4Function", CoreOnCpu)
        monkeypatch.setattr(dcnv4_module, "DepthwiseConvNHWCFunction", DepthwiseOnCpu)
        want = model(x)
    assert [tuple(f.shape) for f in got] == [(2, 32, 8, 12), (2, 64, 4, 6), (2, 128, 2, 3)]
    for g, w in zip(got, want):
        assert _rel_err(g, w) < 1e-3


def test_dcnv4_module_under_autocast_runs_the_half_kernels_and_returns_fp32_parameter_gradients():
    """AMP wiring of both autograd Functions (torch.amp.custom_fwd / custom_bwd, device_type="cuda"): activations
    in fp16 inside the module, fp32 parameters and fp32 parameter gradients outside, values within fp16 tolerance of
    the fp32 run."""
    import dcnv4_amd
    torch.manual_seed(4)
    C, G, H, W, N = 64, 4, 10, 9, 2
    m = dcnv4_amd.DCNv4(channels=C, group=G, dw_kernel_size=3).cuda()
    with torch.no_grad():
        m.offset_mask.weight.normal_(0, 0.3)
        m.offset_mask.bias.normal_(0, 0.5)
    x = torch.randn(N, H * W, C, device="cuda")
    ref = m(x.clone().requires_grad_(True), shape=(H, W))
    ref.sum().backward()
    ref_grads = {k: p.grad.clone() for k, p in m.named_parameters()}
    m.zero_grad()
    seen = []
    real = dcnv4_amd.ext.dcnv4_forward
    try:
        dcnv4_amd.ext.dcnv4_forward = lambda v, om, *a: (seen.append((v.dtype, om.dtype)), real(v, om, *a))[1]
        xa = x.clone().requires_grad_(True)
        with torch.autocast(device_type="cuda", dtype=torch.float16):
            out = m(xa, shape=(H, W))
        out.float().sum().backward()
    finally:
        dcnv4_amd.ext.dcnv4_forward = real
    assert seen == [(torch.float16, torch.float16)]
    assert out.dtype == torch.float16 and xa.grad.dtype == torch.float32
    assert _rel_err(out.float().cpu(), ref.detach().cpu()) < 1e-2
    for k, p in m.named_parameters():
        assert p.grad is not None and p.grad.dtype == torch.float32, k
        # gradients that pass through the sampling positions see the fp16 rounding of the offsets
        tol = 0.15 if k.startswith("offset_mask") else 3e-2
        assert _rel_err(p.grad.cpu(), ref_grads[k].cpu()) < tol, k


@pytest.mark.parametrize("options", [dict(gather="direct"), dict(tile=16), dict(gather="direct", tile=8),
                                     dict(gather="tiled", reach=2)])
def test_launch_options_change_the_kernels_not_the_results(oracle, options):
    """Thread-local launch options (what a tuned table entry applies around a call): every result against the oracle,
    and against the library's own choice."""
    import dcnv4_amd
    from dcnv4_amd import ext
    v, om, go = make_dcnv4_inputs(2, 20, 18, 4, 16, offset_range=3.0, seed=7, dtype=torch.float16)
    geom = (3, 3, 1, 1, 1, 1, 1, 1)
    oracle_out = oracle.dcnv4_forward(cabi.f64(v), cabi.f64(om), *geom, 4, 16, 1.0, 0, coord_f32=True)
    oracle_gv, oracle_gom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *geom, 4, 16, 1.0, 0, coord_f32=True)
    v, om, go = v.cuda(), om.cuda(), go.cuda()
    want = ext.dcnv4_forward(v, om, *geom, 4, 16, 1.0, 64, 0, 0, 0, False)
    wgv, wgom = ext.dcnv4_backward(v, om, *geom, 4, 16, 1.0, 64, go, 0, 0, 0, False)
    with ext.launch_options(**options):
        out = ext.dcnv4_forward(v, om, *geom, 4, 16, 1.0, 64, 0, 8, 128, False)
        gv, gom = ext.dcnv4_backward(v, om, *geom, 4, 16, 1.0, 64, go, 0, 0, 0, False)
    for got_out, got_gv, got_gom in ((want, wgv, wgom), (out, gv, gom)):
        cabi.assert_close(got_out, oracle_out, 1e-2, 1e-3, what=f"output, {options}")
        cabi.assert_close(got_gv, oracle_gv, 1e-2, 1e-2, what=f"grad_value, {options}")
        cabi.assert_close(got_gom, oracle_gom, 1e-2, 1e-2, what=f"grad_offset_mask, {options}")
    assert _rel_err(out.float().cpu(), want.float().cpu()) < 2e-3
    assert _rel_err(gv.float().cpu(), wgv.float().cpu()) < 1e-2
    assert _rel_err(gom.float().cpu(), wgom.float().cpu()) < 2e-3
    # the options are back at the library's choice afterwards: same kernels as before (grad_offset_mask has a
    # fixed summation order, so the same bits)
    again = ext.dcnv4_backward(v, om, *geom, 4, 16, 1.0, 64, go, 0, 0, 0, False)
    assert torch.equal(again[1], wgom) and _rel_err(again[0].float().cpu(), wgv.float().cpu()) < 1e-3


def test_fused_block_tail_has_autograd_gradients_and_falls_back_under_autocast():
    """layer_norm_residual: forward on the library's kernel, backward identical to autograd through torch's operators."""
    from dcnv4_amd.functions import layer_norm_residual
    torch.manual_seed(5)
    norm = torch.nn.LayerNorm(48, eps=1e-6).cuda()
    with torch.no_grad():
        norm.weight.normal_(1, 0.2)
        norm.bias.normal_(0, 0.2)
    gamma = torch.randn(48, device="cuda", requires_grad=True)
    y = torch.randn(3, 11, 48, device="cuda", requires_grad=True)
    x = torch.randn(3, 11, 48, device="cuda", requires_grad=True)
    go = torch.randn(3, 11, 48, device="cuda")
    ref = x + gamma * norm(y)
    want = torch.autograd.grad(ref, (y, x, gamma, norm.weight, norm.bias), go)
    out = layer_norm_residual(y, norm, gamma, x)
    assert out.grad_fn is not None and "LayerNormResidualFunction" in type(out.grad_fn).__name__
    got = torch.autograd.grad(out, (y, x, gamma, norm.weight, norm.bias), go)
    assert _rel_err(out.detach().cpu(), ref.detach().cpu()) < 1e-5
    for a, b in zip(got, want):
        assert _rel_err(a.cpu(), b.cpu()) < 1e-5
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        mixed = layer_norm_residual(y, norm, gamma, x)                # torch's operators: autocast semantics kept
    assert "LayerNormResidualFunction" not in type(mixed.grad_fn).__name__


def test_depthwise_and_block_tail_replay_correctly_from_a_hip_graph():
    from dcnv4_amd import ext
    g = torch.Generator().manual_seed(12)
    x = torch.randn(4, 20, 18, 64, generator=g).half().cuda()
    w = (torch.randn(64, 1, 3, 3, generator=g) / 3).half().cuda()
    b = torch.randn(64, generator=g).half().cuda()
    go = torch.randn(4, 20, 18, 64, generator=g).half().cuda()
    gamma = torch.randn(64, generator=g).half().cuda()

    def run():
        y = ext.depthwise_conv_forward(x, w, b, 1)
        gi, gw, gb = ext.depthwise_conv_backward(x, w, go, 1)
        return y, gi, gw, gb, ext.layer_norm_residual_forward(y, x, w.flatten()[:64].contiguous(), b, gamma, 1e-6)

    eager = run()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    for _ in range(3):
        for t in captured:
            t.fill_(7.0)
        (x.float().sum() + 1).item()                                     # unrelated eager work + sync between replays
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a, e) for a, e in zip(captured, eager))


def test_depthwise_adjoint_identities_at_a_benchmark_shape():
    """<go, conv(x)> = <grad_x, x> = <grad_w, w> + <grad_b, b> ... at 32x56x56x112 in fp32 (linear in x and in (w, b))."""
    from dcnv4_amd import ext
    g = torch.Generator().manual_seed(13)
    x = torch.randn(32, 56, 56, 112, generator=g).cuda()
    w = (torch.randn(112, 1, 3, 3, generator=g) / 3).cuda()
    b = torch.randn(112, generator=g).cuda()
    go = torch.randn(32, 56, 56, 112, generator=g).cuda()
    y = ext.depthwise_conv_forward(x, w, b, 1)
    y0 = ext.depthwise_conv_forward(x, w, None, 1)
    gi, gw, gb = ext.depthwise_conv_backward(x, w, go, 1)
    dot = lambda a, c: (a.double() * c.double()).sum().item()
    lhs = dot(go, y0)
    assert abs(dot(gi, x) - lhs) < 1e-5 * abs(lhs) + 1e-2
    assert abs(dot(gw, w) - lhs) < 1e-4 * abs(lhs) + 1e-1
    assert abs(dot(go, y) - lhs - dot(gb, b)) < 1e-4 * abs(lhs) + 1e-1


def test_depthwise_batches_beyond_the_32_bit_addressing_span_are_chunked_consistently():
    # 2.7 GB of input: more than one launch addresses with 32-bit buffer offsets; images are independent, so any
    # slice of the batch must give the same bits, and grad_weight must equal the sum over slices
    torch.manual_seed(6)
    B, H, W, C = 20, 512, 512, 128
    x = torch.randn(B, H, W, C, device="cuda")
    w = torch.randn(C, 3, 3, device="cuda") / 3
    b = torch.randn(C, device="cuda")
    out = cabi.depthwise_forward(x, w, b, 1)
    for lo, hi in [(0, 2), (7, 9), (18, 20)]:
        assert torch.equal(out[lo:hi], cabi.depthwise_forward(x[lo:hi].contiguous(), w, b, 1))
    go = out                                   # any values do as the incoming gradient
    gi, gw, gb = cabi.depthwise_backward(x, w, go, 1)
    pi, _, _ = cabi.depthwise_backward(x[7:9].contiguous(), w, go[7:9].contiguous(), 1)
    assert torch.equal(gi[7:9], pi)
    gw_sum = torch.zeros_like(gw, dtype=torch.float64)
    gb_sum = torch.zeros_like(gb, dtype=torch.float64)
    for lo in range(0, B, 5):
        _, pw, pb = cabi.depthwise_backward(x[lo:lo + 5].contiguous(), w, go[lo:lo + 5].contiguous(), 1)
        gw_sum += pw.double()
        gb_sum += pb.double()
    assert _rel_err(gw.double(), gw_sum) < 1e-5 and _rel_err(gb.double(), gb_sum) < 1e-5


def test_autograd_function_applies_a_tuned_table_entry(oracle, monkeypatch):
    """DCNv4Function looks shapes up as (B, H, W, group, channels per group), the reference's key convention; an
    entry with a kernel family must reach the library as a launch option around the call, and only around it."""
    import dcnv4_amd
    from dcnv4_amd import _lib, ext
    from dcnv4_amd.functions import launch_spec as ls
    B, H, W, G, D = 2, 12, 10, 2, 16
    v, om, go = make_dcnv4_inputs(B, H, W, G, D, seed=14, dtype=torch.float16)
    oracle_out = oracle.dcnv4_forward(cabi.f64(v), cabi.f64(om), *GEOM, G, D, 1.0, 0, coord_f32=True)
    oracle_gv, oracle_gom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *GEOM, G, D, 1.0, 0, coord_f32=True)
    v, om, go = v.cuda(), om.cuda(), go.cuda()
    want = dcnv4_amd.DCNv4Function.apply(v, om, *GEOM, G, D, 1.0, 256, 0)
    monkeypatch.setitem(ls.GFX950_TABLE, ls.table_key(B, H, W, G, D, 2, "fwd"), {"d_stride": 8, "n_thread": 128, "gather": "direct"})
    monkeypatch.setitem(ls.GFX950_TABLE, ls.table_key(B, H, W, G, D, 2, "bwd"), {"d_stride": 1, "n_thread": 64, "tile": 16})
    ls._lookup.cache_clear()
    seen = []
    real = _lib.load().dcnv4_gfx950_set_launch_option

    class Spy:
        def __call__(self, name, value):
            seen.append((name, value))
            return real(name, value)

    monkeypatch.setattr(ext._L, "dcnv4_gfx950_set_launch_option", Spy(), raising=False)
    try:
        vg, omg = v.clone().requires_grad_(True), om.clone().requires_grad_(True)
        out = dcnv4_amd.DCNv4Function.apply(vg, omg, *GEOM, G, D, 1.0, 256, 0)
        out.backward(go)
    finally:
        ls._lookup.cache_clear()
    assert (b"gather", 2) in seen and (b"tile", 16) in seen
    assert seen[-1] == (b"tile", 0) and (b"gather", 0) in seen          # back at the library's choice
    assert _rel_err(out.float().cpu(), want.float().cpu()) < 2e-3
    cabi.assert_close(out.detach(), oracle_out, 1e-2, 1e-3, what="output through the table entry")
    cabi.assert_close(vg.grad, oracle_gv, 1e-2, 1e-2, what="grad_value through the table entry")
    cabi.assert_close(omg.grad, oracle_gom, 1e-2, 1e-2, what="grad_offset_mask through the table entry")


def test_block_tail_at_the_model_stage_one_size_normalises_every_row():
    """128 x 56 x 56 rows of 112 channels (FlashInternImage-B stage 1) in fp16: with unit weight and zero bias every
    output row has zero mean and unit (biased) variance; with residual and gamma the result is that plus the residual."""
    from dcnv4_amd import ext
    torch.manual_seed(15)
    y = (torch.randn(128 * 56 * 56, 112, device="cuda") * 3 + 1).half()
    ones, zeros = torch.ones(112, device="cuda").half(), torch.zeros(112, device="cuda").half()
    out = ext.layer_norm_residual_forward(y, None, ones, zeros, None, 1e-6).float()
    assert out.mean(-1).abs().max().item() < 2e-3
    assert (out.pow(2).mean(-1) - 1).abs().max().item() < 5e-3
    res = torch.randn_like(y)
    gamma = torch.full((112,), 0.5, device="cuda").half()
    both = ext.layer_norm_residual_forward(y, res, ones, zeros, gamma, 1e-6).float()
    assert (both - (res.float() + 0.5 * out)).abs().max().item() < 4e-3


def test_flash_deform_attn_adjoint_identity_at_full_benchmark_size_in_fp16():
    """The attention benchmark configuration in fp16: <g, f(v)> = <grad_value, v> (the operator is linear in value)."""
    torch.manual_seed(6)
    shapes = [(128, 128), (64, 64), (32, 32), (16, 16)]
    B, G, D, L, K = 4, 8, 32, 4, 4
    N = sum(h * w for h, w in shapes)
    dev = "cuda"
    shp = torch.tensor(shapes, device=dev)
    sizes = [h * w for h, w in shapes]
    st = torch.tensor([sum(sizes[:i]) for i in range(L)], device=dev)
    v = torch.randn(B, N, G, D, device=dev).half()
    sla = torch.cat([torch.rand(B, N, G, L * K * 2, device=dev), torch.randn(B, N, G, L * K, device=dev)], -1).half()
    g = torch.randn(B, N, G * D, device=dev).half()
    out = cabi.fda_forward(v, shp, st, sla, K)
    gv, gs = cabi.fda_backward(v, shp, st, sla, g, K)
    lhs = (g.double() * out.double()).sum()
    rhs = (gv.double() * v.double()).sum()
    scale = (g.double().abs() * out.double().abs()).sum()
    assert abs(float(lhs - rhs)) / float(scale) < 1e-3          # outputs and gradients rounded to fp16
    assert float(gs[..., 2 * L * K:].double().sum(-1).abs().max()) < 2e-2


def test_flash_intern_image_b_in_fp16_matches_the_same_weights_on_the_torch_core(monkeypatch):
    """The whole FlashInternImage-B (33 DCNv4 layers, groups 7 / 14 / 28 / 56) in fp16 at batch 8 against the same,
    fp16-rounded weights evaluated in fp32 on the CPU with the operators swapped for torch formulations.  Offsets and
    layer scales are made non-trivial first: at their initial values (zero offsets, 1e-5) the operator would hardly
    show in the logits."""
    import copy
    from dcnv4_amd.models import flash_intern_image
    from dcnv4_amd.modules import dcnv4 as dcnv4_module

    torch.manual_seed(3)
    model = flash_intern_image("b").eval()
    with torch.no_grad():
        for m in model.modules():
            if isinstance(m, dcnv4_module.DCNv4):
                m.offset_mask.weight.normal_(0, 0.02)
                m.offset_mask.bias.normal_(0, 0.7)
        for name, prm in model.named_parameters():
            if name.endswith("gamma1") or name.endswith("gamma2"):
                prm.fill_(0.2)
    x = torch.randn(8, 3, 224, 224)
    half = copy.deepcopy(model).half().cuda()
    with torch.no_grad():
        got = half(x.half().cuda()).float().cpu()
    ref = copy.deepcopy(model)
    ref.load_state_dict({k: v.float().cpu() for k, v in half.state_dict().items()})      # the fp16-rounded weights

    class CoreOnCpu:
        @staticmethod
        def apply(inp, om, kh, kw_, sh, sw, ph, pw, dh, dw, group, group_channels, offset_scale, im2col_step, remove_center):
            return torch_core.dcnv4_core_torch(inp, om, kh, kw_, sh, sw, ph, pw, dh, dw, group, group_channels,
                                               offset_scale, remove_center)

    monkeypatch.setattr(dcnv4_module, "DCNv4Function", CoreOnCpu)
    monkeypatch.setattr(dcnv4_module, "DepthwiseConvNHWCFunction", DepthwiseOnCpu)
    with torch.no_grad():
        want = ref(x.half().float())
    assert got.shape == (8, 1000) and torch.isfinite(got).all()
    assert _rel_err(got, want) < 3e-2


def test_every_committed_table_entry_still_beats_the_library_choice():
    """The dispatch table is measured data: an entry that no longer wins against the library's own planner (the kernels
    have changed since it was measured) must be deleted or re-measured with `python -m dcnv4_amd.tune`."""
    import re
    from dcnv4_amd import ext, tune
    from dcnv4_amd.functions import launch_spec as ls
    for key, entry in ls.GFX950_TABLE.items():
        options = {k: entry[k] for k in ls.OPTION_KEYS if k in entry}
        m = re.fullmatch(r"(\d+)x(\d+)x(\d+)x(\d+)x(\d+):(\d):(fwd|bwd)", key)
        if m is None:
            continue                  # attention entries are timed by the tuner only
        B, H, W, G, D, es, direction = (int(x) if x.isdigit() else x for x in m.groups())
        dtype = torch.float16 if es == 2 else torch.float32
        v, om, go = (t.cuda() for t in make_dcnv4_inputs(B, H, W, G, D, offset_range=3.0, seed=1, dtype=dtype))
        def call(d, n):
            if direction == "fwd":
                return ext.dcnv4_forward(v, om, *GEOM, G, D, 1.0, 64, 0, d, n, False)
            return ext.dcnv4_backward(v, om, *GEOM, G, D, 1.0, 64, go, 0, d, n, False)
        base = min(tune._time(lambda: call(0, 0), 30, 10) for _ in range(3))
        with ext.launch_options(**options):
            tuned = min(tune._time(lambda: call(entry["d_stride"], entry["n_thread"]), 30, 10) for _ in range(3))
        print(f"table entry {key}: library {base * 1e3:.1f} us, entry {tuned * 1e3:.1f} us", flush=True)
        assert tuned <= base, f"{key}: the entry ({tuned * 1e3:.1f} us) lost to the library's choice ({base * 1e3:.1f} us); re-run the tuner"
