"""The committed vectors under tests/golden/ (inputs + outputs of the pinned oracle, see make_fixtures.py there):
the oracle must keep reproducing them on the CPU, and the HIP path must match them through the C ABI."""
import glob
import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DCN_FILES = sorted(glob.glob(os.path.join(GOLDEN, "dcnv4_*.npz")))
FDA_FILES = sorted(glob.glob(os.path.join(GOLDEN, "fda_*.npz")))


def test_fixture_files_are_present():
    assert len(DCN_FILES) == 2 and len(FDA_FILES) == 1 and os.path.exists(os.path.join(GOLDEN, "block_level_ops.npz"))


@pytest.mark.parametrize("path", DCN_FILES, ids=os.path.basename)
def test_oracle_reproduces_the_dcnv4_vectors(path):
    from oracle import c_oracle
    z = np.load(path)
    geom, G, D = tuple(int(v) for v in z["geometry"]), int(z["group"]), int(z["group_channels"])
    rc, scale = int(z["remove_center"]), float(z["offset_scale"])
    v, om, go = (z[k].astype(np.float64) for k in ("value", "offset_mask", "grad_out"))
    np.testing.assert_allclose(c_oracle.dcnv4_forward(v, om, *geom, G, D, scale, rc, coord_f32=True), z["out"], rtol=0, atol=1e-12)
    gv, gom = c_oracle.dcnv4_backward(v, om, go, *geom, G, D, scale, rc, coord_f32=True)
    np.testing.assert_allclose(gv, z["grad_value"], rtol=0, atol=1e-12)
    np.testing.assert_allclose(gom, z["grad_offset_mask"], rtol=0, atol=1e-12)


@pytest.mark.parametrize("path", FDA_FILES, ids=os.path.basename)
def test_oracle_reproduces_the_attention_vectors(path):
    from oracle import c_oracle
    z = np.load(path)
    v, sla, go = (z[k].astype(np.float64) for k in ("value", "sampling_loc_attn", "grad_out"))
    K = int(z["K"])
    out = c_oracle.flash_deform_attn_forward(v, z["spatial_shapes"], z["level_start_index"], sla, K, coord_f32=True)
    np.testing.assert_allclose(out, z["out"], rtol=0, atol=1e-12)
    gv, gs = c_oracle.flash_deform_attn_backward(v, z["spatial_shapes"], z["level_start_index"], sla, go, K, coord_f32=True)
    np.testing.assert_allclose(gv, z["grad_value"], rtol=0, atol=1e-12)
    np.testing.assert_allclose(gs, z["grad_sampling_loc_attn"], rtol=0, atol=1e-12)


def test_oracle_reproduces_the_block_level_vectors():
    from oracle import depthwise, layer_norm
    z = np.load(os.path.join(GOLDEN, "block_level_ops.npz"))
    pad = int(z["pad"])
    y = depthwise.depthwise_forward(z["input"], z["weight"], z["bias"], pad)
    np.testing.assert_allclose(y, z["depthwise_out"], rtol=0, atol=1e-12)
    gx, gw, gb = depthwise.depthwise_backward(z["input"], z["weight"], z["grad_out"], pad)
    for got, key in ((gx, "grad_input"), (gw, "grad_weight"), (gb, "grad_bias")):
        np.testing.assert_allclose(got, z[key], rtol=0, atol=1e-12)
    tail = layer_norm.layer_norm_residual(y.astype(np.float32), z["weight"].reshape(-1)[:8], z["bias"], float(z["eps"]), z["gamma"], z["input"])
    np.testing.assert_allclose(tail, z["tail_out"], rtol=0, atol=1e-12)


@pytest.mark.gpu
@pytest.mark.parametrize("path", DCN_FILES, ids=os.path.basename)
def test_hip_path_matches_the_dcnv4_vectors(path):
    from tests import cabi
    z = np.load(path)
    geom, G, D = tuple(int(v) for v in z["geometry"]), int(z["group"]), int(z["group_channels"])
    rc, scale = int(z["remove_center"]), float(z["offset_scale"])
    v, om, go = (torch.from_numpy(z[k]).cuda() for k in ("value", "offset_mask", "grad_out"))
    cabi.assert_close(cabi.dcnv4_forward(v, om, geom, G, D, scale, rc), z["out"], 1e-4, 1e-5, what="output")
    gv, gom = cabi.dcnv4_backward(v, om, go, geom, G, D, scale, rc)
    cabi.assert_close(gv, z["grad_value"], 1e-3, 1e-4, what="grad_value")
    cabi.assert_close(gom, z["grad_offset_mask"], 1e-3, 1e-4, what="grad_offset_mask")


@pytest.mark.gpu
@pytest.mark.parametrize("path", FDA_FILES, ids=os.path.basename)
def test_hip_path_matches_the_attention_vectors(path):
    from tests import cabi
    z = np.load(path)
    v, sla, go = (torch.from_numpy(z[k]).cuda() for k in ("value", "sampling_loc_attn", "grad_out"))
    shp, st = torch.from_numpy(z["spatial_shapes"]).cuda(), torch.from_numpy(z["level_start_index"]).cuda()
    K = int(z["K"])
    cabi.assert_close(cabi.fda_forward(v, shp, st, sla, K), z["out"], 1e-4, 1e-5, what="output")
    gv, gs = cabi.fda_backward(v, shp, st, sla, go, K)
    cabi.assert_close(gv, z["grad_value"], 1e-3, 1e-4, what="grad_value")
    cabi.assert_close(gs, z["grad_sampling_loc_attn"], 1e-3, 1e-4, what="grad_sampling_loc_attn")


@pytest.mark.gpu
def test_hip_path_matches_the_block_level_vectors():
    from tests import cabi
    z = np.load(os.path.join(GOLDEN, "block_level_ops.npz"))
    pad = int(z["pad"])
    x, w, b, go, gamma = (torch.from_numpy(z[k]).cuda() for k in ("input", "weight", "bias", "grad_out", "gamma"))
    y = cabi.depthwise_forward(x, w, b, pad)
    cabi.assert_close(y, z["depthwise_out"], 1e-4, 1e-5, what="depthwise output")
    gx, gw, gb = cabi.depthwise_backward(x, w, go, pad)
    cabi.assert_close(gx, z["grad_input"], 1e-3, 1e-4, what="grad_input")
    cabi.assert_close(gw, z["grad_weight"], 1e-3, 1e-3, what="grad_weight")
    cabi.assert_close(gb, z["grad_bias"], 1e-3, 1e-3, what="grad_bias")
    y32 = torch.from_numpy(z["depthwise_out"].astype(np.float32)).cuda()
    tail = cabi.layer_norm_residual(y32, x, w.reshape(-1)[:8].contiguous(), b, gamma, float(z["eps"]))
    cabi.assert_close(tail, z["tail_out"], 1e-4, 1e-4, what="block tail")
