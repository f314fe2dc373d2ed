"""Writes tests/golden/*.npz: small seeded inputs and the CPU oracle's outputs for them.

The reference ships no golden vectors for this path (its scripts under DCNv4_op/scripts compare two GPU
operators live), so these are regression vectors of the oracle in this repository, frozen after the oracle was
pinned by tests/test_oracle_pins.py; they are not outputs of the reference.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import c_oracle, depthwise, layer_norm          # noqa: E402
from tests.inputs import make_dcnv4_inputs, make_fda_inputs  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

DCN = {
    # name: (B, H, W, G, D, geometry (kh, kw, sh, sw, ph, pw, dh, dw), remove_center, offset_scale, offset_range, seed)
    "dcnv4_3x3_g2_d16": (2, 9, 8, 2, 16, (3, 3, 1, 1, 1, 1, 1, 1), 0, 1.0, 2.5, 101),
    "dcnv4_stride2_remove_center": (1, 11, 10, 3, 8, (3, 3, 2, 2, 1, 1, 1, 1), 1, 0.5, 3.0, 102),
}
FDA = {"fda_2lvl_k4": (2, [(6, 5), (3, 3)], 2, 16, 4, 9, 103)}      # B, shapes, G, D, K, Q, seed


def main():
    for name, (B, H, W, G, D, geom, rc, scale, rng, seed) in DCN.items():
        v, om, go = make_dcnv4_inputs(B, H, W, G, D, *geom, remove_center=rc, offset_range=rng, seed=seed, dtype=torch.float32)
        v, om, go = (t.double().numpy() for t in (v, om, go))
        out = c_oracle.dcnv4_forward(v, om, *geom, G, D, scale, rc, coord_f32=True)
        gv, gom = c_oracle.dcnv4_backward(v, om, go, *geom, G, D, scale, rc, coord_f32=True)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), value=v.astype(np.float32), offset_mask=om.astype(np.float32),
                            grad_out=go.astype(np.float32), geometry=np.array(geom), group=G, group_channels=D,
                            remove_center=rc, offset_scale=scale, out=out, grad_value=gv, grad_offset_mask=gom)
    for name, (B, shapes, G, D, K, Q, seed) in FDA.items():
        v, shp, st, sla, go = make_fda_inputs(B, shapes, G, D, K, Q, seed=seed, dtype=torch.float32)
        vn, sn, gn = v.double().numpy(), sla.double().numpy(), go.double().numpy()
        out = c_oracle.flash_deform_attn_forward(vn, shp.numpy(), st.numpy(), sn, K, coord_f32=True)
        gv, gs = c_oracle.flash_deform_attn_backward(vn, shp.numpy(), st.numpy(), sn, gn, K, coord_f32=True)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), value=vn.astype(np.float32), spatial_shapes=shp.numpy(),
                            level_start_index=st.numpy(), sampling_loc_attn=sn.astype(np.float32), grad_out=gn.astype(np.float32),
                            K=K, out=out, grad_value=gv, grad_sampling_loc_attn=gs)
    g = np.random.default_rng(104)
    x = g.standard_normal((2, 7, 6, 8)).astype(np.float32)
    w = (g.standard_normal((8, 3, 3)) / 3).astype(np.float32)
    b = g.standard_normal(8).astype(np.float32)
    go = g.standard_normal((2, 7, 6, 8)).astype(np.float32)
    gamma = g.standard_normal(8).astype(np.float32)
    y = depthwise.depthwise_forward(x, w, b, 1)
    gx, gw, gb = depthwise.depthwise_backward(x, w, go, 1)
    tail = layer_norm.layer_norm_residual(y.astype(np.float32), w.reshape(-1)[:8], b, 1e-6, gamma, x)
    np.savez_compressed(os.path.join(HERE, "block_level_ops.npz"), input=x, weight=w, bias=b, grad_out=go, gamma=gamma, pad=1,
                        depthwise_out=y, grad_input=gx, grad_weight=gw, grad_bias=gb, tail_out=tail, eps=1e-6)
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


if __name__ == "__main__":
    main()
