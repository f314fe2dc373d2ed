"""The allocation-free DCNv4 backward (scratch in a device array inside the library) against the entry point that
takes a caller-provided workspace: same kernels, so the same results to the gradient tolerance, on two calls in a row
of which the second is smaller (the shared array keeps the first call's contents)."""
import pytest
import torch

from tests import cabi
from tests.inputs import make_dcnv4_inputs

pytestmark = pytest.mark.gpu

GEOM = (3, 3, 1, 1, 1, 1, 1, 1)
GRAD_TOL = {torch.float32: (1e-3, 1e-4), torch.float16: (1e-2, 1e-2)}


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=["fp32", "fp16"])
def test_static_scratch_backward_matches_workspace_backward_twice_in_a_row(oracle, dtype):
    calls = [(3, 40, 36, 4, 16, 3.0), (2, 9, 11, 3, 16, 2.0)]          # the second call is smaller
    for n, (B, H, W, G, D, rng) in enumerate(calls):
        v, om, go = make_dcnv4_inputs(B, H, W, G, D, offset_range=rng, seed=40 + n, dtype=dtype)
        print(f"static scratch call {n}: {B}x{H}x{W} G{G} D{D} {dtype}", flush=True)
        vd, omd, god = v.cuda(), om.cuda(), go.cuda()
        gv_ws, gom_ws = cabi.dcnv4_backward(vd, omd, god, GEOM, G, D, 1.0)
        # outputs exist before the call; around the call itself neither torch's allocator nor the device's free
        # memory may move (the entry point's own first-call set-up - the scratch address, a kernel attribute - allocates
        # nothing either)
        gv, gom = torch.full_like(vd, float("nan")), torch.full_like(omd, float("nan"))
        torch.cuda.synchronize()
        before = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0])
        cabi.dcnv4_backward_static_scratch(vd, omd, god, GEOM, G, D, 1.0, out=(gv, gom))
        torch.cuda.synchronize()
        after = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0])
        assert after == before, f"the allocation-free entry point moved device memory: {before} -> {after}"
        rtol, atol = GRAD_TOL[dtype]
        cabi.assert_close(gv, cabi.f64(gv_ws), rtol, atol, what=f"grad_value, call {n}")
        cabi.assert_close(gom, cabi.f64(gom_ws), rtol, atol, what=f"grad_offset_mask, call {n}")
        wgv, wgom = oracle.dcnv4_backward(cabi.f64(v), cabi.f64(om), cabi.f64(go), *GEOM, G, D, 1.0, 0, coord_f32=True)
        cabi.assert_close(gv, wgv, rtol, atol, what=f"grad_value vs oracle, call {n}")
        cabi.assert_close(gom, wgom, rtol, atol, what=f"grad_offset_mask vs oracle, call {n}")


def test_static_scratch_backward_reports_errors_like_the_workspace_entry_point():
    """The backward's scratch does not grow with the problem (256 bytes of state), so no size is beyond the static
    array; what the workspace entry point refuses, this one refuses with the same message."""
    from dcnv4_amd import _lib
    L = _lib.load()
    assert L.dcnv4_gfx950_backward_workspace_bytes(_lib.DTYPE_F16, 64, 256, 256, 10, 16) == 256
    t = torch.zeros(16, device="cuda", dtype=torch.float16)
    rc = L.dcnv4_gfx950_backward_static_scratch(t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(),
                                                _lib.DTYPE_F16, 4, 64, 64, 2, 1024, *GEOM, 1.0, 64, 0, 56, 0, 0, 0, None)
    assert rc == _lib.ERR_INVALID_ARGUMENT and b"channels" in L.dcnv4_gfx950_last_error()
