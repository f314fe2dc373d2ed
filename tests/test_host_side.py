"""CPU-only checks of the host side: the C ABI exports what the header declares, the ctypes
signatures match the header, launch hints are well-formed, the nn.Modules keep the reference's
parameter names and shapes, and everything refuses to run without a GPU instead of falling back."""
import ctypes
import math
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dcnv4_gfx950.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = re.findall(r"\b(?:int|size_t|const char \*)\s*\*?\s*(\w+)\s*\(([^;{]*)\)\s*;", text)
    return {name: args for name, args in decls}


def test_library_exports_every_symbol_the_header_declares():
    from dcnv4_amd import _lib
    lib = ctypes.CDLL(_lib.LIB_PATH)
    declared = _declared_functions()
    assert len(declared) == 23, sorted(declared)
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/dcnv4_gfx950.h but not exported"
    assert set(declared) == set(_lib.SIGNATURES), "ctypes table and header list different functions"


def test_ctypes_signatures_have_the_arity_of_the_header():
    from dcnv4_amd import _lib
    for name, args in _declared_functions().items():
        args = args.strip()
        n = 0 if args in ("", "void") else len([a for a in args.split(",") if a.strip()])
        assert n == len(_lib.SIGNATURES[name][1]), f"{name}: header has {n} parameters"


def test_abi_version_and_error_string_work_without_a_gpu():
    from dcnv4_amd import _lib
    lib = _lib.load()
    assert lib.dcnv4_gfx950_abi_version() == _lib.ABI_VERSION
    # argument errors are detected before anything touches the device
    rc = lib.dcnv4_gfx950_forward(None, None, None, 7, 1, 4, 4, 1, 16, 3, 3, 1, 1, 1, 1, 1, 1, 1.0, 64, 0, 32, 0, 0, 0, None)
    assert rc == _lib.ERR_RUNTIME and b"dtype" in lib.dcnv4_gfx950_last_error()
    rc = lib.dcnv4_gfx950_forward(None, None, None, 1, 1, 4, 4, 1, 16, 3, 3, 1, 1, 1, 1, 1, 1, 1.0, 64, 0, 32, 0, 5, 0, None)
    assert rc == _lib.ERR_INVALID_ARGUMENT and b"d_stride" in lib.dcnv4_gfx950_last_error()
    rc = lib.flash_deform_attn_gfx950_forward(None, None, None, None, None, 1, 1, 16, 1, 16, 6, 4, 16, 64, 0, 0, None)
    assert rc == _lib.ERR_INVALID_ARGUMENT and b"points" in lib.dcnv4_gfx950_last_error()
    assert lib.dcnv4_gfx950_backward_workspace_bytes(1, 64, 56, 56, 4, 16) == 256
    assert lib.dcnv4_gfx950_backward_workspace_bytes(1, 2, 8, 8, 1, 128) == 256
    assert lib.dcnv4_gfx950_backward_workspace_bytes(0, 2, 8, 8, 1, 384) == 256


def test_cpu_tensors_are_refused_like_the_reference():
    import dcnv4_amd
    v, om = torch.zeros(1, 4, 4, 16), torch.zeros(1, 4, 4, 32)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        dcnv4_amd.DCNv4Function.apply(v, om, 3, 3, 1, 1, 1, 1, 1, 1, 1, 16, 1.0, 256, 0)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        dcnv4_amd.ext.flash_deform_attn_forward(torch.zeros(1, 16, 1, 16), torch.tensor([[4, 4]]), torch.tensor([0]),
                                                torch.zeros(1, 3, 1, 12), 64, 4, 8, 128)
    with pytest.raises(RuntimeError, match="contiguous"):
        dcnv4_amd.ext.dcnv4_forward(v.transpose(1, 2), om, 3, 3, 1, 1, 1, 1, 1, 1, 1, 16, 1.0, 256, 0, 8, 128, False)


def test_reference_package_name_is_importable():
    import DCNv4
    from DCNv4 import ext                                   # noqa: F401
    from DCNv4.functions import DCNv4Function, FlashDeformAttnFunction      # noqa: F401
    from DCNv4.modules import DCNv4 as Mod
    assert Mod is DCNv4.DCNv4


@pytest.mark.parametrize("G,C,es", [(4, 16, 2), (4, 16, 4), (80, 16, 2), (7, 16, 2), (8, 32, 2), (8, 32, 4), (3, 6, 2), (1, 1, 4)])
def test_launch_hints_are_well_formed(G, C, es):
    from dcnv4_amd.functions import launch_spec as ls
    for fn in (ls.findspec, ls.find_spec_bwd):
        d_stride, n_thread = fn(64, 56, 56, G, C, es)
        assert d_stride in (1, 2, 4, 8) and C % d_stride == 0 and d_stride * es <= 16
        lanes = 1
        while lanes < C // d_stride:
            lanes *= 2
        assert n_thread % (G * lanes) == 0 and n_thread >= G * lanes
    # the backward gathers as well (grad_value is a gather): the same 16-byte lanes as the forward, never a narrowing hint
    assert ls.find_spec_bwd(64, 56, 56, G, C, es) == ls.findspec(64, 56, 56, G, C, es)
    assert ls.findspec_attn_bwd(4, 21760, G, C, es) == ls.findspec_attn(4, 21760, G, C, es)


def test_dcnv4_module_keeps_the_reference_parameter_schema():
    from dcnv4_amd import DCNv4
    m = DCNv4(channels=112, group=7, offset_scale=0.5, dw_kernel_size=3, center_feature_scale=True, output_bias=False)
    sd = {k: tuple(v.shape) for k, v in m.state_dict().items()}
    K = 7 * 9
    assert sd == {
        "center_feature_scale_proj_weight": (7, 112), "center_feature_scale_proj_bias": (7,),
        "offset_mask_dw.weight": (112, 1, 3, 3), "offset_mask_dw.bias": (112,),
        "offset_mask.weight": (int(math.ceil(K * 3 / 8) * 8), 112), "offset_mask.bias": (int(math.ceil(K * 3 / 8) * 8),),
        "value_proj.weight": (112, 112), "value_proj.bias": (112,), "output_proj.weight": (112, 112),
    }
    assert m.offset_mask.weight.abs().sum() == 0 and m.offset_mask.bias.abs().sum() == 0
    assert DCNv4(channels=64, group=4, remove_center=True).offset_mask.out_features == 96
    assert "value_proj.weight" not in DCNv4(channels=64, group=4, without_pointwise=True).state_dict()
    with pytest.raises(ValueError):
        DCNv4(channels=65, group=4)


def test_flash_deform_attn_module_keeps_the_reference_parameter_schema():
    from dcnv4_amd import FlashDeformAttn
    m = FlashDeformAttn(d_model=256, n_levels=4, n_heads=8, n_points=4)
    sd = {k: tuple(v.shape) for k, v in m.state_dict().items()}
    assert sd == {"sampling_offsets.weight": (256, 256), "sampling_offsets.bias": (256,),
                  "attention_weights.weight": (128, 256), "attention_weights.bias": (128,),
                  "value_proj.weight": (256, 256), "value_proj.bias": (256,),
                  "output_proj.weight": (256, 256), "output_proj.bias": (256,)}
    bias = m.sampling_offsets.bias.view(8, 4, 4, 2)
    assert torch.allclose(bias[0, 0, :, 0], torch.tensor([1.0, 2.0, 3.0, 4.0])) and bias[0, 0, :, 1].abs().max() < 1e-6
    assert m.im2col_step == 64


@pytest.mark.parametrize("variant,millions", [("t", 30), ("s", 50), ("b", 97), ("l", 223)])
def test_flash_intern_image_parameter_counts_match_the_published_model_sizes(variant, millions):
    # README.md:29-32 of the reference lists 30M / 50M / 97M / 223M parameters for T / S / B / L
    from dcnv4_amd.models import flash_intern_image
    m = flash_intern_image(variant)
    n = sum(p.numel() for p in m.parameters())
    assert abs(n / 1e6 - millions) < 0.6, n


def test_flash_intern_image_state_dict_uses_the_reference_key_names():
    from dcnv4_amd.models import flash_intern_image
    keys = set(flash_intern_image("b").state_dict())
    for k in ["patch_embed.conv1.weight", "patch_embed.norm1.0.running_mean", "patch_embed.norm2.0.weight",
              "levels.0.blocks.0.gamma1", "levels.0.blocks.0.norm1.0.weight", "levels.0.blocks.0.dcn.offset_mask_dw.weight",
              "levels.0.blocks.0.dcn.offset_mask.weight", "levels.0.blocks.0.dcn.value_proj.bias",
              "levels.0.blocks.0.dcn.output_proj.weight", "levels.0.blocks.0.mlp.fc1.bias", "levels.0.blocks.0.mlp.fc2.weight",
              "levels.0.downsample.conv.weight", "levels.0.downsample.norm.1.weight", "levels.2.blocks.20.norm2.0.bias",
              "conv_head.0.weight", "conv_head.1.0.running_var", "head.weight", "head.bias"]:
        assert k in keys, k
    assert "levels.0.blocks.0.dcn.output_proj.bias" not in keys          # dcn_output_bias is False for B
    assert "levels.3.downsample.conv.weight" not in keys and "levels.0.norm.0.weight" not in keys   # post_norm variant
    t_keys = set(flash_intern_image("t").state_dict())
    assert "levels.0.norm.0.weight" in t_keys and "levels.0.blocks.0.gamma1" not in t_keys


@pytest.mark.parametrize("variant", ["t", "s", "b", "l"])
def test_model_state_dict_equals_the_schema_written_from_the_reference_definitions(variant):
    """Names, shapes and order of every parameter and buffer, both ways (classification/models/flash_intern_image.py)."""
    from dcnv4_amd.models import check_state_dict, flash_intern_image, reference_schema
    schema = reference_schema(variant)
    state = flash_intern_image(variant).state_dict()
    assert check_state_dict(state, schema) == []
    assert list(state) == list(schema)


def test_offset_mask_projection_is_padded_to_a_multiple_of_eight():
    from dcnv4_amd.models import offset_mask_features, reference_schema
    assert [offset_mask_features(g) for g in (4, 7, 5, 10, 56)] == [112, 192, 136, 272, 1512]   # 108, 189, 135, 270, 1512
    assert reference_schema("b")["levels.0.blocks.0.dcn.offset_mask.weight"] == (192, 112)
    assert reference_schema("t")["levels.3.blocks.3.dcn.offset_mask.bias"] == (864,)


def test_checkpoint_in_the_reference_file_layout_loads_and_misfits_are_named(tmp_path):
    from dcnv4_amd.models import FlashInternImage, check_state_dict, load_checkpoint, reference_schema
    kw = dict(channels=16, depths=(1, 1), groups=(1, 2), layer_scale=1e-5, post_norm=True, dw_kernel_size=3, num_classes=5)
    src, dst = FlashInternImage(**kw), FlashInternImage(**kw)
    with torch.no_grad():
        for p in src.parameters():
            p.normal_()
    path = tmp_path / "flash_intern_image_tiny.pth"
    torch.save({"model": {"module." + k: v for k, v in src.state_dict().items()}, "epoch": 3}, path)   # classification/utils.py layout
    assert load_checkpoint(dst, path) == []
    assert all(torch.equal(a, b) for a, b in zip(src.state_dict().values(), dst.state_dict().values()))
    # a checkpoint whose offset_mask projection was saved without the padding is reported, with the reason
    bad = dict(src.state_dict())
    bad["levels.0.blocks.0.dcn.offset_mask.weight"] = bad["levels.0.blocks.0.dcn.offset_mask.weight"][:27]
    del bad["head.bias"]
    bad["extra.weight"] = torch.zeros(1)
    problems = check_state_dict(bad, {k: tuple(v.shape) for k, v in dst.state_dict().items()})
    assert len(problems) == 3 and any("multiple of 8" in p for p in problems) and any("missing key head.bias" in p for p in problems)
    assert any("unexpected key extra.weight" in p for p in problems)
    torch.save({"model": bad}, path)
    with pytest.raises(RuntimeError, match="does not fit"):
        load_checkpoint(dst, path)


def test_launch_table_entries_reach_the_dispatcher_and_lookups_are_memoised(monkeypatch):
    """A tuned entry (dcnv4_amd/tune.py output format) overrides the O(1) hints and carries kernel-family options."""
    from dcnv4_amd.functions import launch_spec as ls
    key = ls.table_key(3, 11, 13, 2, 32, 2, "fwd")
    monkeypatch.setitem(ls.GFX950_TABLE, key, {"d_stride": 4, "n_thread": 128, "gather": "direct"})
    ls._lookup.cache_clear()
    try:
        assert ls.findspec(3, 11, 13, 2, 32, 2) == (4, 128)
        assert ls.launch_options_for(3, 11, 13, 2, 32, 2, "fwd") == {"gather": "direct"}
        assert ls.launch_options_for(3, 11, 13, 2, 32, 2, "bwd") == {}                  # no entry: the library chooses
        assert ls.find_spec_bwd(3, 11, 13, 2, 32, 2) == ls._spec(2, 32, 2, scatter=True)
        hits = ls._lookup.cache_info().hits
        ls.findspec(3, 11, 13, 2, 32, 2)
        assert ls._lookup.cache_info().hits == hits + 1
    finally:
        ls._lookup.cache_clear()


def test_launch_options_are_validated_without_a_gpu():
    from dcnv4_amd import _lib
    lib = _lib.load()
    assert lib.dcnv4_gfx950_set_launch_option(b"gather", 2) == 0 and lib.dcnv4_gfx950_set_launch_option(b"gather", 0) == 0
    assert lib.dcnv4_gfx950_set_launch_option(b"reach", 7) == 0 and lib.dcnv4_gfx950_set_launch_option(b"reach", -1) == 0
    assert lib.dcnv4_gfx950_set_launch_option(b"tile", 16) == 0 and lib.dcnv4_gfx950_set_launch_option(b"tile", 0) == 0
    assert lib.dcnv4_gfx950_set_launch_option(b"tile", 12) == _lib.ERR_INVALID_ARGUMENT
    assert lib.dcnv4_gfx950_set_launch_option(b"gather_tile", 8) == 0 and lib.dcnv4_gfx950_set_launch_option(b"gather_tile", 0) == 0
    assert lib.dcnv4_gfx950_set_launch_option(b"gather_tile", 5) == _lib.ERR_INVALID_ARGUMENT
    assert lib.dcnv4_gfx950_set_launch_option(b"gv_threads", 512) == 0 and lib.dcnv4_gfx950_set_launch_option(b"gv_threads", 0) == 0
    assert lib.dcnv4_gfx950_set_launch_option(b"gv_threads", 256) == _lib.ERR_INVALID_ARGUMENT
    assert lib.dcnv4_gfx950_set_launch_option(b"dual", 2) == 0 and lib.dcnv4_gfx950_set_launch_option(b"dual", 0) == 0
    assert lib.dcnv4_gfx950_set_launch_option(b"dual", 3) == _lib.ERR_INVALID_ARGUMENT
    assert lib.dcnv4_gfx950_set_launch_option(b"gather", 5) == _lib.ERR_INVALID_ARGUMENT
    assert lib.dcnv4_gfx950_set_launch_option(b"nonsense", 1) == _lib.ERR_INVALID_ARGUMENT
    assert b"nonsense" in lib.dcnv4_gfx950_last_error()


def test_layer_level_entry_points_check_their_arguments_without_a_gpu():
    from dcnv4_amd import _lib
    lib = _lib.load()
    # centre-feature blend: group widths must be whole 16-byte vectors, channels a multiple of the groups
    rc = lib.dcnv4_gfx950_center_feature_blend_forward(None, None, None, None, None, 1, 10, 24, 6, None)
    assert rc == _lib.ERR_INVALID_ARGUMENT and b"group width" in lib.dcnv4_gfx950_last_error()
    rc = lib.dcnv4_gfx950_center_feature_blend_forward(None, None, None, None, None, 1, 10, 64, 5, None)
    assert rc == _lib.ERR_INVALID_ARGUMENT and b"equal groups" in lib.dcnv4_gfx950_last_error()
    rc = lib.dcnv4_gfx950_center_feature_blend_forward(None, None, None, None, None, 1, 10, 64, 4, None)
    assert rc == _lib.ERR_RUNTIME and b"null" in lib.dcnv4_gfx950_last_error()
    # block tail backward: bias is needed with gamma; workspace is checked
    rc = lib.dcnv4_gfx950_layer_norm_residual_backward(None, None, None, None, None, None, None, None, None, None, 0, 7, 10, 64, 1e-6, None)
    assert rc == _lib.ERR_RUNTIME and b"dtype" in lib.dcnv4_gfx950_last_error()
    # attention on un-packed rows: locations are fp32 or of the value's dtype
    rc = lib.flash_deform_attn_gfx950_forward_split(None, None, None, None, None, None, 0, 1, 1, 16, 1, 16, 1, 4, 4, 64, 0, 0, None)
    assert rc == _lib.ERR_RUNTIME and b"fp32 or of the value's dtype" in lib.dcnv4_gfx950_last_error()
    rc = lib.flash_deform_attn_gfx950_forward_split(None, None, None, None, None, None, 1, 0, 1, 16, 1, 16, 6, 4, 16, 64, 0, 0, None)
    assert rc == _lib.ERR_INVALID_ARGUMENT and b"points" in lib.dcnv4_gfx950_last_error()
    # the streaming copy wants whole 16-byte vectors (checked after the pointers)
    assert lib.dcnv4_gfx950_stream_copy(None, None, 32, None) == _lib.ERR_RUNTIME


def test_launch_option_contexts_nest_and_restore_what_they_found():
    import ctypes
    from dcnv4_amd import _lib, ext
    lib = _lib.load()

    def get(name):
        v = ctypes.c_int(123)
        assert lib.dcnv4_gfx950_get_launch_option(name, ctypes.byref(v)) == 0
        return v.value

    assert get(b"reach") == -1 and get(b"gather") == 0
    with ext.launch_options(reach=3, gather="direct"):
        assert get(b"reach") == 3 and get(b"gather") == 2
        with ext.launch_options(reach=9):
            assert get(b"reach") == 9 and get(b"gather") == 2
        assert get(b"reach") == 3
    assert get(b"reach") == -1 and get(b"gather") == 0
    assert lib.dcnv4_gfx950_get_launch_option(b"nonsense", ctypes.byref(ctypes.c_int())) == _lib.ERR_INVALID_ARGUMENT


def test_workspace_sizes_do_not_depend_on_launch_options_or_threads():
    """The size query and the call must agree whatever happens between them: the sizes are functions of the
    arguments only."""
    import threading
    from dcnv4_amd import _lib, ext
    lib = _lib.load()
    dcn = lambda: lib.dcnv4_gfx950_backward_workspace_bytes(1, 2, 8, 8, 2, 16)
    fda = lambda: lib.flash_deform_attn_gfx950_backward_workspace_bytes(1, 2, 80, 4, 32, 2, 50, 4)
    base = (dcn(), fda())
    assert base[0] == 256 and base[1] > 0
    ln = lambda: lib.dcnv4_gfx950_layer_norm_residual_backward_workspace_bytes(1, 5000, 112)
    assert ln() > 0 and ln() % 16 == 0 and ln() <= 2048 * 3 * 112 * 4
    assert lib.dcnv4_gfx950_layer_norm_residual_backward_workspace_bytes(1, 5000, 12) == 0      # not whole 16-byte vectors
    for options in (dict(scatter="atomic"), dict(gather="direct", tile=8), dict(fda_order="rows", reach=0), dict(gv_threads=512, gather_tile=8)):
        with ext.launch_options(**options):
            assert (dcn(), fda()) == base
    seen = []
    t = threading.Thread(target=lambda: seen.append((dcn(), fda())))
    with ext.launch_options(scatter="atomic"):
        t.start()
        t.join()
    assert seen == [base]


def test_tuner_candidates_are_valid_hints_and_start_with_the_library_choice():
    from dcnv4_amd import tune
    for G, D, es in [(4, 16, 2), (4, 16, 4), (8, 32, 2), (5, 24, 4)]:
        fwd = tune.candidates(G, D, es, "fwd")
        assert fwd[0] == ("library", {}, 0, 0)
        for _, options, d_stride, n_thread in fwd[1:]:
            if options == {"gather": "direct"}:
                assert D % d_stride == 0 and d_stride * es <= 16 and n_thread in (128, 256, 512)
            else:       # parameters of the tiled family: hints stay with the library
                assert set(options) <= {"reach", "gather_tile"} and (d_stride, n_thread) == (0, 0)
        assert {"reach": 3} in [c[1] for c in fwd] and {"gather_tile": 8} in [c[1] for c in fwd]
        bwd = tune.candidates(G, D, es, "bwd")
        assert bwd[0] == ("library", {}, 0, 0) and {"tile": 16} in [c[1] for c in bwd] and {"reach": 2} in [c[1] for c in bwd]
    assert {"gv_threads": 512} in [c[1] for c in bwd] and {"dual": "off"} in [c[1] for c in bwd]
    assert set(tune.SHAPES) == {"t", "b", "dense", "wide"} and all(len(v) in (2, 4) for v in tune.SHAPES.values())
    att = tune.attention_candidates("bwd")
    assert att[0] == ("library", {}) and {"scatter": "atomic"} in [c[1] for c in att] and {"fda_order": "heads"} in [c[1] for c in att]
    # every option the tuner may write is one the table loader passes on
    from dcnv4_amd.functions import launch_spec
    used = {k for c in tune.candidates(4, 16, 2, "fwd") + tune.candidates(4, 16, 2, "bwd") for k in c[1]} | {k for c in att for k in c[1]}
    assert used <= set(launch_spec.OPTION_KEYS)


def test_committed_table_entries_are_well_formed():
    from dcnv4_amd.functions import launch_spec
    for key, entry in launch_spec.GFX950_TABLE.items():
        assert key.split(":")[-1] in ("fwd", "bwd")
        assert set(entry) <= set(launch_spec.OPTION_KEYS) | {"d_stride", "n_thread"}, key
        if not key.startswith("attn:"):
            assert entry["d_stride"] in (1, 2, 4, 8, 16) and entry["n_thread"] > 0


def test_module_initial_values_follow_the_reference_recipe():
    """Xavier-uniform projections with zero biases, zero offset / modulation / attention projections, and the
    attention offsets' bias on a square ring (DCNv4_op/DCNv4/modules/dcnv4.py:95-103, flash_deform_attn.py:64-82)."""
    import math
    from dcnv4_amd import DCNv4, FlashDeformAttn
    torch.manual_seed(0)
    dcn = DCNv4(channels=128, group=8)
    att = FlashDeformAttn(d_model=128, n_levels=3, n_heads=8, n_points=4)
    for proj in (dcn.value_proj, dcn.output_proj, att.value_proj, att.output_proj):
        bound = math.sqrt(6.0 / (proj.in_features + proj.out_features))
        w = proj.weight.detach()
        assert w.abs().max() <= bound and w.abs().max() > 0.95 * bound          # uniform on [-bound, bound]
        assert abs(float(w.std()) - bound / math.sqrt(3.0)) < 0.03 * bound
        assert proj.bias.abs().sum() == 0
    for lin in (dcn.offset_mask, att.attention_weights):
        assert lin.weight.abs().sum() == 0 and lin.bias.abs().sum() == 0
    assert att.sampling_offsets.weight.abs().sum() == 0
    bias = att.sampling_offsets.bias.detach().view(8, 3, 4, 2)
    for h in range(8):
        theta = 2 * math.pi * h / 8
        d = torch.tensor([math.cos(theta), math.sin(theta)])
        d = d / d.abs().max()
        for k in range(4):
            assert torch.allclose(bias[h, :, k], (d * (k + 1)).expand(3, 2), atol=1e-6)


def test_committed_table_records_the_library_it_was_tuned_on():
    """The tuner stamps its table with the commit and a hash of the library's sources (DCNv4_op/scripts/find_best.py
    pastes its winners into table.py by hand; here a reader can tell which kernels the numbers belong to)."""
    import json
    from dcnv4_amd import tune
    from dcnv4_amd.functions import launch_spec as ls
    table = json.load(open(ls.TABLE_PATH))
    assert isinstance(table.get("entries"), dict) and table.get("cases", 0) >= 56
    assert isinstance(table.get("library_commit"), str) and len(table["library_commit"]) >= 7
    sha = table.get("library_sources_sha256")
    assert isinstance(sha, str) and len(sha) == 64 and len(tune.library_sources_sha256()) == 64
