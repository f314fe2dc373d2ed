"""Launch-spec tuner for gfx950: ``python -m dcnv4_amd.tune [--shapes t,b,dense] [--dtypes float16,float32]``.

Counterpart of the reference's DCNv4_op/scripts/search_dcnv4.py, search_dcnv4_bwd.py and find_best.py, which
time every (d_stride, block_thread) pair per ``BxHxWxGxC`` and paste the winners into functions/table.py.
Here the candidates are the kernel family (LDS-tiled or direct gathers), the two hints of the direct family, the
reach and output-tile cap of the tiled gathers, the input-tile cap of the grad_value kernel and, for flash deformable
attention, the workgroup order and the grad_value scheme (binned LDS accumulation or global atomics); each is timed with HIP events through the same
``dcnv4_amd.ext`` calls the autograd Function makes, and the winners go to ``functions/gfx950_table.json``, which
``functions/launch_spec.py`` loads at import.  An entry is only written when it beats the library's own choice by
more than ``--margin`` (default 3 %) and by more than ``--min-gain-us`` (default 10 us: applying an entry's
kernel-family options costs a few microseconds of host time per call), so an empty table is a valid outcome.
"""
import argparse
import glob
import hashlib
import json
import math
import os
import sys
import time

SHAPES = {
    # the reference's benchmark shapes (DCNv4_op/scripts/test_dcnv4.py:23-31, classification configs)
    "t": [(64, 56, 56, 4, 16), (64, 28, 28, 8, 16), (64, 14, 14, 16, 16), (64, 7, 7, 32, 16)],
    "b": [(128, 56, 56, 7, 16), (128, 28, 28, 14, 16), (128, 14, 14, 28, 16), (128, 7, 7, 56, 16)],
    "dense": [(2, 256, 256, 10, 16), (2, 128, 128, 20, 16), (2, 64, 64, 40, 16), (2, 32, 32, 80, 16)],
    # groups of 64 channels: keys of the reference's table (DCNv4_op/DCNv4/functions/table.py:452-461)
    "wide": [(64, 56, 56, 4, 64), (64, 28, 28, 4, 64)],
}
GEOM = (3, 3, 1, 1, 1, 1, 1, 1)


def library_sources_sha256():
    """Hash of the library's sources (csrc/*.hip, *.hpp and the C header): a table records which kernels it was tuned on,
    also where no git history travels with the tree."""
    here = os.path.dirname(os.path.abspath(__file__))
    files = sorted(glob.glob(os.path.join(here, "csrc", "*.hip")) + glob.glob(os.path.join(here, "csrc", "*.hpp")) +
                   [os.path.join(os.path.dirname(here), "include", "dcnv4_gfx950.h")])
    h = hashlib.sha256()
    for f in files:
        h.update(os.path.basename(f).encode() + b"\0")
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def _time(fn, iters, warm):
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def candidates(G, D, elem_bytes, direction):
    """(label, options, d_stride, n_thread) for a DCNv4 call; the first one is the library's own choice.  Every launch
    parameter the kernels have is swept, as the reference's search scripts sweep theirs
    (DCNv4_op/scripts/search_dcnv4.py:100-115): kernel family, hints of the direct family, the staged reach and the
    output-tile cap of the LDS-tiled gathers, the input-tile cap and the workgroup size of the grad_value kernel, one launch or two for the backward of small images."""
    out = [("library", {}, 0, 0)]
    for reach in (2, 3, 4, 6):
        out.append((f"reach {reach}", {"reach": reach}, 0, 0))
    for gt in (8, 4):
        out.append((f"gather tile {gt}", {"gather_tile": gt}, 0, 0))
        out.append((f"gather tile {gt} reach 3", {"gather_tile": gt, "reach": 3}, 0, 0))
    if direction == "fwd":
        widths = [c for c in (8, 4, 2) if D % c == 0 and c * elem_bytes <= 16]
        for d in widths:
            for n in (128, 256, 512):
                out.append((f"direct d{d} n{n}", {"gather": "direct"}, d, n))
    else:
        out.append(("direct gathers", {"gather": "direct"}, 0, 0))
        for tile in (16, 8):
            out.append((f"grad_value tile {tile}", {"tile": tile}, 0, 0))
            out.append((f"grad_value tile {tile} reach 3", {"tile": tile, "reach": 3}, 0, 0))
        out.append(("two launches", {"dual": "off"}, 0, 0))
        out.append(("one launch, two workgroup roles", {"dual": "on", "gv_threads": 512}, 0, 0))
        for threads in (512, 1024):
            out.append((f"grad_value {threads} lanes", {"gv_threads": threads}, 0, 0))
            out.append((f"grad_value {threads} lanes tile 16", {"gv_threads": threads, "tile": 16}, 0, 0))
    return out


def attention_candidates(direction):
    out = [("library", {})]
    for order in ("rows", "heads"):
        out.append((f"order {order}", {"fda_order": order}))
    if direction == "fwd":
        out.append(("heads, small levels in LDS", {"fda_order": "heads", "fda_stage": "on"}))
        out.append(("heads, all levels from memory", {"fda_order": "heads", "fda_stage": "off"}))
    if direction == "bwd":
        out.append(("atomic scatter", {"scatter": "atomic"}))
        out.append(("atomic scatter, rows", {"scatter": "atomic", "fda_order": "rows"}))
    return out


# flash deformable attention shapes: (B, level shapes, heads, head channels, points); queries = all pixels
ATTN_SHAPES = {
    "detr": [(4, [(128, 128), (64, 64), (32, 32), (16, 16)], 8, 32, 4)],
    "detr_coco": [(2, [(100, 152), (50, 76), (25, 38), (13, 19)], 8, 32, 8)],       # DCNv4_op/scripts/test_flash_deform_attn.py:104-111
}


def _keep(entries, report, key, timings, margin, min_gain_us, make_entry, log):
    base, best = timings[0][0], min(timings, key=lambda t: t[0])
    report.append({"key": key, "library_ms": round(base, 5), "best_ms": round(best[0], 5), "best": best[1],
                   "all": {t[1]: round(t[0], 5) for t in timings}})
    log(f"{key:40s} library {base * 1e3:8.1f} us   best {best[0] * 1e3:8.1f} us  ({best[1]})")
    if best[0] < base * (1.0 - margin) and (base - best[0]) * 1e3 > min_gain_us:
        entries[key] = make_entry(best)


def tune(shape_sets, dtypes, iters=50, warm=10, margin=0.03, min_gain_us=10.0, offset_range=None, rounds=2, log=print):
    import torch
    from . import ext
    from .functions import launch_spec
    dev = torch.device("cuda:0")
    entries, report = {}, []
    for set_name in shape_sets:
        for B, H, W, G, D in SHAPES.get(set_name, []):
            C, K = G * D, 9
            p_pad = int(math.ceil(G * K * 3 / 8) * 8)
            for dt_name in dtypes:
                dtype = getattr(torch, dt_name)
                es = torch.empty(0, dtype=dtype).element_size()
                value = torch.randn(B, H, W, C, device=dev).to(dtype)
                om = torch.zeros(B, H, W, p_pad, device=dev)
                rng = offset_range if offset_range is not None else (4.0 if set_name == "dense" else 3.0)      # the benchmark's ranges
                om[..., :G * K * 3] = torch.cat([(torch.rand(B, H, W, G, 2 * K, device=dev) * 2 - 1) * rng,
                                                 torch.randn(B, H, W, G, K, device=dev)], -1).reshape(B, H, W, G * K * 3)
                om = om.to(dtype)
                go = torch.randn(B, H, W, C, device=dev).to(dtype)
                for direction in ("fwd", "bwd"):
                    cands = candidates(G, D, es, direction)
                    best_ms = [float("inf")] * len(cands)
                    for _ in range(rounds):       # every candidate in every round: clocks and caches settle for all alike
                        for ci, (label, options, d_stride, n_thread) in enumerate(cands):
                            if direction == "fwd":
                                call = lambda: ext.dcnv4_forward(value, om, *GEOM, G, D, 1.0, 64, 0, d_stride, n_thread, False)
                            else:
                                call = lambda: ext.dcnv4_backward(value, om, *GEOM, G, D, 1.0, 64, go, 0, d_stride, n_thread, False)
                            with ext.launch_options(**options):
                                best_ms[ci] = min(best_ms[ci], _time(call, iters, warm))
                    timings = [(ms,) + c for ms, c in zip(best_ms, cands)]
                    key = launch_spec.table_key(B, H, W, G, D, es, direction)      # C of the key = channels per group

                    def make_entry(best, direction=direction):
                        d, n = (best[3], best[4]) if best[3] else launch_spec._spec(G, D, es, scatter=direction == "bwd")
                        return dict(d_stride=d, n_thread=n, **best[2])
                    _keep(entries, report, key, timings, margin, min_gain_us, make_entry, log)
                del value, om, go
        for B, shapes, G, D, K in ATTN_SHAPES.get(set_name, []):
            L, N = len(shapes), sum(h * w for h, w in shapes)
            sizes = [h * w for h, w in shapes]
            shp = torch.tensor(shapes, dtype=torch.int64, device=dev)
            starts = torch.tensor([sum(sizes[:i]) for i in range(L)], dtype=torch.int64, device=dev)
            for dt_name in dtypes:
                dtype = getattr(torch, dt_name)
                es = torch.empty(0, dtype=dtype).element_size()
                v = torch.randn(B, N, G, D, device=dev).to(dtype)
                sla = torch.cat([torch.rand(B, N, G, L * K * 2, device=dev), torch.randn(B, N, G, L * K, device=dev)], -1).to(dtype)
                go = torch.randn(B, N, G * D, device=dev).to(dtype)
                for direction in ("fwd", "bwd"):
                    cands = attention_candidates(direction)
                    best_ms = [float("inf")] * len(cands)
                    for _ in range(rounds):
                        for ci, (label, options) in enumerate(cands):
                            if direction == "fwd":
                                call = lambda: ext.flash_deform_attn_forward(v, shp, starts, sla, 64, K, 0, 0)
                            else:
                                call = lambda: ext.flash_deform_attn_backward(v, shp, starts, sla, go, 64, K, 0, 0)
                            with ext.launch_options(**options):
                                best_ms[ci] = min(best_ms[ci], _time(call, iters, warm))
                    timings = [(ms,) + c for ms, c in zip(best_ms, cands)]
                    key = launch_spec.attn_table_key(B, N, G, D, L, K, es, direction)
                    _keep(entries, report, key, timings, margin, min_gain_us, lambda best: dict(best[2]), log)
                del v, sla, go
    return entries, report


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--shapes", default="t,b,dense,wide,detr,detr_coco",
                    help="comma-separated shape sets: " + ", ".join(list(SHAPES) + list(ATTN_SHAPES)))
    ap.add_argument("--dtypes", default="float16,float32")
    ap.add_argument("--iters", type=int, default=50)
    ap.add_argument("--margin", type=float, default=0.03)
    ap.add_argument("--min-gain-us", type=float, default=10.0)
    ap.add_argument("--out", default=None, help="table file (default: dcnv4_amd/functions/gfx950_table.json)")
    ap.add_argument("--report", default=None, help="also write every timing to this JSON file")
    ap.add_argument("--library-commit", default=None, help="git commit of the library the table is made on (recorded in the table)")
    args = ap.parse_args(argv)
    import torch
    if not torch.cuda.is_available():
        sys.exit("the tuner needs an MI355X (torch.cuda.is_available() is False)")
    from . import _lib
    from .functions import launch_spec
    entries, report = tune(args.shapes.split(","), args.dtypes.split(","), iters=args.iters, margin=args.margin,
                           min_gain_us=args.min_gain_us)
    table = {"device": torch.cuda.get_device_name(0), "made": time.strftime("%Y-%m-%d"), "abi_version": _lib.ABI_VERSION,
             "library_commit": args.library_commit, "library_sources_sha256": library_sources_sha256(),
             "cases": len(report), "margin": args.margin,
             "min_gain_us": args.min_gain_us, "entries": entries}
    out = args.out or launch_spec.TABLE_PATH
    with open(out, "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
    if args.report:
        with open(args.report, "w") as f:
            json.dump(report, f, indent=1)
    print(f"{len(entries)} of {len(report)} cases beat the library's choice by more than {args.margin:.0%} and "
          f"{args.min_gain_us:g} us; table written to {out}")


if __name__ == "__main__":
    main()
