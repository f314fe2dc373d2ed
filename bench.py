#!/usr/bin/env python3
"""Benchmark of the DCNv4 / flash-deformable-attention hot path on one MI355X.

One "step" is one pass of the hot path over one batch of synthetic input: DCNv4 forward +
backward at the four FlashInternImage-T stage shapes (batch 64, 3x3, group width 16), once
with fp16 and once with fp32 tensors (16 operator calls).  The headline value is the
algorithmic-byte throughput of that step: every tensor counted once in its I/O dtype,
  forward  s*B*Q*(2C + P_pad)      backward  s*B*Q*(3C + 2*P_pad)
divided by the step time, inputs resident in HBM.  Per-operator timings (HIP events on the
stream the kernels run on) for these shapes, the dense-prediction shapes and the
Deformable-DETR attention shape are reported under "detail"; "roofline" describes the operator
that takes the largest share of the step; "cpu_baseline" times the pure-PyTorch grid_sample
formulation of the same operator (oracle/torch_core.py) on the host cores on a reduced batch;
"flash_intern_image_b" is the end-to-end classification forward (batch 128, fp16) with the share of
its time spent inside the DCNv4 operator.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0           # MI355X HBM3E, published
GEOM = (3, 3, 1, 1, 1, 1, 1, 1)  # kh kw sh sw ph pw dh dw

# (name, B, H, W, C, G)
CFG2 = [("T-stage1", 64, 56, 56, 64, 4), ("T-stage2", 64, 28, 28, 128, 8),
        ("T-stage3", 64, 14, 14, 256, 16), ("T-stage4", 64, 7, 7, 512, 32)]
CFG3 = [("L-dense1", 2, 256, 256, 160, 10), ("L-dense2", 2, 128, 128, 320, 20),
        ("L-dense3", 2, 64, 64, 640, 40), ("L-dense4", 2, 32, 32, 1280, 80)]
# per-layer shapes of the FlashInternImage-B forward at batch 128 (offsets U(-3,3) here; the random-init model itself has zero offsets)
CFG5 = [("B-stage1", 128, 56, 56, 112, 7), ("B-stage2", 128, 28, 28, 224, 14),
        ("B-stage3", 128, 14, 14, 448, 28), ("B-stage4", 128, 7, 7, 896, 56)]
CFG4_SHAPES = [(128, 128), (64, 64), (32, 32), (16, 16)]
# the shape of the reference's only timing note (DCNv4_op/scripts/test_dcnv4_bwd.py:94-106: 64 x 56 x 56 x 128, 4 groups of 32)
DEVNOTE = [("ref-note-56x56-C128-G4", 64, 56, 56, 128, 4)]
# groups of 64 channels: two of the reference's tuned keys (DCNv4_op/DCNv4/functions/table.py:452-461, "64x56x56x4x64", "64x28x28x4x64")
WIDE = [("ref-key-56x56-G4-D64", 64, 56, 56, 256, 4), ("ref-key-28x28-G4-D64", 64, 28, 28, 256, 4)]


def p_pad(G, K=9):
    return int(math.ceil(G * K * 3 / 8) * 8)


def dcn_bytes(s, B, H, W, C, G):
    q = B * H * W
    return s * q * (2 * C + p_pad(G)), s * q * (3 * C + 2 * p_pad(G))


def fda_bytes(s, B, N, Q, G, D, L, K):
    v, sla, out = B * N * G * D, B * Q * G * L * K * 3, B * Q * G * D
    return s * (v + sla + out), s * (2 * v + 2 * sla + out)


# HBM bytes moved per operator launch, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of
# `bench.py --only-op <key>`, each counter scaled by its reading for a plain copy of known size
# (`--only-op copy:256`: FETCH_SIZE x 2.0, WRITE_SIZE x 1.0, KiB).  The summaries are in profiles/.
MEASURED_TRAFFIC_BYTES = {
    # (profiles/dcnv4_step_operators_traffic.txt; the backward's excess over its algorithmic bytes: the grad_value kernel reads
    # offset_mask and grad_out a second time, and the fp32 gradients' nontemporal stores are counted in the pieces in which
    # the workgroups that share a line write it)
    "dcnv4_fwd:T-stage1:float16": 96.5e6,      # algorithmic 96.3e6
    "dcnv4_bwd:T-stage1:float16": 238.0e6,     # algorithmic 167.0e6
    "dcnv4_fwd:T-stage2:float16": 47.5e6,      # algorithmic 47.4e6
    "dcnv4_bwd:T-stage2:float16": 116.8e6,     # algorithmic 81.9e6
    "dcnv4_fwd:T-stage3:float16": 23.8e6,      # algorithmic 23.7e6
    "dcnv4_bwd:T-stage3:float16": 51.5e6,      # algorithmic 40.9e6
    "dcnv4_fwd:T-stage4:float16": 12.0e6,      # algorithmic 11.8e6
    "dcnv4_bwd:T-stage4:float16": 23.0e6,      # algorithmic 20.5e6
    "dcnv4_fwd:T-stage1:float32": 192.8e6,     # algorithmic 192.7e6
    "dcnv4_bwd:T-stage1:float32": 550.1e6,     # algorithmic 334.0e6
    "dcnv4_fwd:T-stage2:float32": 94.9e6,      # algorithmic 94.7e6
    "dcnv4_bwd:T-stage2:float32": 262.7e6,     # algorithmic 163.8e6
    "dcnv4_fwd:T-stage3:float32": 47.5e6,      # algorithmic 47.4e6
    "dcnv4_bwd:T-stage3:float32": 121.4e6,     # algorithmic 81.9e6
    "dcnv4_fwd:T-stage4:float32": 23.9e6,      # algorithmic 23.7e6
    "dcnv4_bwd:T-stage4:float32": 45.1e6,      # algorithmic 40.9e6
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--offset-range", type=float, default=None,
                    help="with --only-op dcnv4_*: offsets uniform in +-this many pixels instead of the benchmark's +-3 (+-4 for the dense shapes)")
    ap.add_argument("--far-offset", action="store_true",
                    help="with --only-op dcnv4_*: one sampling point of one pixel is sent 200 pixels away (the robustness row of the detail table)")
    ap.add_argument("--op-iters", type=int, default=100, help="timed launches per operator in the detail table")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-detail", action="store_true", help="skip per-operator timings other than the step's own")
    ap.add_argument("--no-model", action="store_true", help="skip the FlashInternImage-B end-to-end forward")
    ap.add_argument("--no-graph", action="store_true", help="skip the HIP-graph replay of the step (step_graph_ms)")
    ap.add_argument("--only-op", default=None, metavar="OP:SHAPE:DTYPE",
                    help="profiling aid: run just one operator of the step --steps times and exit, e.g. "
                         "dcnv4_bwd:T-stage1:float32 (prints its HIP-event time); also copy:MB for a plain device copy")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this operator has no cross-GPU communication and every box here "
                 "has a single MI355X; run with --gpus 1 (data-parallel scaling is a plain batch split: the operator exchanges nothing between images).")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X (torch.cuda.is_available() is False)")
    from dcnv4_amd import ext
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    torch.manual_seed(0)

    def dcn_inputs(B, H, W, C, G, dtype, off_range):
        K = 9
        value = torch.randn(B, H, W, C, device=dev, dtype=torch.float32)
        om = torch.zeros(B, H, W, p_pad(G), device=dev, dtype=torch.float32)
        body = torch.cat([(torch.rand(B, H, W, G, 2 * K, device=dev) * 2 - 1) * off_range,
                          torch.randn(B, H, W, G, K, device=dev)], -1).reshape(B, H, W, G * K * 3)
        om[..., : G * K * 3] = body
        go = torch.randn(B, H, W, C, device=dev)
        return value.to(dtype), om.to(dtype), go.to(dtype)

    def dcn_fwd(t, G, C):
        return ext.dcnv4_forward(t[0], t[1], *GEOM, G, C // G, 1.0, 64, 0, 0, 0, False)

    def dcn_bwd(t, G, C):
        return ext.dcnv4_backward(t[0], t[1], *GEOM, G, C // G, 1.0, 64, t[2], 0, 0, 0, False)

    def dw_inputs(B, H, W, C, dtype):
        return (torch.randn(B, H, W, C, device=dev).to(dtype), (torch.randn(C, 1, 3, 3, device=dev) / 3).to(dtype),
                torch.randn(C, device=dev).to(dtype), torch.randn(B, H, W, C, device=dev).to(dtype))

    def dw_bytes(s, B, H, W, C):
        # forward: input read + output written; backward: input and grad_out read, grad_input written
        # (grad_weight and grad_bias are C * 10 elements)
        t = B * H * W * C * s
        return 2 * t, 3 * t

    def tail_inputs(B, H, W, C, dtype):
        # the tail of a FlashInternImage block: x + gamma * LayerNorm(y) over rows of C channels
        rows = B * H * W
        return (torch.randn(rows, C, device=dev).to(dtype), torch.randn(rows, C, device=dev).to(dtype),
                (1 + 0.1 * torch.randn(C, device=dev)).to(dtype), (0.1 * torch.randn(C, device=dev)).to(dtype),
                torch.randn(C, device=dev).to(dtype), torch.randn(rows, C, device=dev).to(dtype))

    def tail_bytes(s, B, H, W, C):
        # forward: y and the residual read, the result written; backward: y and grad_out read, grad_y written
        t = B * H * W * C * s
        return 3 * t, 3 * t

    def time_op(fn, iters, warm=None):
        # per-operator timings warm up for as many launches as they time: some kernels (the attention forward with
        # levels staged in LDS) settle only after ~120 launches, while the device's power management follows them
        warm = iters if warm is None else warm
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters      # ms per call

    def stream_ceiling(mb, iters, warm):
        """GB/s (bytes read + bytes written) of the library's own streaming copy over `mb` MB."""
        n = int(mb * 1e6) // 16 * 4
        src, dst = torch.randn(n, device=dev), torch.empty(n, device=dev)
        ms = time_op(lambda: ext.stream_copy(src, dst), iters, warm=warm)
        return ms, n * 4, 2 * n * 4 / (ms * 1e-3) / 1e9

    if args.only_op == "lds_probe":
        # LDS read patterns: ticks per wave-level 16-byte read, and each pattern against the best one
        names = ["consecutive addresses (slot = lane, one cell per wave)", "random cells, slot = lane & 15 (16 lanes cover 256 B)",
                 "random cells, slot = lane & 7 (8 lanes cover 128 B)", "random cells, random slots (a gather of rows)",
                 "random cells, every lane on slot 0"]
        ticks = [min(ext.lds_read_probe(pat, 4000) for _ in range(3)) for pat in range(5)]
        print(json.dumps({"only_op": "lds_probe", "unit": "cycle-counter ticks per wave instruction (ds_read_b128, 16 waves, 8 reads in flight)",
                          "patterns": [{"pattern": n, "ticks": round(t, 2), "vs_best": round(t / min(ticks), 2)} for n, t in zip(names, ticks)]}))
        return

    if args.only_op and args.only_op.startswith("copy:"):
        # plain copy of known size: calibrates FETCH_SIZE / WRITE_SIZE counters and shows the HBM ceiling
        ms, nbytes, gbps = stream_ceiling(float(args.only_op.split(":")[1]), args.steps, args.warmup)
        print(json.dumps({"only_op": args.only_op, "ms": round(ms, 5), "read_MB": nbytes / 1e6, "write_MB": nbytes / 1e6,
                          "GBps_read_plus_write": round(gbps, 1)}))
        return

    def fda_inputs(dtype):
        B, G, D, L, K = 4, 8, 32, 4, 4
        N = sum(h * w for h, w in CFG4_SHAPES)
        shapes = torch.tensor(CFG4_SHAPES, dtype=torch.int64, device=dev)
        sizes = [h * w for h, w in CFG4_SHAPES]
        starts = torch.tensor([sum(sizes[:i]) for i in range(L)], dtype=torch.int64, device=dev)
        v = torch.randn(B, N, G, D, device=dev).to(dtype)
        sla = torch.cat([torch.rand(B, N, G, L * K * 2, device=dev), torch.randn(B, N, G, L * K, device=dev)], -1).to(dtype)
        go = torch.randn(B, N, G * D, device=dev).to(dtype)
        return (B, N, G, D, L, K), shapes, starts, v, sla, go

    if args.only_op and args.only_op.startswith("model:"):
        # FlashInternImage forward only (for profiling): model:<t|s|b|l>:<dtype>, batch 128, --warmup / --steps passes
        from dcnv4_amd.models import flash_intern_image
        _, variant, dt_name = args.only_op.split(":")
        dtype = getattr(torch, dt_name)
        torch.backends.cudnn.benchmark = True         # as the reference's entry point does (classification/main.py:635)
        model = flash_intern_image(variant).to(dev).to(dtype).eval()
        images = torch.randn(128, 3, 224, 224, device=dev).to(dtype)
        with torch.no_grad():
            ms = time_op(lambda: model(images), args.steps, warm=args.warmup)
        print(json.dumps({"only_op": args.only_op, "ms": round(ms, 4), "img_per_s": round(128 / (ms * 1e-3), 1)}))
        return

    if args.only_op:
        op, shape_name, dt_name = args.only_op.split(":")
        dtype = getattr(torch, dt_name)
        if op.startswith("flash_deform_attn"):
            (B, N, G, D, L, K), shapes, starts, v, sla, go = fda_inputs(dtype)
            if op.endswith("fwd"):
                fn = lambda: ext.flash_deform_attn_forward(v, shapes, starts, sla, 64, K, 0, 0)
            else:
                fn = lambda: ext.flash_deform_attn_backward(v, shapes, starts, sla, go, 64, K, 0, 0)
            ms = time_op(fn, args.steps, warm=args.warmup)
            nbytes = fda_bytes(v.element_size(), B, N, N, G, D, L, K)[0 if op.endswith("fwd") else 1]
            print(json.dumps({"only_op": args.only_op, "ms": round(ms, 5), "algorithmic_MB": round(nbytes / 1e6, 2),
                              "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1)}))
            return
        if op.startswith("center_blend"):    # gate = sigmoid(y W^T + b) per (pixel, group); y (1 - gate) + x gate
            for name, B, H, W, C, G in CFG2 + CFG5:
                if name != shape_name:
                    continue
                y, x, _, _, _, go = tail_inputs(B, H, W, C, dtype)
                w, b = (torch.randn(G, C, device=dev) / C ** 0.5).to(dtype), torch.randn(G, device=dev).to(dtype)
                fn = (lambda: ext.center_feature_blend_forward(y, x, w, b)) if op == "center_blend_fwd" else \
                     (lambda: ext.center_feature_blend_backward(go, y, x, w, b))
                ms = time_op(fn, args.steps, warm=args.warmup)
                t = B * H * W * C * y.element_size()
                nbytes = 3 * t if op == "center_blend_fwd" else 5 * t      # y, x in, out; backward: grad_out, y, x in, two gradients out
                print(json.dumps({"only_op": args.only_op, "ms": round(ms, 5), "algorithmic_MB": round(nbytes / 1e6, 2),
                                  "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1)}))
                return
            sys.exit(f"--only-op {args.only_op}: no such shape")
        if op.startswith("block_tail"):      # residual + gamma * LayerNorm(y), forward / backward
            for name, B, H, W, C, G in CFG2 + CFG5:
                if name != shape_name:
                    continue
                y, x, w, b, gamma, go = tail_inputs(B, H, W, C, dtype)
                fn = (lambda: ext.layer_norm_residual_forward(y, x, w, b, gamma, 1e-6)) if op == "block_tail_fwd" else \
                     (lambda: ext.layer_norm_residual_backward(go, y, w, b, gamma, 1e-6))
                ms = time_op(fn, args.steps, warm=args.warmup)
                nbytes = tail_bytes(y.element_size(), B, H, W, C)[0 if op == "block_tail_fwd" else 1]
                print(json.dumps({"only_op": args.only_op, "ms": round(ms, 5), "algorithmic_MB": round(nbytes / 1e6, 2),
                                  "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1)}))
                return
            sys.exit(f"--only-op {args.only_op}: no such shape")
        if op.startswith("depthwise"):       # the offset_mask_dw layer of a DCNv4 block, 3x3, NHWC
            for name, B, H, W, C, G in CFG2 + CFG5:
                if name != shape_name:
                    continue
                x, w, b, go = dw_inputs(B, H, W, C, dtype)
                fn = (lambda: ext.depthwise_conv_forward(x, w, b, 1)) if op == "depthwise_fwd" else \
                     (lambda: ext.depthwise_conv_backward(x, w, go, 1))
                ms = time_op(fn, args.steps, warm=args.warmup)
                nbytes = dw_bytes(x.element_size(), B, H, W, C)[0 if op == "depthwise_fwd" else 1]
                print(json.dumps({"only_op": args.only_op, "ms": round(ms, 5), "algorithmic_MB": round(nbytes / 1e6, 2),
                                  "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1)}))
                return
            sys.exit(f"--only-op {args.only_op}: no such shape")
        for table, off in ((CFG2, 3.0), (CFG3, 4.0), (CFG5, 3.0), (DEVNOTE, 3.0), (WIDE, 3.0)):
            for name, B, H, W, C, G in table:
                if name != shape_name:
                    continue
                t = dcn_inputs(B, H, W, C, G, dtype, off if args.offset_range is None else args.offset_range)
                if args.far_offset:
                    t[1][0, 10, 10, 0] = 200.0
                fn = (lambda: dcn_fwd(t, G, C)) if op == "dcnv4_fwd" else (lambda: dcn_bwd(t, G, C))
                ms = time_op(fn, args.steps, warm=args.warmup)
                nbytes = dcn_bytes(t[0].element_size(), B, H, W, C, G)[0 if op == "dcnv4_fwd" else 1]
                print(json.dumps({"only_op": args.only_op, "ms": round(ms, 5), "algorithmic_MB": round(nbytes / 1e6, 2),
                                  "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1)}))
                return
        sys.exit(f"--only-op {args.only_op}: no such DCNv4 shape")

    # ------------------------------------------------------------------ the step (configs[1])
    work = []
    for dtype, s in ((torch.float16, 2), (torch.float32, 4)):
        for name, B, H, W, C, G in CFG2:
            work.append((name, dtype, s, (B, H, W, C, G), dcn_inputs(B, H, W, C, G, dtype, 3.0)))

    def step():
        for _, _, _, (B, H, W, C, G), t in work:
            dcn_fwd(t, G, C)
            dcn_bwd(t, G, C)

    step_bytes = sum(sum(dcn_bytes(s, *shape)) for _, _, s, shape, _ in work)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # The same step captured once in a HIP graph and replayed: what remains of a step when the host only submits one
    # graph instead of making 16 operator calls (reported beside ms_per_step, never in place of it).
    step_graph_ms = None
    if not args.no_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        step_graph_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        del graph

    # ------------------------------------------------------------------ per-operator detail
    detail = []

    def add(op, name, dtype, ms, nbytes):
        gbps = nbytes / (ms * 1e-3) / 1e9
        detail.append({"op": op, "shape": name, "dtype": str(dtype).replace("torch.", ""), "ms": round(ms, 5),
                       "MB": round(nbytes / 1e6, 2), "GBps": round(gbps, 1), "pct_hbm_peak": round(100 * gbps / HBM_PEAK_GBPS, 2)})

    for name, dtype, s, shape, t in work:
        B, H, W, C, G = shape
        fb, bb = dcn_bytes(s, *shape)
        add("dcnv4_fwd", name, dtype, time_op(lambda: dcn_fwd(t, G, C), args.op_iters), fb)
        add("dcnv4_bwd", name, dtype, time_op(lambda: dcn_bwd(t, G, C), args.op_iters), bb)
    step_ops = list(detail)

    if not args.no_detail:
        for name, B, H, W, C, G in CFG3:
            t = dcn_inputs(B, H, W, C, G, torch.float16, 4.0)
            fb, bb = dcn_bytes(2, B, H, W, C, G)
            add("dcnv4_fwd", name, torch.float16, time_op(lambda: dcn_fwd(t, G, C), args.op_iters), fb)
            add("dcnv4_bwd", name, torch.float16, time_op(lambda: dcn_bwd(t, G, C), args.op_iters), bb)
            if name == "L-dense1":
                # robustness row: the same call with ONE sampling point of one pixel sent 200 pixels away (the backward
                # keeps the common reach for all workgroups but the one that point lands in)
                t[1][0, 10, 10, 0] = 200.0
                add("dcnv4_bwd", name + " + one offset of 200 px", torch.float16, time_op(lambda: dcn_bwd(t, G, C), max(10, args.op_iters // 5)), bb)
            del t
        for name, B, H, W, C, G in DEVNOTE + WIDE:
            t = dcn_inputs(B, H, W, C, G, torch.float16, 3.0)
            fb, bb = dcn_bytes(2, B, H, W, C, G)
            add("dcnv4_fwd", name, torch.float16, time_op(lambda: dcn_fwd(t, G, C), args.op_iters), fb)
            add("dcnv4_bwd", name, torch.float16, time_op(lambda: dcn_bwd(t, G, C), args.op_iters), bb)
            del t
        for name, B, H, W, C, G in CFG5:
            t = dcn_inputs(B, H, W, C, G, torch.float16, 3.0)
            add("dcnv4_fwd", name, torch.float16, time_op(lambda: dcn_fwd(t, G, C), args.op_iters), dcn_bytes(2, B, H, W, C, G)[0])
            del t
            x, w, b, go = dw_inputs(B, H, W, C, torch.float16)
            add("depthwise_fwd", name, torch.float16, time_op(lambda: ext.depthwise_conv_forward(x, w, b, 1), args.op_iters),
                dw_bytes(2, B, H, W, C)[0])
            add("depthwise_bwd", name, torch.float16, time_op(lambda: ext.depthwise_conv_backward(x, w, go, 1), args.op_iters),
                dw_bytes(2, B, H, W, C)[1])
            del x, w, b, go
            if name == "B-stage1":
                y, x, w, b, gamma, go = tail_inputs(B, H, W, C, torch.float16)
                add("block_tail_fwd", name, torch.float16, time_op(lambda: ext.layer_norm_residual_forward(y, x, w, b, gamma, 1e-6), args.op_iters),
                    tail_bytes(2, B, H, W, C)[0])
                add("block_tail_bwd", name, torch.float16, time_op(lambda: ext.layer_norm_residual_backward(go, y, w, b, gamma, 1e-6), args.op_iters),
                    tail_bytes(2, B, H, W, C)[1])
                del w, b, gamma
                # the centre-feature blend of a DCNv4 layer (off in the FlashInternImage configs): y, x in, out; backward
                # grad_out, y, x in, two gradients out
                G7 = G
                w = (torch.randn(G7, C, device=dev) / C ** 0.5).to(torch.float16)
                b = torch.randn(G7, device=dev).to(torch.float16)
                t_bytes = B * H * W * C * 2
                add("center_blend_fwd", name, torch.float16, time_op(lambda: ext.center_feature_blend_forward(y, x, w, b), args.op_iters), 3 * t_bytes)
                add("center_blend_bwd", name, torch.float16, time_op(lambda: ext.center_feature_blend_backward(go, y, x, w, b), args.op_iters), 5 * t_bytes)
                del y, x, w, b, go
        for dtype, s in ((torch.float16, 2), (torch.float32, 4)):
            (B, N, G, D, L, K), shapes, starts, v, sla, go = fda_inputs(dtype)
            fb, bb = fda_bytes(s, B, N, N, G, D, L, K)
            add("flash_deform_attn_fwd", "DETR-enc 4lvl Q=21760", dtype,
                time_op(lambda: ext.flash_deform_attn_forward(v, shapes, starts, sla, 64, K, 0, 0), args.op_iters), fb)
            add("flash_deform_attn_bwd", "DETR-enc 4lvl Q=21760", dtype,
                time_op(lambda: ext.flash_deform_attn_backward(v, shapes, starts, sla, go, 64, K, 0, 0), args.op_iters), bb)
            del v, sla, go

    # ------------------------------------------------------------------ FlashInternImage-B end to end (configs[4])
    model_line = None
    if not args.no_model:
        from dcnv4_amd.models import flash_intern_image
        torch.backends.cudnn.benchmark = True         # as the reference's entry point does (classification/main.py:635)
        model = flash_intern_image("b").to(dev).half().eval()
        images = torch.randn(128, 3, 224, 224, device=dev).half()
        spans = []                                    # (start, end) events around every DCNv4 operator call
        real_forward = ext.dcnv4_forward

        def timed_forward(*a):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            out = real_forward(*a)
            e1.record()
            spans.append((e0, e1))
            return out

        with torch.no_grad():
            for _ in range(50):                       # protocol of the reference's throughput(): 50 warm-up, 30 timed
                model(images)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(30):
                model(images)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            ext.dcnv4_forward = timed_forward
            try:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(5):
                    model(images)
                e1.record()
                torch.cuda.synchronize()
            finally:
                ext.dcnv4_forward = real_forward
            op_ms = sum(a.elapsed_time(b) for a, b in spans)
            total_ms = e0.elapsed_time(e1)
        model_line = {"model": "FlashInternImage-B, random init, eval forward, fp16, batch 128, 224x224, synthetic input",
                      "img_per_s": round(30 * 128 / dt, 1), "ms_per_batch": round(dt / 30 * 1e3, 3),
                      "dcnv4_calls_per_forward": len(spans) // 5,
                      "dcnv4_kernel_share": round(op_ms / total_ms, 4)}
        del model, images

    # ------------------------------------------------------------------ roofline of the dominant operator
    dom = max(step_ops, key=lambda d: d["ms"])
    dom_bytes = dom["MB"] * 1e6
    _, _, ceiling = stream_ceiling(512, 50, 10)
    roofline = {
        "bound": "hbm", "achieved": dom["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": round(dom["GBps"] / HBM_PEAK_GBPS, 4),
        "traffic": MEASURED_TRAFFIC_BYTES.get(f'{dom["op"]}:{dom["shape"]}:{dom["dtype"]}'),
        "kernel": f'{dom["op"]} {dom["shape"]} {dom["dtype"]}', "ms": dom["ms"],
        "algorithmic_bytes": int(dom_bytes),
        "measured_ceiling": round(ceiling, 1), "frac_of_measured_ceiling": round(dom["GBps"] / ceiling, 4),
        "note": "HIP events around whole operator calls (backward = state reset + grad_offset_mask kernel + tiled grad_value kernel); measured_ceiling = read+write GB/s of the library's own streaming copy over 512 MB in this run; traffic = rocprofv3 FETCH_SIZE/WRITE_SIZE per call, scaled by a copy of known size (profiles/)",
    }

    # ------------------------------------------------------------------ CPU baseline (rank 0, bounded sample)
    # The pure-PyTorch grid_sample formulation on the host cores: 2 warm-ups, median of 5, forward and
    # forward+backward separately.  `value` is the forward+backward rate over the step's own four shapes on a batch
    # sample; `detail` adds configs[0] (its full size, batch 2) and one image of the attention configuration.
    cpu = None
    if not args.no_cpu_baseline:
        import statistics
        from oracle import torch_core
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
        torch.set_num_threads(cores)

        def cpu_times(fwd_fn, leaves, go):
            def f():
                with torch.no_grad():
                    fwd_fn()

            def fb():
                out = fwd_fn()
                out.backward(go)
                for t in leaves:
                    t.grad = None
            res = []
            for fn in (f, fb):
                for _ in range(2):
                    fn()
                ts = []
                for _ in range(5):
                    t0 = time.perf_counter()
                    fn()
                    ts.append(time.perf_counter() - t0)
                res.append(statistics.median(ts))
            return res      # seconds: forward, forward+backward

        cpu_detail = []
        Bc = 8
        cpu_bytes, cpu_time = 0, 0.0
        for cfg_name, table, Bs, off in (("cfg1", [("56x56 C64 G4", 2, 56, 56, 64, 4)], None, 2.0), ("cfg2", CFG2, Bc, 3.0)):
            for name, B, H, W, C, G in table:
                Bn = B if Bs is None else Bs
                v, om, go = (x.cpu().float().contiguous() for x in dcn_inputs(Bn, H, W, C, G, torch.float32, off))
                v.requires_grad_(True)
                om.requires_grad_(True)
                tf, tfb = cpu_times(lambda: torch_core.dcnv4_core_torch(v, om, *GEOM, G, C // G, 1.0), (v, om), go)
                cpu_detail.append({"config": cfg_name, "shape": name, "batch": Bn, "fwd_ms": round(tf * 1e3, 2), "fwd_bwd_ms": round(tfb * 1e3, 2)})
                if cfg_name == "cfg2":
                    cpu_time += tfb
                    cpu_bytes += sum(dcn_bytes(4, Bn, H, W, C, G))
        (B4, N4, G4, D4, L4, K4), shapes4, starts4, v4, sla4, go4 = fda_inputs(torch.float32)
        v1, s1, g1 = v4[:1].cpu().contiguous().requires_grad_(True), sla4[:1].cpu().contiguous().requires_grad_(True), go4[:1].cpu().contiguous()
        tf, tfb = cpu_times(lambda: torch_core.msda_core_torch(v1, CFG4_SHAPES, [int(x) for x in starts4.cpu()], s1, K4), (v1, s1), g1)
        cpu_detail.append({"config": "cfg4", "shape": "DETR-enc 4lvl Q=21760", "batch": 1, "fwd_ms": round(tf * 1e3, 2), "fwd_bwd_ms": round(tfb * 1e3, 2)})
        del v4, sla4, go4
        cpu = {"value": round(cpu_bytes / cpu_time / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": f"DCNv4 fwd+bwd, four FlashInternImage-T stage shapes at batch {Bc} (of 64), fp32, torch grid_sample "
                         f"formulation + autograd, median of 5 after 2 warm-ups, {cpu_time * 1e3:.0f} ms per pass; detail: "
                         "configs[0] at its full batch 2, configs[1] at batch 8, configs[3] one image of 4",
               "detail": cpu_detail}

    line = {
        "metric": "DCNv4 fwd+bwd achieved HBM GB/s (algorithmic bytes / time)", "value": round(value, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "step_graph_ms": None if step_graph_ms is None else round(step_graph_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "DCNv4 forward+backward, FlashInternImage-T stages (56x56 C64 G4, 28x28 C128 G8, "
                               "14x14 C256 G16, 7x7 C512 G32), batch 64, 3x3 s1 p1, fp16 and fp32 tensors, fp32 arithmetic",
                   "step_algorithmic_MB": round(step_bytes / 1e6, 1), "pct_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2)},
        "roofline": roofline, "cpu_baseline": cpu, "detail": detail, "flash_intern_image_b": model_line,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
