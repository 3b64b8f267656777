#!/usr/bin/env python3
"""Roofline benchmark of the depthwise oriented 1D convolution on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: fprop, dgrad and
wgrad at each of the four ConvNeXt-T stage shapes (batch 64, K=31, theta_c = (c mod 8)*22.5
degrees), i.e. 12 launches of the C-ABI entry points.  Inputs are resident in HBM before the
timed region; buffer sets rotate so consecutive steps do not re-hit the 256 MB Infinity Cache.

Timing protocol.  The first 20-30 ms of any burst of launches after an idle spell run up to 25 %
slower than what follows (the power management settles the clocks); every measurement here is
taken in the sustained state a continuous job runs in: the step loop is preceded by untimed
steps, every per-kernel timing by at least 40 ms of launches of that kernel, and the median of
20 repeats of 100 back-to-back launches is reported (`us`: rotating buffers, more than twice
the 256 MB Infinity Cache per operator; `warm_us`: one fixed buffer set).  The step time right
after the idle spell is listed beside it (`ms_per_step_first_window`).

Prints ONE JSON line: `value` is the algorithmic GB/s of the whole step (sum of the 12
operators' algorithmic bytes / step time, eager C-ABI calls); `detail` carries GB/s and the
HBM-roofline fraction of every (shape, op); `roofline` is the dominant kernel, i.e. the one of
the twelve with the longest launch, timed with events on the launch stream, and `roofline_min`
the lowest fraction among the twelve; `cpu_baseline` is the oracle's single-thread
reference-order loops on a bounded sample of the same workload; `table5` repeats the
reference's own micro-benchmark (analysis/benchmark.py:19-67,84-104).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E peak
STAGES = [(96, 56), (192, 28), (384, 14), (768, 7)]
BATCH, KSIZE = 64, 31
ELEM = {"f32": 4, "bf16": 2, "f16": 2}


def algorithmic_bytes(op, N, C, H, W, K, b, stride=1):
    """Bytes an ideal implementation moves: each activation tensor once, plus weights and
    the int8 tap table (fprop/dgrad) or the dw output (wgrad).  No halo re-reads, no
    transposes, no reduction scratch."""
    P, Q = -(-H // stride), -(-W // stride)
    act = (N * C * H * W + N * C * P * Q) * b
    if op == "wgrad":
        return act + C * K * 4
    return act + C * K * 4 + C * K * 2


VALU_LANES = 256 * 4 * 16   # CUs x SIMDs x lanes: one fp32 multiply-add per lane and cycle
PEAK_CLOCK_HZ = 2.4e9       # MI355X peak engine clock


def issue_bound_us(op_mod, theta, C, HW, K, N, clock_hz=PEAK_CLOCK_HZ):
    """Second bound of a launch beside the HBM one: the time its multiply-adds alone occupy
    the vector ALUs.  Per output one multiply-add per distinct tap offset that can reach the
    plane (taps that truncation puts on the same pixel are folded into one weight, taps with
    |dh| >= H or |dw| >= W only ever read zeros); the chip issues VALU_LANES of them per cycle
    (packed fp32 is switched off for this library and a depthwise stencil has nothing for the
    matrix cores).  Priced at the peak clock, so a lower bound of the bound: the sustained
    clock under this load is lower."""
    import torch

    dh, dw = op_mod.taps_to_numpy(op_mod.build_taps(torch.from_numpy(theta), C, K), C, K)
    fmas = 0
    for c in range(C):
        live = {(int(a), int(b)) for a, b in zip(dh[c], dw[c]) if abs(a) < HW and abs(b) < HW}
        fmas += len(live)
    return fmas * N * HW * HW / VALU_LANES / clock_hz * 1e6


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--dtype", default="f32", choices=list(ELEM))
    ap.add_argument("--layout", default="nchw", choices=["nchw", "nhwc"])
    ap.add_argument("--theta", default="roundrobin", choices=["roundrobin", "grouped", "arbitrary"])
    ap.add_argument("--precondition-ms", type=float, default=60.0,
                    help="untimed steps run for this long before the warm-up steps, so that the "
                         "timed steps see the clocks of a continuous job")
    ap.add_argument("--kernel-warm-ms", type=float, default=40.0,
                    help="untimed launches of a kernel before its per-kernel timing")
    ap.add_argument("--kernel-iters", type=int, default=100,
                    help="back-to-back launches per (shape, op) for the per-kernel timings")
    ap.add_argument("--kernel-repeats", type=int, default=20,
                    help="repeats of the per-kernel measurement (the median is reported)")
    ap.add_argument("--no-graph", dest="graph", action="store_false",
                    help="skip the two informational hipGraph timings of the step (`value` is "
                         "always the eager C-ABI calls)")
    ap.add_argument("--table5-iters", type=int, default=20,
                    help="timed iterations per angle of the reference's Table-5 protocol "
                         "(the reference uses 100); 0 skips it")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra-sweeps", action="store_true",
                    help="skip the bf16 / NHWC / grouped-angle rows (other_configs)")
    ap.add_argument("--arbitrary-row", action="store_true",
                    help="add the other_configs row with angles that are no multiples of 22.5 degrees")
    ap.add_argument("--only", default="", help="restrict the per-kernel table, e.g. 96x56:fprop")
    ap.add_argument("--model-iters", type=int, default=5,
                    help="timed ConvNeXt-T-1D inference forwards (batch 128, bf16); 0 skips it")
    ap.add_argument("--train-iters", type=int, default=3,
                    help="timed steps of the two training configurations (ConvNeXt-B-1D++ "
                         "training, ConvNeXt-T-1D features fwd+bwd); 0 skips them")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run a plain device copy of one 96x56x56 batch-64 tensor (a kernel "
                         "of known traffic, for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (fprop and dgrad have no cross-GPU "
              "exchange, wgrad would need one all-reduce of dw); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from oriented1d_amd import dwoconv1d as op

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")

    import ctypes

    from oriented1d_amd import _lib
    lib = _lib.ready(dev)  # dwo_init: every kernel set up before anything is captured or timed
    # everything runs on one side stream: its handle is what the C ABI launches on, what the
    # timing events are recorded on, and what the step graphs are captured from
    stream = torch.cuda.Stream(dev)
    torch.cuda.set_stream(stream)
    stream_h = ctypes.c_void_p(stream.cuda_stream)

    def theta_for(C, kind):
        if kind == "roundrobin":
            return np.array([(c % 8) * math.pi / 8 for c in range(C)], dtype=np.float32)
        if kind == "arbitrary":  # no multiple of 22.5 degrees among them: the table-driven bodies
            return np.array([0.1 + (c % 8) * 0.37 for c in range(C)], dtype=np.float32)
        return np.array([math.pi * (((8 * (c + 1) - 1) // C) / 8) for c in range(C)],
                        dtype=np.float32)

    def vp(t):
        return ctypes.c_void_p(t.data_ptr())

    def sweep(dtype, layout, theta, steps, warmup, kernel_iters, kernel_repeats, only="",
              warm=False):
        """Whole-step time (when steps > 0) and per-(shape, op) kernel times of one
        configuration.  Inputs are resident before anything is timed; nsets buffer sets rotate
        so consecutive launches do not re-hit the 256 MB Infinity Cache ("cold" numbers); with
        warm=True every launch of an operator also runs on one fixed set ("warm_us")."""
        tdt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[dtype]
        b = ELEM[dtype]
        nhwc = layout == "nhwc"
        g = torch.Generator(device=dev).manual_seed(0)
        # buffer sets per stage: the two tensors an operator touches, times the sets it rotates
        # through, exceed twice the Infinity Cache (5 / 8 / 15 / 28 sets for fp32)
        nsets_of = [max(2, math.ceil(2 * 256e6 / (2 * BATCH * C * HW * HW * b)) + 1)
                    for C, HW in STAGES]
        nsets = nsets_of[0]
        dt_code, lay_code = {"f32": 0, "bf16": 1, "f16": 2}[dtype], int(nhwc)
        keep, calls = [], [[] for _ in STAGES]  # calls[stage][set][op] -> zero-argument callable
        for si, (C, HW) in enumerate(STAGES):
            per_stage = calls[si]
            for _ in range(nsets_of[si]):
                shape = (BATCH, HW, HW, C) if nhwc else (BATCH, C, HW, HW)
                x = torch.randn(shape, device=dev, generator=g).to(tdt)
                dy = torch.randn(shape, device=dev, generator=g).to(tdt)
                w2 = (torch.randn(C, KSIZE, device=dev, generator=g) * 0.02).contiguous()
                taps = op.build_taps(torch.from_numpy(theta_for(C, theta)), C, KSIZE).to(dev)
                # outputs and wgrad scratch are allocated once; the timed region holds nothing
                # but the C-ABI calls (ctypes arguments are converted up front)
                y = torch.empty_like(x)
                dx = torch.empty_like(x)
                dw = torch.empty(C, KSIZE, device=dev)
                nb = lib.dwo_wgrad_scratch_bytes(BATCH, C, HW, HW, KSIZE, 1, dt_code, lay_code)
                scr = torch.empty(max(nb, 16), dtype=torch.uint8, device=dev)
                keep.extend([x, dy, w2, taps, y, dx, dw, scr])
                dims = (BATCH, C, HW, HW, KSIZE, 1, dt_code, lay_code)
                fa = (vp(x), vp(w2), None, vp(taps), vp(y)) + dims
                da = (vp(dy), vp(w2), vp(taps), vp(dx)) + dims
                wa = (vp(dy), vp(x), vp(taps), vp(dw), None, vp(scr), nb) + dims
                per_stage.append({
                    "fprop": (lambda sh=stream_h, a=fa: lib.dwo_fprop(*a, sh)),
                    "dgrad": (lambda sh=stream_h, a=da: lib.dwo_dgrad(*a, sh)),
                    "wgrad": (lambda sh=stream_h, a=wa: lib.dwo_wgrad(*a, sh)),
                    "out": (y, dx, dw),
                })

        def checked_pass():
            """Every call of every buffer set once, with its status checked and its outputs
            tested for non-finite values."""
            for per_stage in calls:
                for ops in per_stage:
                    for name in ("fprop", "dgrad", "wgrad"):
                        _lib.check(ops[name](), "dwo_" + name)
            torch.cuda.synchronize()
            for per_stage in calls:
                for ops in per_stage:
                    for t in ops["out"]:
                        if not bool(torch.isfinite(t).all()):
                            raise RuntimeError("non-finite values in an operator output")

        checked_pass()  # any launch error surfaces here, before anything is timed

        def step(i):
            for si in range(len(STAGES)):
                ops = calls[si][i % nsets_of[si]]
                ops["fprop"]()
                ops["dgrad"]()
                ops["wgrad"]()

        step_bytes = sum(algorithmic_bytes(o, BATCH, C, HW, HW, KSIZE, b)
                         for C, HW in STAGES for o in ("fprop", "dgrad", "wgrad"))
        ms_per_step, ms_eager, ms_branches, ms_graph, ms_first = None, None, None, None, None
        n_pre = 0

        def precondition():
            """Untimed steps for args.precondition_ms: the clocks of a continuous job."""
            n, t0 = 0, time.perf_counter()
            while (time.perf_counter() - t0) * 1e3 < args.precondition_ms:
                for _ in range(8):
                    step(n)
                    n += 1
                torch.cuda.synchronize()
            return n

        def timed_steps():
            for i in range(warmup):
                step(i)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(steps):
                step(i)
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) * 1e3 / steps

        if steps > 0:
            time.sleep(0.3)  # the GPU idles: what a first call after a pause sees
            ms_first = timed_steps()
            n_pre = precondition()
            ms_eager = timed_steps()
            ms_per_step = ms_eager
            if args.graph:
                # For information (not `value`): the same 12 C-ABI calls per step, captured once
                # per buffer set and replayed
                graphs = []
                for i in range(nsets):
                    gr = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(gr, stream=stream):
                        step(i)
                    graphs.append(gr)
                precondition()
                for i in range(warmup):
                    graphs[i % nsets].replay()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for i in range(steps):
                    graphs[i % nsets].replay()
                torch.cuda.synchronize()
                ms_graph = (time.perf_counter() - t0) * 1e3 / steps
                del graphs
                # For information (not `value`): the same step with fprop, dgrad and wgrad of a
                # shape on three parallel branches of the graph (they do not depend on each other;
                # in a training step dgrad and wgrad of a layer do not either), so the fill and
                # drain of one kernel overlaps its neighbours'.
                side = [torch.cuda.Stream(dev), torch.cuda.Stream(dev)]
                side_h = [ctypes.c_void_p(s_.cuda_stream) for s_ in side]
                graphs = []
                for i in range(nsets):
                    gr = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(gr, stream=stream):
                        for s_ in side:
                            s_.wait_stream(stream)
                        for si in range(len(STAGES)):
                            ops = calls[si][i % nsets_of[si]]
                            ops["fprop"]()
                            ops["dgrad"](side_h[0])
                            ops["wgrad"](side_h[1])
                        for s_ in side:
                            stream.wait_stream(s_)
                    graphs.append(gr)
                precondition()
                for i in range(warmup):
                    graphs[i % nsets].replay()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for i in range(steps):
                    graphs[i % nsets].replay()
                torch.cuda.synchronize()
                ms_branches = (time.perf_counter() - t0) * 1e3 / steps
                del graphs
            checked_pass()  # the timed calls discard their status: re-check every set afterwards

        # per-kernel timings: HIP events on the launch stream (torch's current stream is the
        # one passed to the C ABI), median over the repeats
        def timed(name, si, fixed):
            fns = [ops[name] for ops in calls[si]]
            if fixed:
                fns = fns[:1]
            n, t0 = 0, time.perf_counter()
            while n < 10 or (time.perf_counter() - t0) * 1e3 < args.kernel_warm_ms:
                for _ in range(20):
                    fns[n % len(fns)]()
                    n += 1
                torch.cuda.synchronize()
            reps = []
            for _ in range(kernel_repeats):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for i in range(kernel_iters):
                    fns[i % len(fns)]()
                e1.record(stream)
                torch.cuda.synchronize()
                reps.append(e0.elapsed_time(e1) * 1e3 / kernel_iters)
            return sorted(reps)[len(reps) // 2]

        issue_us = [issue_bound_us(op, theta_for(C, theta), C, HW, KSIZE, BATCH) for C, HW in STAGES]
        detail = {}
        for si, (C, HW) in enumerate(STAGES):
            for name in ("fprop", "dgrad", "wgrad"):
                key = "%dx%d:%s" % (C, HW, name)
                if only and only != key:
                    continue
                us = timed(name, si, False)
                ab = algorithmic_bytes(name, BATCH, C, HW, HW, KSIZE, b)
                gbs = ab / (us * 1e-6) / 1e9
                detail[key] = {"us": round(us, 2), "GB/s": round(gbs, 1),
                               "frac_hbm": round(gbs / HBM_PEAK_GBS, 4), "bytes": ab,
                               "hbm_bound_us": round(ab / HBM_PEAK_GBS / 1e3, 2),
                               "issue_bound_us": round(issue_us[si], 2)}
                if warm:
                    detail[key]["warm_us"] = round(timed(name, si, True), 2)
        copy_src = keep[0]
        res = {"ms_per_step": ms_per_step, "ms_per_step_eager": ms_eager,
               "ms_per_step_first_window": ms_first, "precondition_steps": n_pre,
               "nsets_per_stage": nsets_of,
               "ms_per_step_branches": ms_branches, "ms_per_step_graph": ms_graph, "detail": detail,
               "nsets": nsets,
               "step_bytes": step_bytes, "copy_src": copy_src if args.calibration_copy else None}
        return res

    main_res = sweep(args.dtype, args.layout, args.theta, args.steps, args.warmup,
                     args.kernel_iters, args.kernel_repeats, args.only, warm=True)
    ms_per_step, detail = main_res["ms_per_step"], main_res["detail"]
    main_res_eager = main_res["ms_per_step_eager"]
    main_res_graph, main_res_branches = main_res["ms_per_step_graph"], main_res["ms_per_step_branches"]
    nsets, step_bytes = main_res["nsets"], main_res["step_bytes"]
    nsets_per_stage, ms_first = main_res["nsets_per_stage"], main_res["ms_per_step_first_window"]
    n_pre = main_res["precondition_steps"]
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    if args.calibration_copy:
        src = main_res["copy_src"]
        dstc = torch.empty_like(src)
        for _ in range(3):
            dstc.copy_(src)
        torch.cuda.synchronize()

    # HBM bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by what the same
    # counter reads for a plain copy of known size: the figures and the commands that produced
    # them are committed under profiles/ (a .md summary and the same numbers as .json); only
    # valid for the configuration they were measured on.
    traffic = {}
    tpath = os.path.join(ROOT, "profiles", "dwoconv1d_stage_sweep_%s_%s_hbm_traffic.json"
                         % (args.dtype, args.layout))
    if args.theta == "roundrobin" and os.path.exists(tpath):
        with open(tpath) as fh:
            traffic = json.load(fh).get("traffic_bytes_per_launch", {})

    # the dominant kernel is the one of the twelve with the longest launch
    roofline, roofline_min = None, None
    if detail:
        dom_key = max(detail, key=lambda k: detail[k]["us"])
        dom = detail[dom_key]
        C_, rest = dom_key.split("x")
        HW_, op_ = rest.split(":")
        roofline = {"bound": "hbm",
                    "kernel": "%s C=%s %sx%s N=%d %s %s" % (op_, C_, HW_, HW_, BATCH, args.dtype,
                                                           args.layout),
                    "achieved": dom["GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(dom["GB/s"] / HBM_PEAK_GBS, 4),
                    "traffic": traffic.get(dom_key),
                    "launch_us": dom["us"], "algorithmic_bytes": dom["bytes"],
                    "hbm_bound_us": dom["hbm_bound_us"], "issue_bound_us": dom["issue_bound_us"],
                    "binding_bound": "hbm" if dom["hbm_bound_us"] >= dom["issue_bound_us"] else "valu issue",
                    "issue_bound": "multiply-adds after folding duplicate and dead taps / (%d lanes "
                                   "x %.1f GHz peak clock), no packed fp32, no matrix cores"
                                   % (VALU_LANES, PEAK_CLOCK_HZ / 1e9)}
        low_key = min(detail, key=lambda k: detail[k]["frac_hbm"])
        roofline_min = {"kernel": low_key, "frac": detail[low_key]["frac_hbm"],
                        "launch_us": detail[low_key]["us"],
                        "ops_at_or_above_0.60": sum(v["frac_hbm"] >= 0.6 for v in detail.values()),
                        "ops": len(detail)}

    # ------------------------------------------------------------------ the other rows
    # Same sweep in the other element type / layout / angle assignment (per-kernel times only,
    # same launches per timing and repeats as the main table): bf16 NCHW, fp32 and bf16 NHWC-native, fp32 NCHW with the networks'
    # contiguous-group angles, and, with --arbitrary-row, fp32 NCHW with angles that are no multiples of
    # 22.5 degrees (every channel on the table-driven bodies; not in the default run: those launches
    # carry the same kernel names and grids as the main sweep's and would blur a kernel trace of it).
    others = {}
    if not args.no_extra_sweeps and not args.only:
        for dt_, lay_, th_ in (("bf16", "nchw", "roundrobin"), ("f32", "nhwc", "roundrobin"),
                               ("bf16", "nhwc", "roundrobin"), ("f32", "nchw", "grouped"),
                               ("f32", "nchw", "arbitrary")):
            if th_ == "arbitrary" and not args.arbitrary_row:
                continue
            if (dt_, lay_, th_) == (args.dtype, args.layout, args.theta):
                continue
            r = sweep(dt_, lay_, th_, 0, 0, args.kernel_iters, args.kernel_repeats)
            tot_us = sum(v["us"] for v in r["detail"].values())
            tr_ = {}
            tp_ = os.path.join(ROOT, "profiles", "dwoconv1d_stage_sweep_%s_%s_hbm_traffic.json"
                               % (dt_, lay_))
            if th_ == "roundrobin" and os.path.exists(tp_):
                with open(tp_) as fh:
                    tr_ = json.load(fh).get("traffic_bytes_per_launch", {})
            others["%s/%s/%s" % (dt_, lay_, th_)] = {
                "sum_us": round(tot_us, 1),
                "GB/s": round(r["step_bytes"] / tot_us / 1e3, 1),
                "ops": {k: [v["us"], v["frac_hbm"]] for k, v in r["detail"].items()},
                "traffic": {k: tr_.get(k) for k in r["detail"]} if tr_ else None}
            torch.cuda.empty_cache()

    # ------------------------------------------------------------------ shapes without planes
    # Per-kernel times of shapes outside the sweep, bf16, the networks' contiguous-group angles:
    # on the tile kernels (any extent, stride and layout) the two stem convolutions of the networks
    # at batch 128 (NHWC, stride 2) and the stage shapes of a 512 x 512 input at batch 8 (NCHW); on
    # the NHWC plane kernels the second convolution of the ConvNeXt-B-1D++ blocks at batch 64
    # (4 x dim channels: the launches of the training configuration).
    other_shapes = {}
    if not args.no_extra_sweeps and not args.only:
        for tag, (N_, C_, HW_, st_, lay_) in (
                ("stem1 128x64x224 s2 nhwc", (128, 64, 224, 2, "nhwc")),
                ("stem2 128x64x112 s2 nhwc", (128, 64, 112, 2, "nhwc")),
                ("8x96x128 nchw", (8, 96, 128, 1, "nchw")), ("8x192x64 nchw", (8, 192, 64, 1, "nchw")),
                ("8x384x32 nchw", (8, 384, 32, 1, "nchw")), ("8x768x16 nchw", (8, 768, 16, 1, "nchw")),
                ("64x512x56 nhwc", (64, 512, 56, 1, "nhwc")), ("64x1024x28 nhwc", (64, 1024, 28, 1, "nhwc")),
                ("64x2048x14 nhwc", (64, 2048, 14, 1, "nhwc")), ("64x4096x7 nhwc", (64, 4096, 7, 1, "nhwc"))):
            nhwc = lay_ == "nhwc"
            PQ = -(-HW_ // st_)
            g = torch.Generator(device=dev).manual_seed(1)
            xs = (N_, HW_, HW_, C_) if nhwc else (N_, C_, HW_, HW_)
            ys = (N_, PQ, PQ, C_) if nhwc else (N_, C_, PQ, PQ)
            x = torch.randn(xs, device=dev, generator=g).to(torch.bfloat16)
            dy = torch.randn(ys, device=dev, generator=g).to(torch.bfloat16)
            w2 = (torch.randn(C_, KSIZE, device=dev, generator=g) * 0.02).contiguous()
            taps = op.build_taps(torch.from_numpy(theta_for(C_, "grouped")), C_, KSIZE).to(dev)
            y, dx = torch.empty_like(dy), torch.empty_like(x)
            dw = torch.empty(C_, KSIZE, device=dev)
            nb = lib.dwo_wgrad_scratch_bytes(N_, C_, HW_, HW_, KSIZE, st_, 1, int(nhwc))
            scr = torch.empty(max(nb, 16), dtype=torch.uint8, device=dev)
            dims = (N_, C_, HW_, HW_, KSIZE, st_, 1, int(nhwc), stream_h)
            fns = {"fprop": (lambda a=(vp(x), vp(w2), None, vp(taps), vp(y)) + dims: lib.dwo_fprop(*a)),
                   "dgrad": (lambda a=(vp(dy), vp(w2), vp(taps), vp(dx)) + dims: lib.dwo_dgrad(*a)),
                   "wgrad": (lambda a=(vp(dy), vp(x), vp(taps), vp(dw), None, vp(scr), nb) + dims:
                             lib.dwo_wgrad(*a))}
            row = {}
            torch.cuda.synchronize()  # inputs were made on torch's stream, the calls run on `stream`
            outs_ = {"fprop": y, "dgrad": dx, "wgrad": dw}
            for name, fn in fns.items():
                _lib.check(fn(), "dwo_" + name)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                while (time.perf_counter() - t0) * 1e3 < args.kernel_warm_ms:
                    for _ in range(5):
                        fn()
                    torch.cuda.synchronize()
                reps = []
                for _ in range(5):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(stream)
                    for _ in range(20):
                        fn()
                    e1.record(stream)
                    torch.cuda.synchronize()
                    reps.append(e0.elapsed_time(e1) * 50.0)
                us = sorted(reps)[2]
                ab = algorithmic_bytes(name, N_, C_, HW_, HW_, KSIZE, 2, st_)
                if not bool(torch.isfinite(outs_[name]).all()):
                    raise RuntimeError("non-finite values in %s of %s" % (name, tag))
                row[name] = [round(us, 1), round(ab / us / 1e3 / HBM_PEAK_GBS, 4)]
            other_shapes[tag] = row
            del x, dy, y, dx, scr
            torch.cuda.empty_cache()

    # ------------------------------------------------------------------ the reference's Table 5
    # analysis/benchmark.py:19-67,84-104: one depthwise layer through the module and autograd,
    # N=64, C=512, fp32, bias=False, stride 1, H=W in {14, 28, 56}, K in {7, 31}, one angle for all
    # channels; per angle 10 warm-up iterations, then the mean wall-clock of `y = model(x);
    # (y.mean() * 1024).backward()` between synchronisations, averaged over the eight angles.  x
    # does not require a gradient there, so "fwd+bwd" is fprop + wgrad + the loss kernels.  The
    # script passes its angles in degrees to a module that reads radians (and 66.75 for 67.5):
    # "as_published" feeds those same numbers (non-canonical tap patterns: table-driven bodies),
    # "canonical" the eight orientations k * 22.5 degrees the table's header means.  Published
    # (README.md:318-327, one RTX 3090): 0.3/0.8, 0.9/2.6, 3.2/9.9 ms for K=7/31.
    table5 = None
    if args.table5_iters > 0 and not args.only:
        from oriented1d_amd.dwoconv1d import DepthwiseOrientedConv1d as Conv

        table5 = {"protocol": "N=64 C=512 f32 bias=False, fwd+bwd through the module as "
                              "analysis/benchmark.py:19-67 times it, 10 warm-up + %d timed "
                              "iterations per angle, mean over 8 angles, ms" % args.table5_iters,
                  "published_rtx3090_ms": {"14": [0.3, 0.8], "28": [0.9, 2.6], "56": [3.2, 9.9]}}
        published_angles = [0, 22.5, 45, 66.75, 90, 112.5, 135, 157.5]
        torch.cuda.set_stream(torch.cuda.default_stream(dev))
        for HW_ in (14, 28, 56):
            xb = torch.randn(64, 512, HW_, HW_, device=dev)
            row = {}
            for K_ in (7, 31):
                for tag, angles in (("as_published", published_angles),
                                    ("canonical", [math.radians(a) for a in
                                                   (0, 22.5, 45, 67.5, 90, 112.5, 135, 157.5)])):
                    means = []
                    for ang in angles:
                        layer = Conv(512, 512, K_, angle=float(ang), padding=K_ // 2, stride=1,
                                     bias=False, groups=512).to(dev)
                        times = []
                        for it in range(10 + args.table5_iters):
                            torch.cuda.synchronize()
                            t0 = time.perf_counter()
                            (layer(xb).mean() * 1024).backward()
                            for p_ in layer.parameters():
                                p_.grad = None
                            torch.cuda.synchronize()
                            if it >= 10:
                                times.append((time.perf_counter() - t0) * 1e3)
                        means.append(sum(times) / len(times))
                    row["K%d_%s" % (K_, tag)] = round(sum(means) / len(means), 3)
            table5[str(HW_)] = row
            del xb
        torch.cuda.set_stream(stream)
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ CPU baseline (oracle)
    cpu, cpu_all = None, None
    if not args.no_cpu_baseline:
        from oracle import dwo_oracle as oracle

        rng = np.random.default_rng(0)
        n_cpu = BATCH  # the whole step once: every stage shape at batch 64, all three ops
        cpu_bytes, cpu_s = 0, 0.0
        for C, HW in STAGES:
            th = theta_for(C, args.theta)
            x = rng.standard_normal((n_cpu, C, HW, HW)).astype(np.float32)
            dy = rng.standard_normal((n_cpu, C, HW, HW)).astype(np.float32)
            w = (rng.standard_normal((C, 1, 1, KSIZE)) * 0.02).astype(np.float32)
            c0 = time.perf_counter()
            oracle.fprop(x, w, th, acc="f32")
            oracle.dgrad(dy, w, th, acc="f32")
            oracle.wgrad(dy, x, th, KSIZE, acc="f32")
            cpu_s += time.perf_counter() - c0
            cpu_bytes += sum(algorithmic_bytes(o, n_cpu, C, HW, HW, KSIZE, 4)
                             for o in ("fprop", "dgrad", "wgrad"))
        # the same loops with the channels spread over all host threads (the reference has no
        # threaded CPU path; reported for scale), on the largest stage only
        nthr = oracle.max_threads()
        C, HW = STAGES[0]
        th = theta_for(C, args.theta)
        x = rng.standard_normal((n_cpu, C, HW, HW)).astype(np.float32)
        w = (rng.standard_normal((C, 1, 1, KSIZE)) * 0.02).astype(np.float32)
        c0 = time.perf_counter()
        oracle.fprop(x, w, th, acc="f32", threads=nthr)
        oracle.dgrad(x, w, th, acc="f32", threads=nthr)
        oracle.wgrad(x, x, th, KSIZE, acc="f32", threads=nthr)
        mt_s = time.perf_counter() - c0
        mt_bytes = sum(algorithmic_bytes(o, n_cpu, C, HW, HW, KSIZE, 4)
                       for o in ("fprop", "dgrad", "wgrad"))
        cpu_all = {"value": round(mt_bytes / mt_s / 1e9, 3), "unit": "GB/s", "cores": nthr,
                   "sample": "fprop+dgrad+wgrad at C=96, 56x56, batch 64, channels over %d "
                             "threads (%.1f s)" % (nthr, mt_s)}
        cpu = {"value": round(cpu_bytes / cpu_s / 1e9, 4), "unit": "GB/s", "cores": 1,
               "kind": "port",
               "sample": "one whole step: fp32 fprop+dgrad+wgrad at each of the four stage shapes, "
                         "batch 64, single thread, reference loop order and fp32 accumulation "
                         "(%.1f s)" % cpu_s,
               "host_cpus": os.cpu_count()}

    # ------------------------------------------------------------------ ConvNeXt-T-1D images/s
    # Second half of the metric: inference forward of the harness (random-init weights, bf16,
    # batch 128 of 3x224x224 N(0,1) images, 1000 classes); its CPU counterpart (same harness on
    # the host, fp32, batch 8, oriented convs by the oracle) is reported beside it.
    model_info = None
    if args.model_iters > 0:
        main_res = None
        torch.cuda.empty_cache()
        from oriented1d_amd.convnext1d import convnext_tiny_1d
        from oriented1d_amd.dwoconv1d import DepthwiseOrientedConv1d

        torch.manual_seed(0)
        model = convnext_tiny_1d(variant="1d").to(dev).to(torch.bfloat16).eval()
        imgs = torch.randn(128, 3, 224, 224, device=dev).to(torch.bfloat16)
        with torch.no_grad():
            for _ in range(2):
                logits = model(imgs)
            torch.cuda.synchronize()
            if logits.shape != (128, 1000) or not bool(torch.isfinite(logits).all()):
                raise RuntimeError("ConvNeXt-T-1D forward: wrong shape or non-finite logits")
            w0 = time.perf_counter()  # the clocks of a continuous job before the timed forwards
            while (time.perf_counter() - w0) * 1e3 < args.precondition_ms:
                model(imgs)
                torch.cuda.synchronize()
            m0 = time.perf_counter()
            for _ in range(args.model_iters):
                model(imgs)
            torch.cuda.synchronize()
            m1 = time.perf_counter()
        gpu_ips = 128 * args.model_iters / (m1 - m0)
        model_info = {"model": "ConvNeXt-T-1D inference, random init, bf16, batch 128, 3x224x224; "
                               "oriented convs and the block/stem glue (LayerNorm, layout "
                               "changes, residual) by this library, pointwise layers by PyTorch",
                      "images_per_s": round(gpu_ips, 1),
                      "ms_per_batch": round((m1 - m0) * 1e3 / args.model_iters, 2)}
        if not args.no_cpu_baseline:
            from oracle import dwo_oracle as oracle

            cpu_model = convnext_tiny_1d(variant="1d").eval()
            nthreads = oracle.max_threads()

            def host_conv(mod):
                def fwd(t):
                    o = oracle.module_forward(
                        t.numpy(), mod.weight.detach().numpy(), mod.theta.detach().numpy(),
                        bias=mod.bias.detach().numpy(), stride=mod.stride[0], nhwc=mod.nhwc,
                        resid=mod.resid is not None, acc="f32")
                    return torch.from_numpy(o)
                return fwd

            # threads only affects the C loops' channel partition (bit-identical results)
            _fprop = oracle.fprop
            oracle.fprop = lambda *a, **k: _fprop(*a, **{**k, "threads": nthreads})
            for mod in cpu_model.modules():
                if isinstance(mod, DepthwiseOrientedConv1d):
                    mod.forward = host_conv(mod)
            cimgs = torch.randn(8, 3, 224, 224)
            with torch.no_grad():
                cpu_model(cimgs)
                c0 = time.perf_counter()
                for _ in range(3):
                    cpu_model(cimgs)
                c1 = time.perf_counter()
            oracle.fprop = _fprop
            model_info["cpu_images_per_s"] = round(8 * 3 / (c1 - c0), 2)
            model_info["cpu_config"] = ("same harness on the host: fp32, batch 8, 3 forwards, torch "
                                        "CPU ops with %d threads, oriented convs by the oracle's "
                                        "loops on %d threads" % (torch.get_num_threads(), nthreads))

    # ------------------------------------------------------------------ the two training configurations
    # ConvNeXt-B-1D++ training step (fwd + bwd + AdamW, bf16 autocast over fp32 masters, batch 64,
    # stochastic depth 0.5, random labels) and ConvNeXt-T-1D dense features at 8 x 3 x 512 x 512
    # (bf16, the four stage outputs, loss = sum <out_i, R_i>, fwd + bwd).  Reported, not part of
    # `value`.
    train_info = None
    if args.train_iters > 0:
        model = None
        torch.cuda.empty_cache()
        from oriented1d_amd.convnext1d import convnext_base_1d, convnext_tiny_1d
        train_info = {}
        try:
            torch.manual_seed(0)
            net = convnext_base_1d(variant="1dpp", drop_path_rate=0.5).to(dev).train()
            opt = torch.optim.AdamW(net.parameters(), lr=1e-3, weight_decay=0.05)
            imgs = torch.randn(64, 3, 224, 224, device=dev)
            labels = torch.randint(0, 1000, (64,), device=dev)

            def train_step():
                opt.zero_grad(set_to_none=True)
                with torch.autocast("cuda", dtype=torch.bfloat16):
                    loss = torch.nn.functional.cross_entropy(net(imgs).float(), labels)
                loss.backward()
                opt.step()
                return loss

            for _ in range(2):
                loss_ = train_step()
            torch.cuda.synchronize()
            if not math.isfinite(float(loss_.detach())) or not all(
                    bool(torch.isfinite(p_).all()) for p_ in net.parameters()):
                raise RuntimeError("ConvNeXt-B-1D++ training step: non-finite loss or parameters")
            t0 = time.perf_counter()
            for _ in range(args.train_iters):
                train_step()
            torch.cuda.synchronize()
            dt = (time.perf_counter() - t0) / args.train_iters
            train_info["convnext_b_1dpp_train"] = {
                "config": "fwd+bwd+AdamW, bf16 autocast, batch 64, 3x224x224, drop path 0.5",
                "ms_per_step": round(dt * 1e3, 2), "images_per_s": round(64 / dt, 1)}
            del net, opt, imgs, labels
            torch.cuda.empty_cache()

            net = convnext_tiny_1d(variant="1d", out_stages=True).to(dev).to(torch.bfloat16).train()
            imgs = torch.randn(8, 3, 512, 512, device=dev).to(torch.bfloat16)
            targets = []

            def feature_step():
                for p_ in net.parameters():
                    p_.grad = None
                outs = net(imgs)
                if not targets:
                    targets.extend(torch.randn_like(o) for o in outs)
                loss = sum((o.float() * r.float()).sum() for o, r in zip(outs, targets))
                loss.backward()
                return loss

            for _ in range(2):
                loss_ = feature_step()
            torch.cuda.synchronize()
            if not math.isfinite(float(loss_.detach())) or not all(
                    p_.grad is None or bool(torch.isfinite(p_.grad).all()) for p_ in net.parameters()):
                raise RuntimeError("ConvNeXt-T-1D features step: non-finite loss or gradients")
            t0 = time.perf_counter()
            for _ in range(args.train_iters):
                feature_step()
            torch.cuda.synchronize()
            dt = (time.perf_counter() - t0) / args.train_iters
            train_info["convnext_t_1d_features"] = {
                "config": "fwd+bwd, bf16, 8x3x512x512, four stage outputs, loss = sum <out_i, R_i>",
                "ms_per_step": round(dt * 1e3, 2), "images_per_s": round(8 / dt, 1)}
            del net, imgs, targets
        except RuntimeError as exc:  # e.g. out of memory next to another process: keep the main line
            train_info["error"] = str(exc).splitlines()[0][:200]
        torch.cuda.empty_cache()

    out = {
        "metric": "dwoconv1d fprop/dgrad/wgrad GB/s (% HBM peak); ConvNeXt-T-1D img/s",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "dwoconv1d fprop+dgrad+wgrad sweep at ConvNeXt-T stage shapes "
                               "(C=96@56x56, 192@28x28, 384@14x14, 768@7x7), batch 64, K=31, "
                               "8 orientations %s, stride 1" % args.theta,
                   "layout": args.layout, "buffer_sets_per_stage": nsets_per_stage,
                   "timing": "sustained state: %d untimed steps (%.0f ms) run before the warm-up "
                             "steps; the same warm-up + timed steps right after an idle spell are "
                             "ms_per_step_first_window; per-kernel: >= %.0f ms of launches, then "
                             "the median of %d x %d launches"
                             % (n_pre, args.precondition_ms, args.kernel_warm_ms,
                                args.kernel_repeats, args.kernel_iters),
                   "ms_per_step_first_window": round(ms_first, 4) if ms_first else None,
                   "launch": "eager C-ABI calls on one stream (value, ms_per_step); the hipGraph "
                             "replays of the same step are listed for information",
                   "ms_per_step_graph": round(main_res_graph, 4) if main_res_graph else None,
                   "ms_per_step_eager": round(main_res_eager, 4),
                   "ms_per_step_parallel_branches": (round(main_res_branches, 4)
                                                     if main_res_branches else None),
                   "algorithmic_bytes_per_step": step_bytes},
        "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "detail": detail, "roofline": roofline, "roofline_min": roofline_min, "cpu_baseline": cpu,
        "table5": table5,
        "cpu_baseline_all_threads": cpu_all, "other_configs": others, "other_shapes_bf16": other_shapes,
        "convnext_t_1d": model_info, "training_configs": train_info,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
