#!/usr/bin/env python3
"""Benchmark of the int8 ConvBias hot path on one MI355X.

A "step" is one pass over the 53 ConvBias layers of the ResNet-50 int8 conv stack at batch 64
(workload "config 2" of megengine_amd/workloads.py) on synthetic, HBM-resident tensors; activations are requantised between
layers and the residual z tensors are the real producer outputs.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

value      = images per second over the timed region (K steps, events on the launch stream)
roofline   = algorithmic bytes per launch / average launch duration over the timed region (HIP events
             on the launch stream around K x 53 back-to-back launches), against 8 TB/s HBM; a second
             pass with an event after every launch gives the per-layer table
cpu_baseline = the CPU parity checker (a port of the reference's naive ConvBias) timed on this
             host on a bounded sample (one image through the same 53 layers), scaled to images/s
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_PEAK_OPS = 5.0e15   # dense INT8 MFMA, MI355X
HBM_PEAK = 8.0e12        # bytes/s


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-extras", action="store_true", help="skip the per-config side measurements")
    ap.add_argument("--extras-only", action="store_true",
                    help="side measurements only (short runs for profilers): prints their JSON, no headline")
    ap.add_argument("--side-iters", type=int, default=50, help="launches per side measurement")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only")
    ap.add_argument("--no-preprocess", action="store_true", help="exec with the filters in the reference layout only")
    ap.add_argument("--tiles", default="", metavar="LAYER=TILE,...",
                    help="run the named layers of the stack on the named tiles instead of the heuristic's (measurements; "
                         "the output line says so)")
    ap.add_argument("--no-memory-plan", action="store_true",
                    help="one buffer per layer output instead of the static activation-memory plan")
    ap.add_argument("--no-residual-in-place", action="store_true",
                    help="memory plan without letting a layer write its output over a residual it reads last")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also launch one plain 256 MiB streaming kernel (counter calibration for profilers)")
    ap.add_argument("--layers-out", default=None, help="write the per-layer table to this JSON file")
    ap.add_argument("--sweep-layers", default=None,
                    help="comma-separated ResNet-50 layer names for --batch-sweep, or 'all' (default: ten representative ones)")
    ap.add_argument("--batch-sweep", action="store_true",
                    help="time ten representative ResNet-50 layers alone at batch 4..128 with their batch-64 tile, print the "
                         "table (JSON on stdout, text on stderr) and exit: where a layer's time goes")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU (the path shards by batch with no exchange); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from megengine_amd import _abi, lib, ops, workloads

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    L = lib.lib()  # raises if the HIP extension is missing
    info = lib.device_info(0)
    log("device: %s %s, %d CUs, %.0f MHz" % (info.name.decode(), info.arch.decode(), info.compute_units,
                                             info.clock_khz / 1e3))
    torch.manual_seed(1234)
    if args.batch_sweep:
        side = torch.cuda.Stream()
        torch.cuda.set_stream(side)
        print(json.dumps(dict(batch_sweep=run_batch_sweep(torch, _abi, lib, ops, workloads, args.sweep_layers))), flush=True)
        return
    if args.extras_only:
        side = torch.cuda.Stream()
        torch.cuda.set_stream(side)
        print(json.dumps(dict(other_configs=run_extras(torch, np, _abi, lib, ops, workloads, args.side_iters))), flush=True)
        if args.calib_copy:
            calib_copy(torch)
        return
    batch = 64
    layers = workloads.resnet50(batch)
    plan = workloads.build_stack(layers, 7)
    # activation memory laid out once by liveness, as the graph runtime above the operator does before it runs a
    # computing sequence (--no-memory-plan: one buffer per layer output); a block's last layer writes its output over
    # the residual it adds, which nothing reads after it
    mem = None if args.no_memory_plan else workloads.plan_memory(plan, residual_in_place=not args.no_residual_in_place)
    # algorithm choice and weight pre-processing happen once, before the timed region (exec_preprocess is the
    # reference's own hook for hoisting filter re-tiling out of exec)
    forced = dict(item.split("=") for item in args.tiles.split(",") if item)
    workloads.choose_algorithms(plan, weight_preprocess=not args.no_preprocess, tiles=forced)
    side = torch.cuda.Stream()          # default priority; every launch of the bench goes here
    torch.cuda.set_stream(side)
    stream = torch.cuda.current_stream()
    raw_stream = stream.cuda_stream
    calls = workloads.bind_plan(plan)

    def step():
        for c in calls:
            c()

    for _ in range(max(1, args.warmup)):
        step()
    torch.cuda.synchronize()
    want = [p["dst"].clone() for p in plan]

    # ---- timed region, eager launches through the C ABI
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(args.steps):
        step()
    e1.record(stream)
    torch.cuda.synchronize()
    eager_ms = e0.elapsed_time(e1) / args.steps

    # ---- the same K steps as replays of one captured HIP graph of the 53 launches (kernel nodes only)
    graph_ms, graph_note = None, "not attempted"
    if not args.no_graph:
        try:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                step()
            ok = True
            for rep in range(3):            # replays separated by eager work and synchronisation
                for p in plan:
                    p["dst"].fill_(rep)
                torch.cuda.synchronize()
                g.replay()
                torch.cuda.synchronize()
                ok = ok and all(torch.equal(p["dst"], w) for p, w in zip(plan, want))
            if ok:
                for _ in range(args.warmup):
                    g.replay()
                torch.cuda.synchronize()
                e0.record(stream)
                for _ in range(args.steps):
                    g.replay()
                e1.record(stream)
                torch.cuda.synchronize()
                graph_ms = e0.elapsed_time(e1) / args.steps
                graph_note = "replays bit-identical to eager launches (3 checked)"
            else:
                graph_note = "replay differed from eager launches; not used"
        except Exception as e:  # capture is an optimisation of the launch path only
            graph_note = "capture failed: %r" % (e,)
    log("eager %.4f ms/step, graph %s ms/step (%s)" % (eager_ms, graph_ms, graph_note))
    ms_per_step = graph_ms if graph_ms is not None else eager_ms
    launch_mode = "hipGraph replay" if graph_ms is not None else "eager"

    # ---- the same stack with one buffer per layer output (what the memory plan is worth), fewer replays
    unplanned_ms = None
    if mem is not None and graph_ms is not None:
        try:
            plan2 = workloads.choose_algorithms(workloads.build_stack(layers, 7), weight_preprocess=not args.no_preprocess,
                                                tiles=forced)
            calls2 = workloads.bind_plan(plan2)
            for c in calls2:
                c()
            torch.cuda.synchronize()
            g2 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g2, stream=side):
                for c in calls2:
                    c()
            reps2 = max(20, args.steps // 4)
            for _ in range(3):
                g2.replay()
            torch.cuda.synchronize()
            e0.record(stream)
            for _ in range(reps2):
                g2.replay()
            e1.record(stream)
            torch.cuda.synchronize()
            unplanned_ms = e0.elapsed_time(e1) / reps2
            del g2, calls2, plan2
        except Exception as e:  # a comparison figure must not lose the headline
            log("one-buffer-per-layer stack: %r" % (e,))
    img_s = batch * 1000.0 / ms_per_step
    tot_ops = sum(l.ops for l in layers)
    tot_bytes = sum(l.bytes for l in layers)

    # ---- second pass over the same K steps: a HIP event after every launch, on the launch stream
    nl = len(plan)
    timer = EventTimer(torch, raw_stream, args.steps * (nl + 1))
    torch.cuda.synchronize()
    for s in range(args.steps):
        timer.record()
        for c in calls:
            c()
            timer.record()
    torch.cuda.synchronize()
    per_layer_ms = [sum(timer.elapsed(s * (nl + 1) + i, s * (nl + 1) + i + 1) for s in range(args.steps)) / args.steps
                    for i in range(nl)]
    assert all(torch.equal(p["dst"], w) for p, w in zip(plan, want)), "outputs changed between passes"
    kern_ms = sum(per_layer_ms)
    table = []
    for p, ms in zip(plan, per_layer_ms):
        l = p["layer"]
        t = ms * 1e-3
        roof = max(l.ops / INT8_PEAK_OPS, l.bytes / HBM_PEAK)
        table.append(dict(name=l.name, ic=l.ic, oc=l.oc, hw=l.ih, f=l.f, s=l.stride, z=l.z is not None,
                          algo=lib.algo_names()[p["algo"].id], tile=lib.tile_names()[p["algo"].tile_cfg],
                          us=round(ms * 1e3, 2), tops=round(l.ops / t / 1e12, 1), gbs=round(l.bytes / t / 1e9, 1),
                          frac_roof=round(roof / t, 3)))
    # dominant kernels = the MFMA ConvBias kernels (all 53 launches).  Average launch duration = the
    # timed region of K steps (two HIP events on the launch stream) / (K * 53): the launches run
    # back to back, so this is the kernel duration plus the sub-microsecond gap between launches.
    t_launch = ms_per_step * 1e-3 / nl
    roofline = dict(bound="hbm", achieved=round(tot_bytes / nl / t_launch / 1e9, 1), peak=HBM_PEAK / 1e9,
                    unit="GB/s", frac=round(tot_bytes / nl / t_launch / HBM_PEAK, 4), traffic=None,
                    kernel="ConvBias MFMA kernels (igemm2_kernel, igemm3_kernel, igemm_dma_kernel, pw32s_kernel, c4_kernel), 53 launches per step",
                    bytes_per_launch=round(tot_bytes / nl), avg_launch_us=round(t_launch * 1e6, 2),
                    per_launch_event_sum_ms=round(kern_ms, 4),
                    mfma_tops=round(tot_ops / (ms_per_step * 1e-3) / 1e12, 1),
                    mfma_frac_of_int8_peak=round(tot_ops / (ms_per_step * 1e-3) / INT8_PEAK_OPS, 4),
                    frac_of_binding_roof=round(sum(max(l.ops / INT8_PEAK_OPS, l.bytes / HBM_PEAK) for l in layers)
                                               / (ms_per_step * 1e-3), 4))
    tr = os.path.join(ROOT, "profiles", "traffic_resnet50_stack.json")
    if os.path.exists(tr):
        try:
            trj = json.load(open(tr))
            roofline["traffic"] = trj["hbm_bytes_per_launch"]
            # not measured by this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE passes over this same command
            roofline["traffic_source"] = "profiles/traffic_resnet50_stack.json (%s)" % trj.get("measured", "earlier counter pass")
        except Exception:
            pass

    # ---- what the launches and the memory traffic alone cost here: the same 53 dependent launches as plain streaming
    # kernels that read and write each layer's bytes (mi355_stream_probe), replayed from a captured graph like the stack
    if not args.no_graph:
        try:
            chain_ms = streaming_chain_ms(torch, L, layers, side, stream, max(20, args.steps // 4))
            roofline["streaming_chain_ms"] = round(chain_ms, 4)
            roofline["vs_streaming_chain"] = round(ms_per_step / chain_ms, 3)
        except Exception as e:  # a measuring stick must not lose the headline
            roofline["streaming_chain_ms"] = None
            log("streaming chain: %r" % (e,))

    out = dict(metric="ResNet-50 int8 conv-stack throughput @ bs64 (53 ConvBias layers)", value=round(img_s, 1),
               unit="img/s", n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=round(ms_per_step, 4),
               higher_is_better=True, scaling="weak", vs_baseline=None, dtype="s8",
               data="synthetic",
               config=dict(arithmetic="s8 x s8 products accumulated in s32 (exact), requantised to s8 through f32 as the reference does",
                           workload="BASELINE configs[2]: ResNet-50 v1.5 int8 conv stack, batch 64, 224x224, "
                                    "NCHW4 stem + NCHW32, fused residual z + RELU, random per-tensor scales",
                           batch=batch, layers=nl, launch=launch_mode, graph=graph_note,
                           **(dict(forced_tiles=forced) if forced else {}),
                           activation_memory=("one buffer per layer output, %.0f MB" % (sum(p["dst"].numel() for p in plan) / 1e6)
                                              if mem is None else
                                              "static plan by liveness: %.0f MB for the %.0f MB of layer outputs%s"
                                              % (mem["planned"] / 1e6, mem["one_buffer_per_layer"] / 1e6,
                                                 "" if args.no_residual_in_place else
                                                 ", outputs written over residuals read for the last time")),
                           weight_preprocess="%d of %d filters pre-processed once through exec_preprocess, outside the timed "
                                             "region" % (sum(p.get("pre") is not None for p in plan), nl)),
               eager_ms_per_step=round(eager_ms, 4),
               ms_per_step_one_buffer_per_layer=None if unplanned_ms is None else round(unplanned_ms, 4),
               tops=round(tot_ops / (ms_per_step * 1e-3) / 1e12, 1),
               pct_int8_peak=round(100 * tot_ops / (ms_per_step * 1e-3) / INT8_PEAK_OPS, 2),
               roofline=roofline)

    if args.calib_copy:
        calib_copy(torch)

    extras = {}
    if not args.no_extras:
        try:
            extras = run_extras(torch, np, _abi, lib, ops, workloads, args.side_iters)
        except Exception as e:  # side measurements must not lose the headline
            extras = dict(error=repr(e))
        out["other_configs"] = extras

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(np, plan, workloads.snapshot_run(plan, calls, min(batch, 16)))

    if args.layers_out:
        with open(args.layers_out, "w") as f:
            json.dump(dict(layers=table, extras=extras), f, indent=1)
    else:
        for row in table:
            log(row)
    print(json.dumps(out), flush=True)


def calib_copy(torch):
    """One plain streaming kernel of known size (reads 256 MiB, writes 256 MiB): the reference point that scales the
    profiler's FETCH_SIZE / WRITE_SIZE counters."""
    a = torch.randint(0, 255, (256 << 20,), dtype=torch.uint8, device="cuda")
    b = torch.empty_like(a)
    torch.cuda.synchronize()
    torch.bitwise_not(a, out=b)
    torch.cuda.synchronize()
    del a, b


class EventTimer:
    """HIP events recorded straight on a raw stream (cheaper than torch's wrappers, so the host
    stays ahead of the GPU and an interval between two events is the kernel between them)."""

    def __init__(self, torch, raw_stream, n):
        import ctypes as C
        self.C = C
        self.torch = torch
        self.stream = C.c_void_p(raw_stream)
        self.n = 0
        try:
            self.hip = C.CDLL("libamdhip64.so")
            self.ev = (C.c_void_p * n)()
            for i in range(n):
                if self.hip.hipEventCreate(C.byref(self.ev, i * C.sizeof(C.c_void_p))):
                    raise OSError("hipEventCreate failed")
        except OSError:
            self.hip = None
            self.ev = [torch.cuda.Event(enable_timing=True) for _ in range(n)]

    def record(self):
        if self.hip is not None:
            if self.hip.hipEventRecord(self.C.c_void_p(self.ev[self.n]), self.stream):
                raise RuntimeError("hipEventRecord failed")
        else:
            self.ev[self.n].record(self.torch.cuda.current_stream())
        self.n += 1

    def elapsed(self, i, j):
        if self.hip is None:
            return self.ev[i].elapsed_time(self.ev[j])
        ms = self.C.c_float()
        if self.hip.hipEventElapsedTime(self.C.byref(ms), self.C.c_void_p(self.ev[i]), self.C.c_void_p(self.ev[j])):
            raise RuntimeError("hipEventElapsedTime failed")
        return ms.value


def time_launches(torch, fn, iters=20, warm=3, graph=True):
    """Seconds per call of fn (one or more launches on the current stream), `iters` calls back to back.  With `graph`
    the calls are captured once into a HIP graph and the graph is replayed: eager launches through Python cost ~6 us
    of host time each, which would be the figure reported for every kernel shorter than that (the depthwise layers at
    14x14 and 7x7 run 3.6-5.5 us).  Falls back to eager launches if the capture fails."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    st = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    if graph:
        try:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=st):
                for _ in range(iters):
                    fn()
            g.replay()
            torch.cuda.synchronize()
            reps = 3
            e0.record(st)
            for _ in range(reps):
                g.replay()
            e1.record(st)
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / (iters * reps) * 1e-3
        except Exception as e:  # capture is an optimisation of the launch path only
            log("graph capture of a side measurement failed (%r): eager launches" % (e,))
            torch.cuda.synchronize()
    e0.record(st)
    for _ in range(iters):
        fn()
    e1.record(st)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters * 1e-3


def streaming_chain_ms(torch, L, layers, side, stream, reps):
    """One pass over the layer list as plain streaming launches: layer i reads src + filter + bias (+ residual) bytes and
    writes dst bytes, ping-ponging between two buffers; captured once, replayed `reps` times."""
    rd = [((l.bytes - l.n * l.oc * l.oh * l.ow) + 15) // 16 * 16 for l in layers]
    wr = [(l.n * l.oc * l.oh * l.ow + 15) // 16 * 16 for l in layers]
    cap = max(max(rd), max(wr))
    a = torch.ones(cap, dtype=torch.uint8, device="cuda")
    b = torch.ones(cap, dtype=torch.uint8, device="cuda")
    raw = stream.cuda_stream

    def chain():
        for i in range(len(layers)):
            s, d = (a, b) if i % 2 == 0 else (b, a)
            st = L.mi355_stream_probe(raw, s.data_ptr(), rd[i], d.data_ptr(), wr[i])
            if st:
                raise RuntimeError("mi355_stream_probe: status %d" % st)

    chain()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        chain()
    for _ in range(3):
        g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(reps):
        g.replay()
    e1.record(stream)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


_FLUSH = None


def time_launches_cold(torch, fn, iters=8):
    """Like time_launches, but L2 and the 256 MB last-level cache are flushed before every launch (a 512 MiB fill on
    the same stream); only the launch itself is between the two events of an iteration."""
    global _FLUSH
    if _FLUSH is None:
        _FLUSH = torch.empty(512 << 20, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream()
    fn()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for e0, e1 in ev:
        _FLUSH.fill_(1)
        e0.record(st)
        fn()
        e1.record(st)
    torch.cuda.synchronize()
    t = sorted(e0.elapsed_time(e1) for e0, e1 in ev)
    return t[len(t) // 2] * 1e-3


def run_extras(torch, np, _abi, lib, ops, workloads, side_iters=50):
    """Side measurements for the other workload configurations (not the headline value).  Every row carries two
    times: "us" = the launch repeated back to back on the same tensors as replays of a captured HIP graph (operands warm
    in L2 / the last-level cache when they fit; the dependent-launch gap of ~1.8 us is part of it, the host's launch
    cost is not), "us_cold" = median of eager launches that each follow a flush of both caches."""
    res = {}

    def measure(layers, seed):
        plan = workloads.build_stack(layers, seed)
        rows = []
        workloads.choose_algorithms(plan)
        # pre-marshalled launches: the per-call Python work of conv_bias_exec would floor short kernels
        calls = workloads.bind_plan(plan)
        for p, call in zip(plan, calls):
            t = time_launches(torch, call, iters=side_iters)
            tc = time_launches_cold(torch, call, iters=max(3, min(8, side_iters)))
            l = p["layer"]
            roof = max(l.ops / INT8_PEAK_OPS, l.bytes / HBM_PEAK)
            rows.append(dict(name=l.name, algo=lib.algo_names()[p["algo"].id], us=round(t * 1e6, 2),
                             us_cold=round(tc * 1e6, 2), tops=round(l.ops / t / 1e12, 1), gbs=round(l.bytes / t / 1e9, 1),
                             frac_roof=round(roof / t, 3), frac_roof_cold=round(roof / tc, 3)))
        return rows, plan, calls

    rows, _, _ = measure([workloads.config0()], 1)
    res["config0"] = rows[0]
    rows, _, _ = measure(workloads.pointwise_sweep(), 2)
    res["config1_pointwise"] = rows
    torch.cuda.empty_cache()
    mb = workloads.mobilenet_v2()
    rows, _, _ = measure(mb, 3)
    dw = [(r, l) for r, l in zip(rows, mb) if l.group > 1]
    pw = [(r, l) for r, l in zip(rows, mb) if l.group == 1]
    t_dw = sum(r["us"] for r, _ in dw) * 1e-6
    t_pw = sum(r["us"] for r, _ in pw) * 1e-6
    tc_dw = sum(r["us_cold"] for r, _ in dw) * 1e-6
    tc_pw = sum(r["us_cold"] for r, _ in pw) * 1e-6
    res["config3_mobilenetv2"] = dict(
        depthwise=dict(us=round(t_dw * 1e6, 1), gbs=round(sum(l.bytes for _, l in dw) / t_dw / 1e9, 1),
                       frac_hbm=round(sum(l.bytes for _, l in dw) / t_dw / HBM_PEAK, 3), us_cold=round(tc_dw * 1e6, 1),
                       frac_hbm_cold=round(sum(l.bytes for _, l in dw) / tc_dw / HBM_PEAK, 3),
                       layers=[r for r, _ in dw]),
        pointwise=dict(us=round(t_pw * 1e6, 1), gbs=round(sum(l.bytes for _, l in pw) / t_pw / 1e9, 1),
                       tops=round(sum(l.ops for _, l in pw) / t_pw / 1e12, 1),
                       frac_hbm=round(sum(l.bytes for _, l in pw) / t_pw / HBM_PEAK, 3), us_cold=round(tc_pw * 1e6, 1),
                       frac_hbm_cold=round(sum(l.bytes for _, l in pw) / tc_pw / HBM_PEAK, 3)))
    torch.cuda.empty_cache()
    c4 = []
    for l in workloads.large_hswish():
        rows, plan, calls = measure([l], 4)
        p, conv = plan[0], calls[0]
        # NCHW -> NCHW32 relayout of the input and NCHW32 -> NCHW of the output, timed with the conv
        x_nchw = torch.randint(-128, 128, (l.n, l.ic, l.ih, l.iw), dtype=torch.int8, device="cuda")
        y_nchw = torch.empty((l.n, l.oc, l.oh, l.ow), dtype=torch.int8, device="cuda")
        d_in = ops.relayout_desc(_abi.RL_NCHW_NCHW32, tuple(x_nchw.shape))
        d_out = ops.relayout_desc(_abi.RL_NCHW32_NCHW, tuple(p["dst"].shape))

        def full():
            ops.relayout_exec(d_in, x_nchw, p["src"])
            conv()  # the heuristic's algorithm, with its pre-processed filter where it has one
            ops.relayout_exec(d_out, p["dst"], y_nchw)

        n10 = max(2, min(10, side_iters))
        t_full = time_launches(torch, full, iters=n10)
        t_in = time_launches(torch, lambda: ops.relayout_exec(d_in, x_nchw, p["src"]), iters=n10)
        t_out = time_launches(torch, lambda: ops.relayout_exec(d_out, p["dst"], y_nchw), iters=n10)
        rl_bytes_in, rl_bytes_out = 2 * x_nchw.numel(), 2 * y_nchw.numel()
        # the same launch (same instruction stream, same addresses) with every operand byte zero: what the kernel's
        # schedule reaches when the matrix units switch no bits.  The difference from "us" is the part of the time that
        # the power limit of the device, not the schedule, decides.
        for t_ in (p["src"], p["flt"], p["bias"], p["z"], p.get("pre")):
            if t_ is not None:
                t_.zero_()
        conv()
        torch.cuda.synchronize()
        t_zero = min(time_launches(torch, conv, iters=n10), time_launches(torch, conv, iters=n10))
        rows[0]["us_zero_operands"] = round(t_zero * 1e6, 2)
        rows[0]["tops_zero_operands"] = round(l.ops / t_zero / 1e12, 1)
        # (these tensors are 67-134 MB each and stream through both caches: every launch is a cold one)
        c4.append(dict(conv=rows[0], total_us=round(t_full * 1e6, 1),
                       relayout_in_gbs=round(rl_bytes_in / t_in / 1e9, 1),
                       relayout_out_gbs=round(rl_bytes_out / t_out / 1e9, 1),
                       relayout_frac_hbm=round((rl_bytes_in + rl_bytes_out) / (t_in + t_out) / HBM_PEAK, 3)))
        del x_nchw, y_nchw, plan
        torch.cuda.empty_cache()
    res["config4_large_hswish"] = c4
    return res


def run_batch_sweep(torch, _abi, lib, ops, workloads, layers=None):
    """One layer at a time, repeated as replays of a captured graph (operands warm), at batch 4 .. 128 with the tile the
    stack uses at batch 64 forced at every size: the intercept is what a launch of that shape costs before any tile
    count matters, the slope what a tile costs once the device is full."""
    names = lib.tile_names()
    igemm = lib.algo_names().index("MI355_IGEMM_MFMA_I8")
    want = ["s1b0c1", "s1b0c2", "s1b0c3", "s2b1c2", "s3b1c1", "s3b1c2", "s3b1c3", "s4b1c1", "s4b1c2", "s4b1c3", "stem"]
    ref = {l.name: l for l in workloads.resnet50(64)}
    if layers == "all":
        want = list(ref)
    elif layers:
        want = layers.split(",")
    rows = []
    for name in want:
        l0 = ref[name]
        plan0 = workloads.build_stack([l0], 4)
        workloads.choose_algorithms(plan0)
        a0 = plan0[0]["algo"]
        del plan0
        row = dict(layer=name, algo=lib.algo_names()[a0.id], tile=names[a0.tile_cfg] if a0.id == igemm else None, us={})
        for n in (4, 8, 16, 32, 64, 128):
            l = workloads.Layer(l0.name, l0.fmt, n, l0.ic, l0.ih, l0.iw, l0.oc, l0.f, stride=l0.stride, pad=l0.pad,
                                group=l0.group, nonline=l0.nonline, z=("input:z" if l0.z else None))
            plan = workloads.build_stack([l], 4)
            p = plan[0]
            a, _ = ops.conv_bias_query(p["desc"], _abi.ALGO_HEURISTIC_PREPROCESS)
            if a0.id == igemm and lib.tile_usable(p["desc"], a0.tile_cfg):
                a.tile_cfg = a0.tile_cfg
            pre = ops.conv_bias_preprocess(p["desc"], p["flt"], a) if a.id == igemm else None
            call = ops.conv_bias_bind(p["desc"], p["src"], p["flt"], p["bias"], p["z"], p["dst"], a, preprocessed=pre)
            call()
            torch.cuda.synchronize()
            row["us"][str(n)] = round(min(time_launches(torch, call, iters=30) for _ in range(2)) * 1e6, 2)
            del plan, p
        log("%-7s %-28s " % (name, row["tile"] or row["algo"]) + " ".join("n%-3d %6.2f" % (int(k), v) for k, v in row["us"].items()))
        rows.append(row)
    return rows


def cpu_baseline(np, plan, snaps):
    """The CPU parity checker (a port of the reference's naive ConvBias, OpenMP over output rows) on a bounded sample
    of the SAME workload: the first b images of the very tensors the GPU plan ran on (same weights, biases, residuals
    and scales, layer by layer), b chosen so that the whole leg is 10-30 s of CPU work on this host; scaled to images
    per second.  Its outputs are compared with the first b images of the GPU's outputs.  snaps = per layer the host
    copies (source, residual, output) of the first images, taken right after the layer's launch."""
    import copy

    from oracle import oracle
    oracle.lib()
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    os.environ["OMP_NUM_THREADS"] = str(cores)
    total_macs = sum(p["layer"].ops // 2 for p in plan) / plan[0]["layer"].n  # per image

    def run(batch, budget):
        t_tot, macs, done, bad = 0.0, 0, 0, 0
        for p, (h_src, h_z, h_dst) in zip(plan, snaps):
            d = copy.copy(p["desc"])
            d.n = batch
            host = [None if t is None else np.ascontiguousarray(t[:batch]) for t in (h_src, h_z)]
            flt, bias = p["flt"].cpu().numpy(), p["bias"].cpu().numpy()
            t0 = time.perf_counter()
            out = oracle.conv_bias(d, host[0], flt, bias, host[1])
            t_tot += time.perf_counter() - t0
            bad += int((out != h_dst[:batch]).sum())
            macs += p["layer"].ops // 2 // p["layer"].n * batch
            done += 1
            if t_tot > budget:
                break
        return t_tot, macs, done, bad

    t1, m1, _, _ = run(1, 10.0)                 # probe: one image
    est = t1 * total_macs / max(m1, 1)
    batch = int(max(1, min(len(snaps[0][0]), round(15.0 / max(est, 1e-3)))))
    t_tot, macs, done, bad = run(batch, 30.0)
    img_s = (macs / total_macs) / t_tot if t_tot > 0 else 0.0
    return dict(value=round(img_s, 3), unit="img/s", cores=cores, kind="port",
                sample="the first %d images of the GPU plan's own tensors and scales through the first %d of %d layers "
                       "(%.1f GMAC of %.1f per image x %d) in %.1f s on %d threads, scaled by MACs" % (
                           batch, done, len(plan), macs / 1e9, total_macs / 1e9, batch, t_tot, cores),
                outputs_differing_from_gpu=bad)


if __name__ == "__main__":
    main()
