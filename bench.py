#!/usr/bin/env python3
"""bench.py — throughput of the deepxIR op hot path on one MI355X.

A "step" is one pass of BASELINE config 2 (the reductions workload) through libdxhip's C ABI
on synthetic tensors already resident in HBM:
    X fp32 [8192,8192] N(0,1):  sum axis 1, sum axis 0, reducemax axis 1, reducemin axis 1
    P fp32 [8192,64]  U(.9,1.1): prod axis 1
each with keepdims true and false (keepdims only changes the caller's view of the output, so
both launches run the same kernel) = 10 ops, 2,152,005,632 algorithmic bytes per step
(inputs read once + outputs written once per op).  X exists in three copies that the ops
rotate through, so no launch finds its input in the 256 MiB Infinity Cache.

Prints ONE JSON line: value = algorithmic GB/s over the timed region (all ops), `roofline`
for the dominant kernel (reduce_row_kernel, the contiguous-axis reduction: 6 of the 10 ops)
from HIP events recorded on the launch stream inside the timed region, `cpu_baseline` from
the oracle's restatement of op-ompsimd's per-element reduce on the host cores, and `per_op`
with every other BASELINE op measured the same way (events around each launch).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
MFMA_F32_PEAK_TF = 157.3
MFMA_F64_PEAK_TF = 78.6
MFMA_BF16_PEAK_TF = 2500.0  # dense bf16
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")  # HBM bytes per launch from the counter runs


def measured_traffic(kernel):
    """(bytes, provenance) — HBM-side bytes per launch of `kernel` as the last counter collection found them
    (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by a copy kernel of known size; the summary beside the file
    says how).  The file records a hash of the kernel sources the counters were collected on: when those files
    have changed since, or the file has no entry, bytes is None (the figure would describe another kernel) and
    the provenance says so."""
    import hashlib
    try:
        with open(TRAFFIC_JSON) as f:
            doc = json.load(f)
        e = doc["kernels"][kernel]
        h = hashlib.sha256()
        for name in e["sources"]:
            with open(os.path.join(ROOT, "deepx_amd", "csrc", name), "rb") as src:
                h.update(src.read())
        now = h.hexdigest()[:16]
        prov = {"file": "profiles/traffic.json", "collected": doc.get("collected"), "counter_row": e.get("counter_row"),
                "sources_sha16": e["sources_sha16"], "sources_unchanged": now == e["sources_sha16"]}
        return (e["hbm_bytes_per_launch"] if now == e["sources_sha16"] else None), prov
    except (OSError, KeyError, ValueError) as err:
        return None, {"file": "profiles/traffic.json", "error": type(err).__name__}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--ramp-ms", type=float, default=100.0,
                    help="untimed steps run for this long before the warmup steps: from idle the GPU takes "
                         "about 30 ms of load to reach its steady clocks")
    ap.add_argument("--no-per-op", action="store_true", help="skip the per-op table of the other configs")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--in-order-only", action="store_true",
                    help="skip the information passes in which launches overlap on several streams (under a kernel trace they would "
                         "mix overlapped launches into the per-kernel averages of the in-order step)")
    ap.add_argument("--matmul-only", metavar="MxKxN", default="",
                    help="run only the bf16 matmul of that shape, --steps launches after a clock ramp "
                         "(the program a counter collection wraps) and print its own JSON line")
    ap.add_argument("--matmul-tile", type=int, default=0, help="with --matmul-only: force a workgroup tile (DXH_TUNE_MATMUL_TILE), 0 = chosen per shape")
    ap.add_argument("--chain-only", metavar="RUN", default="",
                    help="run only one fused run (a label of per_op.config5.fused_runs, or a prefix of one), --steps launches after a "
                         "clock ramp (the program a counter collection wraps) and print its own JSON line")
    ap.add_argument("--chain-static", type=int, default=1, help="with --chain-only: 1 = the library's compiled kernel, 0 = the interpreting kernel")
    ap.add_argument("--block-only", metavar="MODE", default="",
                    help="run only the config-5 block over deepxIR in one mode (a key of per_op.config5.mlp_block_over_deepxIR, e.g. "
                         "one_batch_fused_us), --steps passes (the program a kernel trace wraps) and print its own JSON line")
    ap.add_argument("--attention-only", metavar="MODE", default="",
                    help="the same for the attention core over deepxIR (a key of per_op.attention_core_over_deepxIR)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this executor path runs on ONE GPU (no sharding, no collectives); "
              "--gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from deepx_amd import lib as dx

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    L = dx.load()
    torch.cuda.init()
    dev = torch.device("cuda:0")
    name = C.create_string_buffer(256)
    L.dxh_device_name(name, 256)

    class Events:
        """pairs of hipEvents recorded on the NULL stream, the stream every op is launched on"""

        def __init__(self):
            self.pairs = []

        def pair(self):
            a, b = C.c_void_p(), C.c_void_p()
            dx.check(L.dxh_event_create(C.byref(a)))
            dx.check(L.dxh_event_create(C.byref(b)))
            self.pairs.append((a, b))
            return a, b

        @staticmethod
        def ms(a, b):
            out = C.c_float()
            dx.check(L.dxh_event_elapsed_ms(a, b, C.byref(out)))
            return out.value

    def ptr(t):
        return C.c_void_p(t.data_ptr())

    if args.matmul_only:
        mm, kk, nn = (int(x) for x in args.matmul_only.lower().split("x"))
        Am = torch.randn(mm * kk, device=dev).to(torch.bfloat16)
        Bm = (torch.randn(kk * nn, device=dev) * 0.02).to(torch.bfloat16)
        Cm = torch.empty(mm * nn, device=dev, dtype=torch.bfloat16)
        dx.check(L.dxh_tune(4, args.matmul_tile), "DXH_TUNE_MATMUL_TILE")
        launch = matmul_call(L, dx, torch, dev, dx.BF16, Am, Bm, Cm, mm, kk, nn)
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < args.ramp_ms:
            launch(0)
            dx.check(L.dxh_device_sync())
        a, b = Events().pair()
        dx.check(L.dxh_event_record(a, None))
        for i in range(args.steps):
            dx.check(launch(i), "matmul")
        dx.check(L.dxh_event_record(b, None))
        dx.check(L.dxh_event_sync(b))
        ms = Events.ms(a, b) / args.steps
        print(json.dumps({"matmul_bf16": args.matmul_only, "tile_knob": args.matmul_tile, "launches": args.steps, "us_per_launch": round(ms * 1e3, 2),
                          "TFLOP/s": round(2 * mm * kk * nn / ms / 1e9, 1), "frac_mfma_bf16": round(2 * mm * kk * nn / ms / 1e9 / MFMA_BF16_PEAK_TF, 4),
                          "device": name.value.decode()}))
        return

    if args.block_only:
        out = config5_block_over_ir(only=args.block_only, iters=args.steps)
        out["device"] = name.value.decode()
        print(json.dumps(out))
        return

    if args.attention_only:
        out = attention_core_over_ir(only=args.attention_only, iters=args.steps)
        out["device"] = name.value.decode()
        print(json.dumps(out))
        return

    if args.chain_only:
        runs = fused_run_calls(L, dx, torch, dev)
        label = [k for k in runs if k.startswith(args.chain_only)][0]
        calls, nbytes = runs[label]
        dx.check(L.dxh_tune(12, args.chain_static), "DXH_TUNE_CHAIN_STATIC")
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < args.ramp_ms:
            dx.check(calls[0](), label)
            dx.check(L.dxh_device_sync())
        a, b = Events().pair()
        dx.check(L.dxh_event_record(a, None))
        for i in range(args.steps):
            dx.check(calls[i % len(calls)](), label)
        dx.check(L.dxh_event_record(b, None))
        dx.check(L.dxh_event_sync(b))
        ms = Events.ms(a, b) / args.steps
        print(json.dumps({"fused_run": label, "compiled_kernel": bool(args.chain_static), "launches": args.steps, "us_per_launch": round(ms * 1e3, 2),
                          "GB/s": round(nbytes / ms / 1e6, 1), "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4), "bytes": nbytes,
                          "device": name.value.decode()}))
        return

    # ---------------- config 2: the step --------------------------------------------------
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    NX = 3
    Xs = [torch.randn(8192, 8192, generator=g, device=dev, dtype=torch.float32) for _ in range(NX)]
    g.manual_seed(4)
    Ps = [torch.rand(8192, 64, generator=g, device=dev, dtype=torch.float32) * 0.2 + 0.9 for _ in range(NX)]
    out = torch.empty(8192, device=dev, dtype=torch.float32)
    shX, shP = dx.i32arr([8192, 8192]), dx.i32arr([8192, 64])
    ax0, ax1 = dx.i32arr([0]), dx.i32arr([1])
    wsb = C.c_size_t(0)
    dx.check(L.dxh_reduce_workspace_bytes(dx.F32, shX, 2, ax0, 1, C.byref(wsb)))
    ws = torch.empty(max(1, wsb.value), device=dev, dtype=torch.uint8)
    XB = 8192 * 8192 * 4 + 8192 * 4
    PB = 8192 * 64 * 4 + 8192 * 4
    # (label, fn, shape, axis, which buffers, algorithmic bytes, kernel)
    row_ops = [("sum_axis1", L.dxh_sum), ("reducemax_axis1", L.dxh_reducemax), ("reducemin_axis1", L.dxh_reducemin)]
    # launch order inside a step: the six contiguous-axis reductions back to back, then the two
    # strided-axis sums, then the two small prods — so that ONE event pair brackets each kernel's
    # launches and the event overhead (~2 us per pair) is not charged to every 40 us kernel
    groups = [
        ("reduce_row_kernel", [(n + "_" + kd, f, shX, ax1, Xs, XB) for kd in ("kd1", "kd0") for n, f in row_ops]),
        ("reduce_col_kernel", [("sum_axis0_" + kd, L.dxh_sum, shX, ax0, Xs, XB) for kd in ("kd1", "kd0")]),
        ("reduce_row_kernel(small)", [("prod_8192x64_axis1_" + kd, L.dxh_prod, shP, ax1, Ps, PB) for kd in ("kd1", "kd0")]),
    ]
    step_bytes = sum(o[5] for _, ops in groups for o in ops)
    n_ops = sum(len(ops) for _, ops in groups)
    rot = [0]

    def run_step(events=None, stream=None):
        for gi, (kern, ops) in enumerate(groups):
            if events is not None and events[gi] is not None:
                L.dxh_event_record(events[gi][0], None)
            for (label, fn, sh, ax, bufs, nbytes) in ops:
                buf = bufs[rot[0] % NX]
                rot[0] += 1
                rc = fn(dx.F32, ptr(buf), sh, 2, ax, 1, ptr(out), ptr(ws), wsb.value, stream)
                if rc != 0:
                    dx.check(rc, label)
            if events is not None and events[gi] is not None:
                L.dxh_event_record(events[gi][1], None)

    # Inside the timed region only the dominant kernel's group carries an event pair (an event
    # record is a barrier packet of its own and costs the step about a microsecond); the other
    # groups are timed the same way in a pass of their own after it.
    ev = Events()
    step_events = [[ev.pair() if gi == 0 else None for gi, _ in enumerate(groups)] for _ in range(args.steps)]
    info_events = [[ev.pair() for _ in groups] for _ in range(args.steps)]
    ramp_t0 = time.perf_counter()
    while (time.perf_counter() - ramp_t0) * 1e3 < args.ramp_ms:  # untimed: clocks settle
        run_step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        run_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(args.steps):
        run_step(step_events[s])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    for s in range(args.steps):  # untimed pass: every group with its own event pair
        run_step(info_events[s])
    torch.cuda.synchronize()
    c2 = {}
    group_ms = {}
    for gi, (kern, ops) in enumerate(groups):
        src = step_events if gi == 0 else info_events
        ms = float(np.mean([Events.ms(*src[s][gi]) for s in range(args.steps)])) / len(ops)
        group_ms[kern] = ms
        nb = ops[0][5]
        c2[kern] = {"ops": [o[0] for o in ops], "avg_launch_ms": round(ms, 5), "GB/s": round(nb / ms / 1e6, 1),
                    "frac_hbm": round(nb / ms / 1e6 / HBM_PEAK_GBS, 4), "bytes_per_launch": nb}
    # For information, not `value`: the same step recorded once into a HIP graph (dxh_graph_*, what
    # the executor does for repeated multi-line datagrams) and replayed; NX steps per graph so the
    # rotation of the input copies is the same as above.
    gst, gexec = C.c_void_p(), C.c_void_p()
    dx.check(L.dxh_stream_create(C.byref(gst)))
    rot[0] = 0
    dx.check(L.dxh_graph_begin_capture(gst))
    for _ in range(NX):
        run_step(stream=gst)
    dx.check(L.dxh_graph_end_capture(gst, C.byref(gexec)))
    for _ in range(40):
        dx.check(L.dxh_graph_launch(gexec, gst))
    dx.check(L.dxh_stream_sync(gst))
    g_t0 = time.perf_counter()
    g_reps = max(1, args.steps // NX + 1)
    for _ in range(g_reps):
        dx.check(L.dxh_graph_launch(gexec, gst))
    dx.check(L.dxh_stream_sync(gst))
    graph_ms_per_step = (time.perf_counter() - g_t0) * 1e3 / (g_reps * NX)
    dx.check(L.dxh_graph_destroy(gexec))
    dx.check(L.dxh_stream_destroy(gst))
    c2["step_as_recorded_hip_graph"] = {"ms_per_step": round(graph_ms_per_step, 4), "GB/s": round(step_bytes / graph_ms_per_step / 1e6, 1),
                                        "frac_hbm": round(step_bytes / graph_ms_per_step / 1e6 / HBM_PEAK_GBS, 4), "bytes": step_bytes}
    # For information, not `value`: the ten ops dealt out over two streams (each with its own output and scratch):
    # none of them reads what another writes, so the end of one launch runs under the start of the next.
    two = []
    for _ in range(0 if args.in_order_only else 2):
        s2 = C.c_void_p()
        dx.check(L.dxh_stream_create(C.byref(s2)))
        two.append((s2, torch.empty(8192, device=dev, dtype=torch.float32), torch.empty(max(1, wsb.value), device=dev, dtype=torch.uint8)))
    flat_ops = [o for _, ops in groups for o in ops]

    def run_step_two_streams():
        for i, (label, fn, sh, ax, bufs, nbytes) in enumerate(flat_ops):
            s2, o2, w2 = two[i % 2]
            buf = bufs[rot[0] % NX]
            rot[0] += 1
            rc = fn(dx.F32, ptr(buf), sh, 2, ax, 1, ptr(o2), ptr(w2), wsb.value, s2)
            if rc != 0:
                dx.check(rc, label)

    if two:
        for _ in range(20):
            run_step_two_streams()
        dx.check(L.dxh_device_sync())
        t_t0 = time.perf_counter()
        for _ in range(args.steps):
            run_step_two_streams()
        dx.check(L.dxh_device_sync())
        two_ms = (time.perf_counter() - t_t0) * 1e3 / args.steps
        for s2, _, _ in two:
            dx.check(L.dxh_stream_destroy(s2))
        c2["step_on_two_streams"] = {"ms_per_step": round(two_ms, 4), "GB/s": round(step_bytes / two_ms / 1e6, 1),
                                     "frac_hbm": round(step_bytes / two_ms / 1e6 / HBM_PEAK_GBS, 4), "bytes": step_bytes}
    del two
    dom_ms = group_ms["reduce_row_kernel"]
    achieved = XB / dom_ms / 1e6
    roofline = {"bound": "hbm", "kernel": "reduce_row_kernel<sum|max|min,f32> [8192,8192] axis 1 (6 of 10 launches per step)",
                "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "avg_launch_ms": round(dom_ms, 5),
                "bytes_per_launch": XB,
                # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by the
                # reading of a plain copy kernel of known size (profiles/bench_pmc_hbm_traffic.md)
                "traffic": None}
    roofline["traffic"], roofline["traffic_from"] = measured_traffic("reduce_row_kernel f32 [8192,8192] axis 1")

    # ---------------- the other BASELINE configs, one op at a time ----------------------------
    per_op = {"config2": c2}
    if not args.no_per_op:
        del Xs, Ps
        torch.cuda.empty_cache()
        per_op.update(bench_other_configs(L, dx, torch, np, dev, ev, Events, ptr))
        per_op["config2"]["step_over_deepxIR"] = config2_step_over_ir(step_bytes, side_streams=not args.in_order_only)
        per_op["attention_core_over_deepxIR"] = attention_core_over_ir()

    # ---------------- CPU baseline: the oracle's restatement of op-ompsimd's reduce ---------
    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(np, dx)
        if not args.no_per_op:
            merge_cpu_per_op(per_op, cpu_per_op(np, dx))

    line = {
        "metric": "achieved HBM GB/s & % of peak per deepxIR op; matmul TFLOP/s; vs op-ompsimd",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config2: reductions on fp32 [8192,8192] (sum axis1/axis0, reducemax, reducemin) + prod [8192,64], keepdims true+false, 10 ops/step",
                   "bytes_per_step": step_bytes, "input_copies_rotated": NX, "clock_ramp_ms_before_warmup": args.ramp_ms,
                   "device": name.value.decode()},
        "roofline": roofline,
        "roofline_matmul": roofline_matmul(per_op),
        "cpu_baseline": cpu,
        "per_op": per_op,
    }
    print(json.dumps(line))


def roofline_matmul(per_op):
    """The kernel furthest from its roofline, beside the headline one: the bf16 GEMMs of config 5
    against the dense bf16 matrix-pipe peak, from the per-op pass (None when that pass was skipped)."""
    c5 = per_op.get("config5")
    if not c5:
        return None
    shapes = {k: v for k, v in c5.items() if k in ("matmul_bf16_2048x896x4864", "matmul_bf16_2048x4864x896")}
    extra = {k: {"TFLOP/s": v["TFLOP/s"], "frac": v["frac_mfma_bf16"], "ms": v["ms"]} for k, v in c5.items() if k.startswith("matmul_bf16_") and k not in shapes}
    worst = min(shapes, key=lambda k: shapes[k]["TFLOP/s"])
    return {"bound": "mfma", "kernel": "bf16 matmul, fp32 accumulate (config 5); `achieved` is the slower of the two shapes",
            "achieved": shapes[worst]["TFLOP/s"], "peak": MFMA_BF16_PEAK_TF, "unit": "TFLOP/s",
            "frac": round(shapes[worst]["TFLOP/s"] / MFMA_BF16_PEAK_TF, 4), "shape": worst,
            "per_shape": {k: {"TFLOP/s": v["TFLOP/s"], "frac": v["frac_mfma_bf16"], "ms": v["ms"]} for k, v in shapes.items()},
            "other_shapes": extra,
            "traffic": measured_traffic("matmul bf16 " + worst.split("_")[-1])[0],
            "traffic_from": measured_traffic("matmul bf16 " + worst.split("_")[-1])[1]}


RAMP_MS = 40.0  # untimed launches before every measurement: from idle the clocks take ~30 ms of load to settle


def time_op(L, dx, torch, Events, ev, launch, reps=20, warm=3):
    """average time (ms) of `launch(i)`: one hipEvent pair on the NULL stream around `reps`
    back-to-back launches (callers rotate buffers through `i` so inputs come from HBM)"""
    t0 = time.perf_counter()
    while True:
        for i in range(warm):
            launch(i)
        torch.cuda.synchronize()
        if (time.perf_counter() - t0) * 1e3 >= RAMP_MS:
            break
    a, b = ev.pair()
    L.dxh_event_record(a, None)
    for i in range(reps):
        rc = launch(warm + i)
        if rc:
            dx.check(rc, "bench op")
    L.dxh_event_record(b, None)
    torch.cuda.synchronize()
    return Events.ms(a, b) / reps


def bench_other_configs(L, dx, torch, np, dev, ev, Events, ptr):
    res = {}

    def entry(ms, nbytes=None, flops=None, peak_tf=MFMA_BF16_PEAK_TF, peak_name="frac_mfma_bf16"):
        e = {"ms": round(ms, 5)}
        if nbytes is not None:
            e.update({"GB/s": round(nbytes / ms / 1e6, 1), "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4), "bytes": nbytes})
        if flops is not None:
            e.update({"TFLOP/s": round(flops / ms / 1e9, 2), peak_name: round(flops / ms / 1e9 / peak_tf, 4), "flops": flops})
        return e

    # ---- the floor under every small op: one launch of a kernel with nothing to do (a fill of one
    # element), timed like every op below (back-to-back launches between two events), and the round
    # trip of launching it and waiting for it (what a caller that needs each result pays per op)
    one = torch.empty(64, device=dev)
    zero = dx.scalar(0.0)
    floor_ms = time_op(L, dx, torch, Events, ev, lambda i: L.dxh_constant(dx.F32, ptr(one), 1, zero, None), reps=200)
    t0 = time.perf_counter()
    for _ in range(500):
        L.dxh_constant(dx.F32, ptr(one), 1, zero, None)
        L.dxh_stream_sync(None)
    res["launch_floor"] = {"back_to_back_us": round(floor_ms * 1e3, 2), "launch_and_wait_us": round((time.perf_counter() - t0) / 500 * 1e6, 2),
                           "note": "ops whose time is within a microsecond or two of back_to_back_us are launch-bound, not bandwidth-bound"}

    # ---- config 1: fp32 [4096,4096] elementwise chain; 4 rotating buffer sets (64 MiB tensors)
    n = 4096 * 4096
    R = 4
    A = [torch.rand(n, device=dev) * 2 - 1 for _ in range(R)]
    B = [torch.rand(n, device=dev) * 2 - 1 for _ in range(R)]
    O = [torch.empty(n, device=dev) for _ in range(R)]
    half = dx.scalar(0.5)
    c1 = {}
    c1["add"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_add(dx.F32, ptr(A[i % R]), ptr(B[i % R]), ptr(O[i % R]), n, None)), 3 * n * 4)
    c1["mul"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_mul(dx.F32, ptr(A[i % R]), ptr(B[i % R]), ptr(O[i % R]), n, None)), 3 * n * 4)
    c1["max"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_max(dx.F32, ptr(A[i % R]), ptr(B[i % R]), ptr(O[i % R]), n, None)), 3 * n * 4)
    c1["div"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_div(dx.F32, ptr(A[i % R]), ptr(B[i % R]), ptr(O[i % R]), n, None)), 3 * n * 4)
    c1["addscalar"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_addscalar(dx.F32, ptr(A[i % R]), half, ptr(O[i % R]), n, None)), 2 * n * 4)
    c1["mulscalar"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_mulscalar(dx.F32, ptr(A[i % R]), half, ptr(O[i % R]), n, None)), 2 * n * 4)
    c1["exp"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_exp(dx.F32, ptr(A[i % R]), ptr(O[i % R]), n, None)), 2 * n * 4)
    res["config1"] = c1
    del A, B, O
    torch.cuda.empty_cache()

    # ---- config 3: changeshape on 16-bit tensors
    c3 = {}
    shape = [32, 2048, 14, 64]
    nt = 32 * 2048 * 14 * 64
    T = [torch.randn(nt, device=dev).to(torch.bfloat16) for _ in range(3)]
    TO = [torch.empty(nt, device=dev, dtype=torch.bfloat16) for _ in range(3)]
    sh, od = dx.i32arr(shape), dx.i32arr([0, 2, 1, 3])
    c3["transpose_bf16_32x2048x14x64_0213"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_transpose(dx.BF16, ptr(T[i % 3]), sh, 4, od, ptr(TO[i % 3]), None)), 2 * nt * 2)
    del T, TO
    torch.cuda.empty_cache()
    nc = 16 * 1024 * 4096
    cs = [torch.randn(nc, device=dev).to(torch.float16) for _ in range(3)]
    co = [torch.empty(3 * nc, device=dev, dtype=torch.float16) for _ in range(2)]
    ins = dx.ptrarr([t.data_ptr() for t in cs])
    axs, osh = dx.i32arr([1024] * 3), dx.i32arr([16, 3072, 4096])
    c3["concat_fp16_3x16x1024x4096_axis1"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_concat(dx.F16, ins, 3, axs, osh, 3, 1, ptr(co[i % 2]), None)), 2 * 3 * nc * 2)
    del cs, co
    torch.cuda.empty_cache()
    r = torch.randn(4096, device=dev).to(torch.bfloat16)
    bo = [torch.empty(8192 * 4096, device=dev, dtype=torch.bfloat16) for _ in range(5)]
    ish, bsh = dx.i32arr([1, 4096]), dx.i32arr([8192, 4096])
    c3["broadcastTo_bf16_1x4096_to_8192x4096"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_broadcastTo(dx.BF16, ptr(r), ish, 2, bsh, 2, ptr(bo[i % 5]), None)), 8192 + 8192 * 4096 * 2)
    del bo
    torch.cuda.empty_cache()
    res["config3"] = c3

    # ---- config 4: int32 2^26 and the embedding gather
    c4 = {}
    n = 1 << 26
    a = [torch.randint(-2 ** 20, 2 ** 20 + 1, (n,), device=dev, dtype=torch.int32) for _ in range(2)]
    b = [torch.randint(-2 ** 20, 2 ** 20 + 1, (n,), device=dev, dtype=torch.int32) for _ in range(2)]
    o = [torch.empty(n, device=dev, dtype=torch.int32) for _ in range(2)]
    m = [torch.empty(n, device=dev, dtype=torch.uint8) for _ in range(2)]
    c4["max_i32_2^26"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_max(dx.I32, ptr(a[i % 2]), ptr(b[i % 2]), ptr(o[i % 2]), n, None)), 3 * n * 4)
    c4["min_i32_2^26"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_min(dx.I32, ptr(a[i % 2]), ptr(b[i % 2]), ptr(o[i % 2]), n, None)), 3 * n * 4)
    c4["greater_i32_2^26"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_greater(dx.I32, ptr(a[i % 2]), ptr(b[i % 2]), ptr(m[i % 2]), n, None)), 2 * n * 4 + n)
    sw = [dx.ptrarr([b[j].data_ptr(), a[j].data_ptr()]) for j in range(2)]
    c4["where_i32_2^26(switch)"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_switch(dx.I32, sw[i % 2], 2, dx.BOOL, ptr(m[i % 2]), ptr(o[i % 2]), n, None)), n + 3 * n * 4)
    del a, b, o, m
    torch.cuda.empty_cache()
    E = (torch.randn(151936, 896, device=dev) * 0.02).to(torch.bfloat16)
    # 48 index sets: 196,608 rows of 1792 bytes = 352 MB of distinct table rows between two uses of a set, more
    # than the 256 MiB last-level cache holds, so the gathered rows come from HBM
    NI = 48
    idx = [torch.randint(0, 151936, (4096,), device=dev, dtype=torch.int64) for _ in range(NI)]
    eo = torch.empty(4096 * 896, device=dev, dtype=torch.bfloat16)
    esh, xsh = dx.i32arr([151936, 896]), dx.i32arr([4096])
    c4["indexselect_bf16_4096_of_151936x896(latency-bound)"] = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_indexselect(dx.BF16, ptr(E), esh, 2, dx.I64, ptr(idx[i % NI]), xsh, 1, 0, ptr(eo), None), reps=NI - 3), 2 * 4096 * 896 * 2 + 4096 * 8)
    c4["indexselect_bf16_4096_of_151936x896(latency-bound)"]["index_sets_rotated"] = NI
    del E, eo
    torch.cuda.empty_cache()
    res["config4"] = c4

    # ---- config 5: the three bf16 GEMMs of the Qwen2-0.5B MLP (fp32 accumulate)
    c5 = {}
    for label, (mm, kk, nn) in [("matmul_bf16_2048x896x4864", (2048, 896, 4864)), ("matmul_bf16_2048x4864x896", (2048, 4864, 896))]:
        Am = torch.randn(mm * kk, device=dev).to(torch.bfloat16)
        Bm = (torch.randn(kk * nn, device=dev) * 0.02).to(torch.bfloat16)
        Cm = torch.empty(mm * nn, device=dev, dtype=torch.bfloat16)
        c5[label] = entry(time_op(L, dx, torch, Events, ev, matmul_call(L, dx, torch, dev, dx.BF16, Am, Bm, Cm, mm, kk, nn)), flops=2 * mm * kk * nn)
        c5[label]["hipblaslt_TFLOP/s"] = vendor_gemm_tflops(torch, Am.view(mm, kk), Bm.view(kk, nn), Cm.view(mm, nn))
    # the gate and the up projection of the block share their activations: both products as one dxh_matmul_shared_a
    # call (what the executor's batch path does with the two consecutive matmul lines), against two dxh_matmul calls
    mm, kk, nn = 2048, 896, 4864
    Am = torch.randn(mm * kk, device=dev).to(torch.bfloat16)
    Bs = [(torch.randn(kk * nn, device=dev) * 0.02).to(torch.bfloat16) for _ in range(2)]
    Cs = [torch.empty(mm * nn, device=dev, dtype=torch.bfloat16) for _ in range(2)]
    bs, cs = dx.ptrarr([t.data_ptr() for t in Bs]), dx.ptrarr([t.data_ptr() for t in Cs])
    e = entry(time_op(L, dx, torch, Events, ev, lambda i: L.dxh_matmul_shared_a(dx.BF16, ptr(Am), bs, cs, 2, mm, kk, nn, None, 0, None)), flops=2 * 2 * mm * kk * nn)
    pair = [matmul_call(L, dx, torch, dev, dx.BF16, Am, Bs[j], Cs[j], mm, kk, nn) for j in range(2)]
    e["as_two_launches_ms"] = round(time_op(L, dx, torch, Events, ev, lambda i: pair[0](i) or pair[1](i)), 5)
    c5["matmul_bf16_2048x896x4864_x2_shared_A(gate+up, one launch)"] = e
    # two square shapes outside BASELINE, where a round of tiles is long against the launch and the stores
    for side in (4096, 8192):
        Am = torch.randn(side * side, device=dev).to(torch.bfloat16)
        Bm = (torch.randn(side * side, device=dev) * 0.02).to(torch.bfloat16)
        Cm = torch.empty(side * side, device=dev, dtype=torch.bfloat16)
        label = f"matmul_bf16_{side}x{side}x{side}(outside BASELINE)"
        c5[label] = entry(time_op(L, dx, torch, Events, ev, matmul_call(L, dx, torch, dev, dx.BF16, Am, Bm, Cm, side, side, side), reps=10), flops=2 * side ** 3)
        c5[label]["hipblaslt_TFLOP/s"] = vendor_gemm_tflops(torch, Am.view(side, side), Bm.view(side, side), Cm.view(side, side), reps=10)
    del Bs, Cs, pair
    # the same shapes in fp32, the dtype the reference's own matmul (cublasSgemm / cblas_sgemm) runs in
    for label, (mm, kk, nn) in [("matmul_f32_2048x896x4864", (2048, 896, 4864)), ("matmul_f32_2048x4864x896", (2048, 4864, 896))]:
        Am = torch.randn(mm * kk, device=dev)
        Bm = torch.randn(kk * nn, device=dev) * 0.02
        Cm = torch.empty(mm * nn, device=dev)
        c5[label] = entry(time_op(L, dx, torch, Events, ev, matmul_call(L, dx, torch, dev, dx.F32, Am, Bm, Cm, mm, kk, nn)),
                          flops=2 * mm * kk * nn, peak_tf=MFMA_F32_PEAK_TF, peak_name="frac_mfma_f32")
        c5[label]["hipblaslt_TFLOP/s"] = vendor_gemm_tflops(torch, Am.view(mm, kk), Bm.view(kk, nn), Cm.view(mm, nn))
    # and in fp64, which the reference's dispatch also accepts (v_mfma_f64_16x16x4_f64)
    for label, (mm, kk, nn) in [("matmul_f64_2048x896x4864", (2048, 896, 4864)), ("matmul_f64_2048x4864x896", (2048, 4864, 896))]:
        Am = torch.randn(mm * kk, device=dev, dtype=torch.float64)
        Bm = torch.randn(kk * nn, device=dev, dtype=torch.float64) * 0.02
        Cm = torch.empty(mm * nn, device=dev, dtype=torch.float64)
        c5[label] = entry(time_op(L, dx, torch, Events, ev, matmul_call(L, dx, torch, dev, dx.F64, Am, Bm, Cm, mm, kk, nn)),
                          flops=2 * mm * kk * nn, peak_tf=MFMA_F64_PEAK_TF, peak_name="frac_mfma_f64")
        c5[label]["hipblaslt_TFLOP/s"] = vendor_gemm_tflops(torch, Am.view(mm, kk), Bm.view(kk, nn), Cm.view(mm, nn))
    del Am, Bm, Cm
    torch.cuda.empty_cache()
    # the glue ops of the block at their own sizes (7-20 MB tensors: they fit the 256 MiB Infinity
    # Cache, so the rates are cache rates and say little about HBM; 6 buffer sets are rotated anyway)
    S, Hd, I, R6 = 2048, 896, 4864, 6
    g16 = [torch.randn(S * I, device=dev).to(torch.bfloat16) for _ in range(R6)]
    u16 = [torch.randn(S * I, device=dev).to(torch.bfloat16) for _ in range(R6)]
    o16 = [torch.empty(S * I, device=dev, dtype=torch.bfloat16) for _ in range(R6)]
    x16 = [torch.randn(S * Hd, device=dev).to(torch.bfloat16) for _ in range(R6)]
    x32 = [torch.randn(S * Hd, device=dev) for _ in range(R6)]
    o32 = [torch.empty(S * Hd, device=dev) for _ in range(R6)]
    col = [torch.rand(S, device=dev) + 0.5 for _ in range(R6)]
    n16, n32 = S * I, S * Hd
    one, two, neg = dx.scalar(1.0), dx.scalar(2.0), dx.scalar(-1.0)
    shx, ax1, shc, shb = dx.i32arr([S, Hd]), dx.i32arr([1]), dx.i32arr([S, 1]), dx.i32arr([S, Hd])
    glue = {
        "mulscalar_bf16_2048x4864": (lambda i: L.dxh_mulscalar(dx.BF16, ptr(g16[i % R6]), neg, ptr(o16[i % R6]), n16, None), 2 * n16 * 2),
        "exp_bf16_2048x4864": (lambda i: L.dxh_exp(dx.BF16, ptr(g16[i % R6]), ptr(o16[i % R6]), n16, None), 2 * n16 * 2),
        "rdivscalar_bf16_2048x4864": (lambda i: L.dxh_rdivscalar(dx.BF16, one, ptr(g16[i % R6]), ptr(o16[i % R6]), n16, None), 2 * n16 * 2),
        "mul_bf16_2048x4864": (lambda i: L.dxh_mul(dx.BF16, ptr(g16[i % R6]), ptr(u16[i % R6]), ptr(o16[i % R6]), n16, None), 3 * n16 * 2),
        "todtype_bf16_to_f32_2048x896": (lambda i: L.dxh_todtype(dx.BF16, ptr(x16[i % R6]), dx.F32, ptr(o32[i % R6]), n32, None), n32 * 6),
        "powscalar_f32_2048x896": (lambda i: L.dxh_powscalar(dx.F32, ptr(x32[i % R6]), two, ptr(o32[i % R6]), n32, None), 2 * n32 * 4),
        "sum_f32_2048x896_axis1_keepdims": (lambda i: L.dxh_sum(dx.F32, ptr(x32[i % R6]), shx, 2, ax1, 1, ptr(col[i % R6]), None, 0, None), n32 * 4 + S * 4),
        "broadcastTo_f32_2048x1_to_2048x896": (lambda i: L.dxh_broadcastTo(dx.F32, ptr(col[i % R6]), shc, 2, shb, 2, ptr(o32[i % R6]), None), n32 * 4 + S * 4),
    }
    c5["glue_ops(cache-resident sizes)"] = {k: entry(time_op(L, dx, torch, Events, ev, fn), nb) for k, (fn, nb) in glue.items()}
    # the same glue as the executor's batch path launches it: the RMSNorm's thirteen lines (row sum included), the
    # SiLU gate's six lines and the softmax's eight lines, one launch each (dxh_chain_rows / dxh_chain); bytes =
    # inputs once + every tensor the lines store.  Each run has a compiled kernel in the library; the same
    # launches through the interpreting kernel (DXH_TUNE_CHAIN_STATIC 0) are timed beside them.
    runs = fused_run_calls(L, dx, torch, dev, R6)
    fused = {}
    for label, (calls, nbytes) in runs.items():
        e = entry(time_op(L, dx, torch, Events, ev, lambda i: calls[i % len(calls)]()), nbytes)
        dx.check(L.dxh_tune(12, 0))
        try:
            probe = calls[0]()
            if probe == 0:
                e["interpreted_ms"] = round(time_op(L, dx, torch, Events, ev, lambda i: calls[i % len(calls)]()), 5)
            else:
                e["interpreted_ms"] = None  # rows too long (or 16-bit row reductions) for the interpreting kernel's lane layout
        finally:
            dx.check(L.dxh_tune(12, 1))
        # outputs of up to 32 MiB leave with write-through stores so that the next kernel finds them in the last-level
        # cache; here, alone and on rotating buffers, nothing reads them: the same launches with non-temporal stores
        dx.check(L.dxh_tune(0, 0))
        try:
            e["with_nt_stores_ms"] = round(time_op(L, dx, torch, Events, ev, lambda i: calls[i % len(calls)]()), 5)
        finally:
            dx.check(L.dxh_tune(0, 32 << 20))
        fused[label] = e
    fused["note"] = ("one launch per run through the library's compiled kernel for that sequence; interpreted_ms = the same launch through "
                     "the op-table interpreter; with_nt_stores_ms = the compiled kernel with DXH_TUNE_NT_STORE_BYTES 0 (what the run costs when "
                     "nothing reads its outputs from the cache afterwards); as separate launches the lines take the sum of the glue_ops entries above")
    c5["fused_runs(one launch each)"] = fused
    del runs
    del g16, u16, o16, x16, x32, o32, col
    torch.cuda.empty_cache()
    c5["mlp_block_over_deepxIR"] = config5_block_over_ir()
    c5["mlp_block_with_its_allocations"] = config5_block_over_ir(with_allocations=True)
    res["config1"]["chain_over_deepxIR"] = config1_chain_over_ir()
    res["config5"] = c5
    return res


def fused_run_calls(L, dx, torch, dev, sets=6):
    """The front's three fixed sequences as single launches on rotating buffer sets: {label: ([call, ...], bytes)}.
    Each call returns the entry point's status."""
    import ctypes as C
    S, Hd, I = 2048, 896, 4864
    FULL, ROW, COL, RES = dx.CHAIN_FULL, dx.CHAIN_ROW, dx.CHAIN_COLUMN, dx.CHAIN_RESULT
    code = dx.CHAIN_CODES.index
    n16, n32 = S * I, S * Hd
    keep = []  # tensors stay alive as long as the calls do

    def norm_run():
        x16 = torch.randn(n32, device=dev).to(torch.bfloat16)
        w16 = torch.ones(Hd, device=dev, dtype=torch.bfloat16)
        xf, sq, rs, wf, xn = (torch.empty(n32, device=dev) for _ in range(5))
        wf1, col, h16 = torch.empty(Hd, device=dev), torch.empty(S, device=dev), torch.empty(n32, device=dev, dtype=torch.bfloat16)
        keep.extend([x16, w16, xf, sq, rs, wf, xn, wf1, col, h16])
        prog = [("copy", 0, 0, 0, dx.F32, FULL, xf), ("square", RES + 0, 0, 2.0, dx.F32, FULL, sq), ("rowsum", RES + 1, 0, 0, dx.F32, COL, None),
                ("divscalar", RES + 2, 0, float(Hd), dx.F32, COL, None), ("addscalar", RES + 3, 0, 1e-6, dx.F32, COL, None),
                ("sqrt", RES + 4, 0, 0, dx.F32, COL, None), ("rdivscalar", RES + 5, 0, 1.0, dx.F32, COL, col),
                ("copy", RES + 6, 0, 0, dx.F32, FULL, rs), ("mul", RES + 0, RES + 7, 0, dx.F32, FULL, None), ("copy", 1, 0, 0, dx.F32, ROW, wf1),
                ("copy", RES + 9, 0, 0, dx.F32, FULL, wf), ("mul", RES + 10, RES + 8, 0, dx.F32, FULL, xn), ("copy", RES + 11, 0, 0, dx.BF16, FULL, h16)]
        tin = (dx.ChainTensor * 2)(dx.ChainTensor(x16.data_ptr(), dx.BF16, FULL), dx.ChainTensor(w16.data_ptr(), dx.BF16, ROW))
        ops = (dx.ChainRowsOp * len(prog))(*[dx.ChainRowsOp(code(n), l, r, dx.scalar(sc), o.data_ptr() if o is not None else None, dt, e)
                                             for n, l, r, sc, dt, e, o in prog])
        return lambda: L.dxh_chain_rows(tin, 2, ops, len(prog), S, Hd, None)

    def gate_run():
        g16, u16 = (torch.randn(n16, device=dev).to(torch.bfloat16) for _ in range(2))
        o16 = torch.empty(n16, device=dev, dtype=torch.bfloat16)
        keep.extend([g16, u16, o16])
        prog = [("mulscalar", 0, 0, -1.0), ("exp", RES + 0, 0, 0), ("addscalar", RES + 1, 0, 1.0), ("rdivscalar", RES + 2, 0, 1.0), ("mul", 0, RES + 3, 0), ("mul", RES + 4, 1, 0)]
        ops = (dx.ChainOp * len(prog))(*[dx.ChainOp(code(n), l, r, dx.scalar(sc), o16.data_ptr() if k == len(prog) - 1 else None) for k, (n, l, r, sc) in enumerate(prog)])
        ins = (C.c_void_p * 2)(g16.data_ptr(), u16.data_ptr())
        return lambda: L.dxh_chain(dx.BF16, ins, 2, ops, len(prog), n16, None)

    def softmax_run(rows, cols, dt, tdt):
        t = (torch.randn(rows * cols, device=dev) * 3).to(tdt)
        full = [torch.empty(rows * cols, device=dev, dtype=tdt) for _ in range(6)]  # mb d e e2 sb y
        cols_ = [torch.empty(rows, device=dev, dtype=tdt) for _ in range(2)]        # m s
        keep.extend([t] + full + cols_)
        mb, d, e, e2, sb, y = full
        prog = [("rowmax", 0, 0, COL, cols_[0]), ("copy", RES + 0, 0, FULL, mb), ("sub", 0, RES + 1, FULL, d), ("exp", RES + 2, 0, FULL, e),
                ("rowsum", RES + 3, 0, COL, cols_[1]), ("exp", RES + 2, 0, FULL, e2), ("copy", RES + 4, 0, FULL, sb), ("div", RES + 5, RES + 6, FULL, y)]
        tin = (dx.ChainTensor * 1)(dx.ChainTensor(t.data_ptr(), dt, FULL))
        ops = (dx.ChainRowsOp * len(prog))(*[dx.ChainRowsOp(code(n), l, r, dx.scalar(0.0), o.data_ptr(), dt, ext) for n, l, r, ext, o in prog])
        return lambda: L.dxh_chain_rows(tin, 1, ops, len(prog), rows, cols, None)

    AR, AC = 14 * 2048, 2048  # scores of one sequence of the attention shape of config 3: 14 heads x 2048 queries x 2048 keys
    return {
        "rmsnorm_13_lines_bf16_in_f32_inside_2048x896": ([norm_run() for _ in range(sets)], n32 * 2 + 5 * n32 * 4 + n32 * 2 + S * 4 + Hd * 6),
        "silu_gate_6_lines_bf16_2048x4864": ([gate_run() for _ in range(sets)], 3 * n16 * 2),
        "softmax_8_lines_f32_28672x2048": ([softmax_run(AR, AC, dx.F32, torch.float32) for _ in range(2)], 7 * AR * AC * 4 + 2 * AR * 4),
        "softmax_8_lines_bf16_2048x896": ([softmax_run(S, Hd, dx.BF16, torch.bfloat16) for _ in range(sets)], 7 * S * Hd * 2 + 2 * S * 2),
    }


def matmul_call(L, dx, torch, dev, dtype, A, B, Cm, m, k, n):
    """One dxh_matmul launch as a closure for time_op: the workspace the library's own query asks
    for is allocated once, outside the timed region, like the executor keeps one per process."""
    import ctypes as C
    need = C.c_size_t(0)
    a, b, c = (C.c_void_p(t.data_ptr()) for t in (A, B, Cm))
    dx.check(L.dxh_matmul_workspace_bytes(dtype, a, b, c, 1, m, k, n, C.byref(need)), "matmul workspace")
    ws = torch.empty(max(1, need.value), dtype=torch.uint8, device=dev)
    wsp = C.c_void_p(ws.data_ptr()) if need.value else None
    return lambda i, ws=ws: L.dxh_matmul(dtype, a, b, c, 1, m, k, n, wsp, need.value, None)


def _executor_lib():
    import ctypes as C
    lib = os.path.join(ROOT, "deepx_amd", "executor", "libdxexec.so")
    if not os.path.exists(lib):
        raise RuntimeError("libdxexec.so is not built: run `python __graft_entry__.py build`")
    E = C.CDLL(lib)
    E.dxe_create.restype = C.c_void_p
    E.dxe_destroy.argtypes = [C.c_void_p]
    E.dxe_execute.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_size_t]
    E.dxe_execute_batch.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_size_t]
    E.dxe_set_graphs.argtypes = [C.c_void_p, C.c_int]
    E.dxe_set_fusion.argtypes = [C.c_void_p, C.c_int]
    E.dxe_set_sync.argtypes = [C.c_void_p, C.c_int]
    E.dxe_set_defer.argtypes = [C.c_void_p, C.c_int]
    E.dxe_flush.argtypes = [C.c_void_p]
    E.dxe_set_streams.argtypes = [C.c_void_p, C.c_int]
    E.dxe_set_pool.argtypes = [C.c_int]
    E.dxe_set_zero_later.argtypes = [C.c_void_p, C.c_int]
    return E


def lines_over_ir(setup, block, iters=30, only=None):
    """`block` (deepxIR lines) through the executor's dispatch core in this process (libdxexec.so, the
    code behind the UDP server): wall time per pass when the lines are executed one by one (replies
    at launch, as op-cuda sends them; with a wait for the device before every reply; and with lines that can
    share a launch held back until their run is complete, the DEEPX_DEFER switch), as one
    batch, as one batch with runs of float elementwise lines fused into single launches, and as a
    recorded HIP graph without and with those fused runs.  The timed region of every mode ends with
    a wait for the device.  Every mode gets a fresh executor (a recorded graph is keyed by the text
    of the batch)."""
    import ctypes as C
    from deepx_amd import lib as dx
    L = dx.load()
    E = _executor_lib()
    lines = [f"{l} // author=miaobyte id={i + 1}" for i, l in enumerate(block)]
    text = "\n".join(lines).encode()
    out = {"ops": len(lines)}
    for label, batched, fused, graphs, wait in (("line_by_line_us", 0, 0, 0, 0), ("line_by_line_waiting_for_each_us", 0, 0, 0, 1),
                                                ("line_by_line_deferred_us", 0, 1, 0, 0),
                                                ("one_batch_us", 1, 0, 0, 0), ("one_batch_fused_us", 1, 1, 0, 0),
                                                ("recorded_graph_us", 1, 0, 1, 0), ("recorded_graph_fused_us", 1, 1, 1, 0)):
        if only and label != only:
            continue
        ex = E.dxe_create()
        buf = C.create_string_buffer(1 << 16)
        for line in setup:
            E.dxe_execute(ex, line.encode(), buf, len(buf))
            reply = buf.value.decode()
            if " ok" not in reply.split("//")[0]:
                raise RuntimeError(f"{line}: {reply}")
        E.dxe_set_graphs(ex, graphs)
        E.dxe_set_fusion(ex, fused)
        E.dxe_set_sync(ex, wait)
        E.dxe_set_defer(ex, int(label == "line_by_line_deferred_us"))

        def once():
            if batched:
                E.dxe_execute_batch(ex, text, buf, len(buf))
            else:
                for l in lines:
                    E.dxe_execute(ex, l.encode(), buf, len(buf))

        for _ in range(4):
            once()
        E.dxe_flush(ex)
        dx.check(L.dxh_device_sync())
        t0 = time.perf_counter()
        for _ in range(iters):
            once()
        E.dxe_flush(ex)  # what the last pass left held
        dx.check(L.dxh_device_sync())
        out[label] = round((time.perf_counter() - t0) / iters * 1e6, 1)
        if any(" ok" not in r.split("//")[0] for r in buf.value.decode().split("\n")):
            raise RuntimeError("block failed: " + buf.value.decode())
        E.dxe_destroy(ex)
    return out


def config2_step_over_ir(step_bytes, iters=30, side_streams=True):
    """The config-2 step (ten reductions) as one datagram of ten deepxIR lines through the executor's dispatch core, and
    sent line by line: in order on the default stream, and with independent lines spread over side streams (the DEEPX_STREAMS switch:
    no line of the step reads what another writes, so the end of one launch runs under the start of the next).
    Three copies of the input in rotation, as in the headline step."""
    import ctypes as C
    from deepx_amd import lib as dx
    L = dx.load()
    E = _executor_lib()
    T = lambda n: f"tensor<float32>:c2_{n}"
    V = lambda v: "vector<int32>:[" + " ".join(str(x) for x in v) + "]"
    setup = [f"newtensor({V([8192, 8192])})->({T('X%d' % i)})" for i in range(3)] + [f"newtensor({V([8192, 64])})->({T('P%d' % i)})" for i in range(3)]
    setup += [f"uniform(var<float32>:0, var<float32>:1, var<int32>:{7 + i})->({T('X%d' % i)}) // author=miaobyte" for i in range(3)]
    setup += [f"uniform(var<float32>:0.9, var<float32>:1.1, var<int32>:{17 + i})->({T('P%d' % i)}) // author=miaobyte" for i in range(3)]
    outs = []
    for kd in (1, 0):
        for name in ("s1", "mx", "mn", "s0", "pr"):
            shape = ([8192, 1] if name != "s0" else [1, 8192]) if kd else [8192]
            setup.append(f"newtensor({V(shape)})->({T(f'{name}_kd{kd}')})")
    texts = []
    for i in range(3):
        lines = []
        for kd in (1, 0):
            kb = "var<bool>:true" if kd else "var<bool>:false"
            lines += [f"sum({T('X%d' % i)}, {V([1])}, {kb})->({T(f's1_kd{kd}')})", f"reducemax({T('X%d' % i)}, {V([1])}, {kb})->({T(f'mx_kd{kd}')})",
                      f"reducemin({T('X%d' % i)}, {V([1])}, {kb})->({T(f'mn_kd{kd}')})", f"sum({T('X%d' % i)}, {V([0])}, {kb})->({T(f's0_kd{kd}')})",
                      f"prod({T('P%d' % i)}, {V([1])}, {kb})->({T(f'pr_kd{kd}')})"]
        texts.append("\n".join(f"{l} // author=miaobyte id={k + 1}" for k, l in enumerate(lines)).encode())
    out = {"ops": 10, "bytes": step_bytes}
    line_sets = [[l for l in t.decode().split("\n")] for t in texts]
    for label, streams in (("one_batch_us", 1), ("one_batch_side_streams_us", 3), ("line_by_line_us", 1), ("line_by_line_side_streams_us", 3)):
        if streams > 1 and not side_streams:
            continue
        batched = label.startswith("one_batch")
        ex = E.dxe_create()
        buf = C.create_string_buffer(1 << 16)
        for line in setup:
            E.dxe_execute(ex, line.encode(), buf, len(buf))
            if " ok" not in buf.value.decode().split("//")[0]:
                raise RuntimeError(f"{line}: {buf.value.decode()}")
        E.dxe_set_streams(ex, streams)
        def once(r):
            if batched:
                E.dxe_execute_batch(ex, texts[r % 3], buf, len(buf))
            else:
                for l in line_sets[r % 3]:
                    E.dxe_execute(ex, l.encode(), buf, len(buf))

        for r in range(6):
            once(r)
        dx.check(L.dxh_device_sync())
        t0 = time.perf_counter()
        for r in range(iters):
            once(r)
        dx.check(L.dxh_device_sync())
        us = (time.perf_counter() - t0) / iters * 1e6
        if any(" ok" not in r.split("//")[0] for r in buf.value.decode().split("\n")):
            raise RuntimeError("step failed: " + buf.value.decode())
        out[label] = round(us, 1)
        out[label.replace("_us", "_GB/s")] = round(step_bytes / us / 1e3, 1)
        E.dxe_destroy(ex)
    return out


def config1_chain_over_ir(side=4096):
    """The 8-op elementwise chain of config 1 on [4096,4096] fp32 as deepxIR lines."""
    T = lambda n: f"tensor<float32>:c1_{n}"
    V = f"vector<int32>:[{side} {side}]"
    names = ["A", "B", "C", "D", "E", "F", "nB", "absB", "den", "G"]
    setup = [f"newtensor({V})->({T(n)})" for n in names]
    setup += [f"uniform(var<float32>:-1, var<float32>:1, var<int32>:{seed})->({T(n)}) // author=miaobyte" for n, seed in (("A", 1), ("B", 2))]
    block = [f"add({T('A')}, {T('B')})->({T('C')})", f"mul({T('C')}, {T('B')})->({T('D')})", f"addscalar({T('D')}, var<float32>:0.5)->({T('E')})",
             f"exp({T('E')})->({T('F')})", f"mulscalar({T('B')}, var<float32>:-1)->({T('nB')})", f"max({T('B')}, {T('nB')})->({T('absB')})",
             f"addscalar({T('absB')}, var<float32>:1)->({T('den')})", f"div({T('F')}, {T('den')})->({T('G')})"]
    return lines_over_ir(setup, block)


def attention_core_over_ir(S=2048, heads=14, hd=64, iters=20, only=None):
    """The core of the front's attention on the activations of config 3 / config 5 (one sequence of 2048 tokens, 14 heads of 64;
    front/py/deepx/nn/modules/transformer/attention.py:15-32, softmax as normalization.py:4-17 spells it), bf16, 12 deepxIR
    lines: transpose of k, q @ k.mT, the scaling, the softmax's eight lines, the product with v.  Not a BASELINE config: the
    caller next to the config-5 block, through the same executor modes."""
    dt = "bfloat16"
    T = lambda n: f"tensor<{dt}>:at_{n}"
    V = lambda v: "vector<int32>:[" + " ".join(str(x) for x in v) + "]"
    full, col, io = [1, heads, S, S], [1, heads, S, 1], [1, heads, S, hd]
    tensors = [("q", io), ("k", io), ("v", io), ("kT", [1, heads, hd, S]), ("sc", full), ("a", full), ("m", col), ("mb", full), ("d", full), ("e", full),
               ("s", col), ("e2", full), ("sb", full), ("y", full), ("o", io)]
    setup = [f"newtensor({V(shape)})->({T(name)})" for name, shape in tensors]
    setup += [f"normal(var<float32>:0, var<float32>:1, var<int32>:{21 + i})->({T(name)}) // author=miaobyte" for i, name in enumerate(("q", "k", "v"))]
    block = [f"transpose({T('k')}, {V([0, 1, 3, 2])})->({T('kT')})", f"matmul({T('q')}, {T('kT')})->({T('sc')})",
             f"mulscalar({T('sc')}, var<float32>:{hd ** -0.5})->({T('a')})",
             f"reducemax({T('a')}, {V([-1])}, var<bool>:true)->({T('m')})", f"broadcastTo({T('m')}, {V(full)})->({T('mb')})",
             f"sub({T('a')}, {T('mb')})->({T('d')})", f"exp({T('d')})->({T('e')})", f"sum({T('e')}, {V([-1])}, var<bool>:true)->({T('s')})",
             f"exp({T('d')})->({T('e2')})", f"broadcastTo({T('s')}, {V(full)})->({T('sb')})", f"div({T('e2')}, {T('sb')})->({T('y')})",
             f"matmul({T('y')}, {T('v')})->({T('o')})"]
    out = lines_over_ir(setup, block, iters=iters, only=only)
    es, n_full = 2, heads * S * S
    # what the twelve lines move when every line is a launch of its own, and when the nine from the scaling to the division are one
    io_b = heads * S * hd * es
    out["bytes_line_by_line"] = (2 * io_b) + (2 * io_b + n_full * es) + 2 * n_full * es + n_full * es + n_full * es + 3 * n_full * es + 2 * n_full * es + n_full * es + 2 * n_full * es + n_full * es + 3 * n_full * es + (n_full * es + 2 * io_b)
    out["bytes_fused"] = (2 * io_b) + (2 * io_b + n_full * es) + 8 * n_full * es + (n_full * es + 2 * io_b)
    out["shape"] = f"[1,{heads},{S},{hd}] {dt}"
    return out


def config5_block_over_ir(rows=2048, hidden=896, inter=4864, only=None, iters=30, with_allocations=False):
    """The whole config-5 block (RMSNorm + gated MLP, 22 deepxIR compute ops on [2048,896] activations)."""
    S, Hd, I = rows, hidden, inter
    b16, f32 = "bfloat16", "float32"
    T = lambda n, dt=f32: f"tensor<{dt}>:{n}"
    V = lambda v: "vector<int32>:[" + " ".join(str(x) for x in v) + "]"
    tensors = [("x", [S, Hd], b16), ("w", [1, Hd], b16), ("Wg", [Hd, I], b16), ("Wu", [Hd, I], b16), ("Wd", [I, Hd], b16),
               ("xf", [S, Hd], f32), ("sq", [S, Hd], f32), ("var", [S, 1], f32), ("rs", [S, Hd], f32), ("xn", [S, Hd], f32),
               ("wf1", [1, Hd], f32), ("wf", [S, Hd], f32), ("h", [S, Hd], b16), ("g", [S, I], b16), ("u", [S, I], b16),
               ("sg", [S, I], b16), ("y", [S, Hd], b16)]
    setup = [f"newtensor({V(shape)})->({T('b5_' + name, dt)})" for name, shape, dt in tensors]
    setup.append(f"normal(var<float32>:0, var<float32>:1, var<int32>:14)->({T('b5_x', b16)}) // author=miaobyte")
    setup.append(f"constant(var<float32>:1)->({T('b5_w', b16)}) // author=miaobyte")
    for name, seed in (("Wg", 15), ("Wu", 16), ("Wd", 17)):
        setup.append(f"normal(var<float32>:0, var<float32>:0.02, var<int32>:{seed})->({T('b5_' + name, b16)}) // author=miaobyte")
    n = lambda name, dt=f32: T("b5_" + name, dt)
    block = [f"todtype({n('x', b16)})->({n('xf')})",
             f"powscalar({n('xf')}, var<float32>:2)->({n('sq')})",
             f"sum({n('sq')}, {V([-1])}, var<bool>:True)->({n('var')})",
             f"divscalar({n('var')}, var<float32>:{Hd})->({n('var')})",
             f"addscalar({n('var')}, var<float32>:1e-06)->({n('var')})",
             f"sqrt({n('var')})->({n('var')})",
             f"rdivscalar(var<float32>:1, {n('var')})->({n('var')})",
             f"broadcastTo({n('var')}, {V([S, Hd])})->({n('rs')})",
             f"mul({n('xf')}, {n('rs')})->({n('xn')})",
             f"todtype({n('w', b16)})->({n('wf1')})",
             f"broadcastTo({n('wf1')}, {V([S, Hd])})->({n('wf')})",
             f"mul({n('wf')}, {n('xn')})->({n('xn')})",
             f"todtype({n('xn')})->({n('h', b16)})",
             f"matmul({n('h', b16)}, {n('Wg', b16)})->({n('g', b16)})",
             f"matmul({n('h', b16)}, {n('Wu', b16)})->({n('u', b16)})",
             f"mulscalar({n('g', b16)}, var<float32>:-1)->({n('sg', b16)})",
             f"exp({n('sg', b16)})->({n('sg', b16)})",
             f"addscalar({n('sg', b16)}, var<float32>:1)->({n('sg', b16)})",
             f"rdivscalar(var<float32>:1, {n('sg', b16)})->({n('sg', b16)})",
             f"mul({n('g', b16)}, {n('sg', b16)})->({n('sg', b16)})",
             f"mul({n('sg', b16)}, {n('u', b16)})->({n('sg', b16)})",
             f"matmul({n('sg', b16)}, {n('Wd', b16)})->({n('y', b16)})"]
    if with_allocations:
        return block_with_its_allocations(setup, block, tensors[5:], lambda name, shape, dt: f"newtensor({V(shape)})->({T('b5_' + name, dt)})",
                                          lambda name, dt: f"deltensor()->({T('b5_' + name, dt)})", iters=iters)
    out = lines_over_ir(setup, block, iters=iters, only=only)
    out["rows"] = S
    return out


def block_with_its_allocations(setup, block, temporaries, new_line, del_line, iters=30):
    """`block` as a front that owns no tensor between passes sends it (front/py/deepx/nn/functional/leaffunc.py:30-38 allocates
    the result of every op right before the op; the tensors go when the Python objects do): each temporary is allocated by a
    `newtensor` line right before the first line that writes it and deleted by a `deltensor` line after the last line of the
    pass.  Wall time per pass with tensor storage from the pool of freed blocks (the default) and from the driver (DEEPX_POOL=0,
    what the reference does), line by line, line by line with runs held back, and as one datagram."""
    import ctypes as C
    from deepx_amd import lib as dx
    L = dx.load()
    E = _executor_lib()
    lines, made = [], set()
    for line in block:
        result = line.split("->(")[1]
        for name, shape, dt in temporaries:
            if name not in made and f":b5_{name})" in result:
                lines.append(new_line(name, shape, dt))
                made.add(name)
        lines.append(line)
    lines += [del_line(name, dt) for name, _, dt in temporaries if name in made]
    lines = [f"{l} // author=miaobyte id={i + 1}" for i, l in enumerate(lines)]
    text = "\n".join(lines).encode()
    out = {"lines": len(lines), "allocations": len(made)}
    for label, pool, defer, batched in (("line_by_line_us", 1, 0, 0), ("line_by_line_storage_from_the_driver_us", 0, 0, 0),
                                        ("line_by_line_deferred_us", 1, 1, 0), ("one_batch_fused_us", 1, 0, 1),
                                        ("one_batch_fused_storage_from_the_driver_us", 0, 0, 1)):
        E.dxe_set_pool(pool)
        try:
            ex = E.dxe_create()
            buf = C.create_string_buffer(1 << 16)
            for line in setup:
                if any(line.startswith("newtensor(") and f":b5_{name})" in line for name in made):
                    continue  # the pass allocates these itself
                E.dxe_execute(ex, line.encode(), buf, len(buf))
                if " ok" not in buf.value.decode().split("//")[0]:
                    raise RuntimeError(f"{line}: {buf.value.decode()}")
            E.dxe_set_defer(ex, defer)

            def once():
                if batched:
                    E.dxe_execute_batch(ex, text, buf, len(buf))
                else:
                    for l in lines:
                        E.dxe_execute(ex, l.encode(), buf, len(buf))
                if any(" ok" not in r.split("//")[0] for r in buf.value.decode().split("\n")):
                    raise RuntimeError("block failed: " + buf.value.decode())

            n = iters if pool else max(5, iters // 3)
            for _ in range(3):
                once()
            E.dxe_flush(ex)
            dx.check(L.dxh_device_sync())
            t0 = time.perf_counter()
            for _ in range(n):
                once()
            E.dxe_flush(ex)
            dx.check(L.dxh_device_sync())
            out[label] = round((time.perf_counter() - t0) / n * 1e6, 1)
            E.dxe_destroy(ex)
        finally:
            E.dxe_set_pool(1)
    return out


def vendor_gemm_tflops(torch, A, B, C, reps=20, warm=5):
    """torch.matmul (hipBLASLt / rocBLAS) on the same operands, for context next to our kernel's rate.
    Timed with torch's own events on torch's current stream, which is where torch launches it."""
    t0 = time.perf_counter()
    while True:
        for _ in range(warm):
            torch.matmul(A, B, out=C)
        torch.cuda.synchronize()
        if (time.perf_counter() - t0) * 1e3 >= RAMP_MS:
            break
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        torch.matmul(A, B, out=C)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    return round(2.0 * A.shape[0] * A.shape[1] * B.shape[1] / ms / 1e9, 2)


def cpu_baseline(np, dx):
    """The oracle's restatement of op-ompsimd's reduce (one callback per input element, index
    vector, atomic accumulate) on this host's cores, on the same step."""
    from tests import helpers as H
    orc = H.oracle()
    cores = orc.orc_num_threads()
    rows = 8192
    rng = np.random.default_rng(3)
    X = rng.standard_normal((rows, 8192), dtype=np.float32)
    P = np.random.default_rng(4).uniform(0.9, 1.1, (8192, 64)).astype(np.float32)
    out = np.empty(8192, dtype=np.float32)
    shX, shP = dx.i32arr([rows, 8192]), dx.i32arr([8192, 64])
    plan = [(0, X, shX, [1]), (0, X, shX, [0]), (2, X, shX, [1]), (3, X, shX, [1]), (1, P, shP, [1])]
    # one untimed pass to fault the pages in, then 5 timed passes of the 5 distinct ops x 2 keepdims; median
    for op, arr, sh, ax in plan:
        orc.orc_faithful_reduce_f32(op, H.hp(arr), sh, 2, dx.i32arr(ax), 1, 0, H.hp(out))
    times = []
    for _ in range(5):
        nbytes = 0
        t0 = time.perf_counter()
        for kd in (1, 0):
            for op, arr, sh, ax in plan:
                assert orc.orc_faithful_reduce_f32(op, H.hp(arr), sh, 2, dx.i32arr(ax), 1, kd, H.hp(out)) == 0
                nbytes += arr.nbytes + 8192 * 4
        times.append(time.perf_counter() - t0)
    dt = sorted(times)[len(times) // 2]
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for ln in f:
                if ln.startswith("model name"):
                    model = ln.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"value": round(nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"full config-2 step (10 ops, {nbytes} bytes), median of 5 timed passes after 1 warm-up: {dt:.2f} s; OMP threads={cores}; cpu='{model}'; -O2, AVX2 auto-vectorisation"}


def cpu_per_op(np, dx):
    """The other configs' ops through the oracle's restatement of op-ompsimd on this host's cores:
    chunked elementwise loops (shape_range.cpp:116-135), the per-element index-vector gathers of
    transpose / broadcastTo / indexselect and the run-wise concat (changeshape_miaobyte.hpp:45-178),
    the per-element reduce (reduce_miaobyte.hpp:30-44).  The reference multiplies through OpenBLAS
    cblas_sgemm (matmul_cblas.hpp:51-57), which this image does not have: torch.matmul on CPU
    tensors stands in for it, in the reference's dtypes (fp32 / fp64; op-ompsimd has no 16-bit
    floats, so the bf16 entries carry the fp32 figure).  Every op at its full BASELINE size, one
    untimed call, then the median of three.  Returns {config: {op label: {cpu_ms, cores, cpu_kind}}}."""
    import ctypes as C
    from tests import helpers as H
    orc = H.oracle()
    hp = H.hp
    cores = orc.orc_num_threads()

    def med(fn, reps=3):
        fn()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            rc = fn()
            ts.append(time.perf_counter() - t0)
            assert rc in (0, None), rc
        return {"cpu_ms": round(sorted(ts)[len(ts) // 2] * 1e3, 3), "cores": cores, "cpu_kind": "port"}

    out = {}
    rng = np.random.default_rng(21)
    # config 1
    n = 4096 * 4096
    a = rng.uniform(-1, 1, n).astype(np.float32)
    b = rng.uniform(-1, 1, n).astype(np.float32)
    c = np.empty(n, dtype=np.float32)
    half = dx.scalar(0.5)
    out["config1"] = {
        "add": med(lambda: orc.orc_add(dx.F32, hp(a), hp(b), hp(c), n)),
        "mul": med(lambda: orc.orc_mul(dx.F32, hp(a), hp(b), hp(c), n)),
        "max": med(lambda: orc.orc_max(dx.F32, hp(a), hp(b), hp(c), n)),
        "div": med(lambda: orc.orc_div(dx.F32, hp(a), hp(b), hp(c), n)),
        "addscalar": med(lambda: orc.orc_addscalar(dx.F32, hp(a), half, hp(c), n)),
        "mulscalar": med(lambda: orc.orc_mulscalar(dx.F32, hp(a), half, hp(c), n)),
        "exp": med(lambda: orc.orc_exp(dx.F32, hp(a), hp(c), n)),
    }
    del a, b, c
    # config 3 (16-bit tensors move as raw bits)
    shape = [32, 2048, 14, 64]
    nt = 32 * 2048 * 14 * 64
    t = rng.integers(0, 65536, nt, dtype=np.uint16)
    to = np.empty(nt, dtype=np.uint16)
    c3 = {"transpose_bf16_32x2048x14x64_0213": med(lambda: orc.orc_faithful_transpose(dx.BF16, hp(t), dx.i32arr(shape), 4, dx.i32arr([0, 2, 1, 3]), hp(to)))}
    del t, to
    nc = 16 * 1024 * 4096
    cs = [rng.integers(0, 65536, nc, dtype=np.uint16) for _ in range(3)]
    co = np.empty(3 * nc, dtype=np.uint16)
    ins = dx.ptrarr([x.ctypes.data for x in cs])
    c3["concat_fp16_3x16x1024x4096_axis1"] = med(lambda: orc.orc_faithful_concat(dx.F16, ins, 3, dx.i32arr([1024] * 3), dx.i32arr([16, 3072, 4096]), 3, 1, hp(co)))
    del cs, co
    r = rng.integers(0, 65536, 4096, dtype=np.uint16)
    bo = np.empty(8192 * 4096, dtype=np.uint16)
    c3["broadcastTo_bf16_1x4096_to_8192x4096"] = med(lambda: orc.orc_faithful_broadcastTo(dx.BF16, hp(r), dx.i32arr([1, 4096]), 2, dx.i32arr([8192, 4096]), 2, hp(bo)))
    del bo
    out["config3"] = c3
    # config 4
    n = 1 << 26
    a = rng.integers(-2 ** 20, 2 ** 20 + 1, n, dtype=np.int32)
    b = rng.integers(-2 ** 20, 2 ** 20 + 1, n, dtype=np.int32)
    o = np.empty(n, dtype=np.int32)
    m = np.empty(n, dtype=np.uint8)
    c4 = {"max_i32_2^26": med(lambda: orc.orc_max(dx.I32, hp(a), hp(b), hp(o), n)),
          "min_i32_2^26": med(lambda: orc.orc_min(dx.I32, hp(a), hp(b), hp(o), n)),
          "greater_i32_2^26": med(lambda: orc.orc_greater(dx.I32, hp(a), hp(b), hp(m), n))}
    sw = dx.ptrarr([b.ctypes.data, a.ctypes.data])
    c4["where_i32_2^26(switch)"] = med(lambda: orc.orc_switch(dx.I32, sw, 2, dx.BOOL, hp(m), hp(o), n))
    del a, b, o, m
    E = rng.integers(0, 65536, 151936 * 896, dtype=np.uint16)
    idx = rng.integers(0, 151936, 4096, dtype=np.int64)
    eo = np.empty(4096 * 896, dtype=np.uint16)
    c4["indexselect_bf16_4096_of_151936x896"] = med(lambda: orc.orc_faithful_indexselect(dx.BF16, hp(E), dx.i32arr([151936, 896]), 2, dx.I64, hp(idx), dx.i32arr([4096]), 1, 0, hp(eo)))
    del E, eo
    out["config4"] = c4
    # config 5: the glue through the oracle (16-bit floats compute in fp32 and round once, op-cuda's
    # convention), the GEMMs through torch on the CPU
    S, Hd, I = 2048, 896, 4864
    n16, n32 = S * I, S * Hd
    g16 = H.f32_to_bf16_bits(rng.standard_normal(n16).astype(np.float32))
    u16 = H.f32_to_bf16_bits(rng.standard_normal(n16).astype(np.float32))
    o16 = np.empty(n16, dtype=np.uint16)
    x16 = H.f32_to_bf16_bits(rng.standard_normal(n32).astype(np.float32))
    x32 = rng.standard_normal(n32).astype(np.float32)
    o32 = np.empty(n32, dtype=np.float32)
    col = np.empty(S, dtype=np.float32)
    one, two, neg = dx.scalar(1.0), dx.scalar(2.0), dx.scalar(-1.0)
    glue = {
        "mulscalar_bf16_2048x4864": med(lambda: orc.orc_mulscalar(dx.BF16, hp(g16), neg, hp(o16), n16)),
        "exp_bf16_2048x4864": med(lambda: orc.orc_exp(dx.BF16, hp(g16), hp(o16), n16)),
        "rdivscalar_bf16_2048x4864": med(lambda: orc.orc_rdivscalar(dx.BF16, one, hp(g16), hp(o16), n16)),
        "mul_bf16_2048x4864": med(lambda: orc.orc_mul(dx.BF16, hp(g16), hp(u16), hp(o16), n16)),
        "todtype_bf16_to_f32_2048x896": med(lambda: orc.orc_todtype(dx.BF16, hp(x16), dx.F32, hp(o32), n32)),
        "powscalar_f32_2048x896": med(lambda: orc.orc_powscalar(dx.F32, hp(x32), two, hp(o32), n32)),
        "sum_f32_2048x896_axis1_keepdims": med(lambda: orc.orc_faithful_reduce_f32(0, hp(x32), dx.i32arr([S, Hd]), 2, dx.i32arr([1]), 1, 1, hp(col))),
        "broadcastTo_f32_2048x1_to_2048x896": med(lambda: orc.orc_faithful_broadcastTo(dx.F32, hp(col), dx.i32arr([S, 1]), 2, dx.i32arr([S, Hd]), 2, hp(o32))),
    }
    c5 = {"glue_ops(cache-resident sizes)": glue}
    import torch
    threads = torch.get_num_threads()
    for mm, kk, nn in ((2048, 896, 4864), (2048, 4864, 896)):
        for dt, tdt in (("f32", torch.float32), ("f64", torch.float64)):
            A = torch.randn(mm, kk, dtype=tdt)
            B = torch.randn(kk, nn, dtype=tdt) * 0.02
            Cm = torch.empty(mm, nn, dtype=tdt)
            e = med(lambda: (torch.matmul(A, B, out=Cm), None)[1])
            e.update({"cores": threads, "cpu_kind": f"torch.matmul on CPU {dt} tensors, standing in for OpenBLAS cblas_{'s' if dt == 'f32' else 'd'}gemm (not in this image)"})
            c5[f"matmul_{dt}_{mm}x{kk}x{nn}"] = e
            if dt == "f32":
                c5[f"matmul_bf16_{mm}x{kk}x{nn}"] = dict(e, cpu_dtype="f32 (op-ompsimd has no 16-bit floats)")
    out["config5"] = c5
    return out


def merge_cpu_per_op(per_op, cpu):
    """cpu_ms / cores / cpu_kind of cpu_per_op() into the per_op entries of the same label (labels may
    carry a remark in parentheses after the CPU leg's label)."""
    for cfg, ops in cpu.items():
        dst = per_op.get(cfg)
        if not isinstance(dst, dict):
            continue
        for label, fig in ops.items():
            if "cpu_ms" not in fig:  # a group of ops (the glue table)
                merge_cpu_per_op(dst, {label: fig})
                continue
            for k, entry in dst.items():
                if isinstance(entry, dict) and (k == label or k.startswith(label + "(")):
                    entry.update(fig)
                    if "ms" in entry and entry["ms"] > 0:
                        entry["gpu_over_cpu"] = round(fig["cpu_ms"] / entry["ms"], 1)


if __name__ == "__main__":
    main()
