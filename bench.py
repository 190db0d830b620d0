#!/usr/bin/env python3
"""Throughput benchmark of the ODLA hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--batch B]
                  [--cpu-sample N] [--dump-steps FILE]

Workloads: resnet50 (default: the configuration the headline metric is quoted
on, "ResNet-50 int8 & fp16 at batch 256" - the int8 plan is timed first and is
the top level of the line, the fp16 plan is timed next in the same process and
nested under "fp16" with its own roofline block; the other benchmark
configurations follow, each nested under its name with its own value,
ms_per_step and roofline: "bert_bf16" (performance mode, with the accuracy mode
under "bert_bf16acc"), "yolov3_fp16", "mnist_fp32"; --headline-only leaves them
out), resnet50_int8, resnet50_fp16, resnet50_bf16, resnet50_fp32, yolov3_fp16,
bert_bf16, bert_bf16acc, mnist_fp32, streaming_fp16.

A step is one odla_ExecuteComputation of the whole graph on one batch of
synthetic input that is already resident in device memory (arguments and
outputs are bound to buffers from odla_AllocateDeviceMemory).  Prints ONE JSON
line with the throughput, the roofline of the dominant kernel class (the
implicit-GEMM convolution / GEMM launches, timed live with HIP events around
un-captured launches on the library's own stream) and the CPU oracle timed on a
bounded sample of the same workload.  Beside that device-resident figure the
line carries an "end_to_end" block: the same step with HOST buffers bound, so
that the copies of the arguments to the device and of the results back are
inside the timed region (what a caller of the reference's harness pays).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

PEAK = {"fp16": 2500.0, "bf16": 2500.0, "bf16acc": 2500.0, "int8": 5000.0, "fp32": 157.3}  # dense MFMA TFLOP/s (TOP/s)
DTYPE = {"fp16": "f16", "bf16": "bf16", "bf16acc": "bf16", "fp32": "f32", "int8": "i8"}
METRIC = "images/sec at batch 256, ResNet-50 int8 & fp16; % MFMA peak / % HBM BW"


def measured_traffic(name):
    """HBM bytes per conv/gemm launch (average over the launches of one step) from the
    rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summaries: the table rows
    `| workload | bytes per launch | ...` of profiles/traffic_per_launch.md.  None when
    the workload has no row (not measured)."""
    path = os.path.join(ROOT, "profiles", "traffic_per_launch.md")
    try:
        with open(path) as f:
            for line in f:
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cells) >= 2 and cells[0] == name:
                    return float(cells[1])
    except (OSError, ValueError):
        pass
    return None


class Workload:
    def __init__(self, name, unit, batch, flop_per_step, desc, build, feeds, ref_run, mode, table=None,
                 conv_elements=None):
        self.name, self.unit, self.batch, self.flop, self.desc = name, unit, batch, flop_per_step, desc
        self.build, self.feeds, self.ref_run, self.mode, self.table = build, feeds, ref_run, mode, table
        self.conv_elements = conv_elements


def make_workload(name, batch, pkg):
    odla, models = pkg.odla, pkg.models
    family, mode = name.rsplit("_", 1)
    if family == "resnet50":
        batch = batch or 256
        w = models.resnet50_weights()
        feeds = models.resnet50_input(batch)
        table = None
        if mode == "int8":
            table = odla.quant_table(models.resnet50_quant_entries(w, calibrate_resnet_on_gpu(odla, models, w)))

        def ref_run(ref, n):
            rb = ref.RefBuilder(models.resnet50_input(n))
            models.build_resnet50(rb, w, n)
        return Workload(name, "images/s", batch, models.RESNET50_GFLOP_PER_IMAGE * 1e9 * batch,
                        "ResNet-50 v1.5 %s NCHW [%d,3,224,224], folded BN, random He-normal weights, softmax head; "
                        "inputs/outputs resident in HBM" % (mode, batch),
                        lambda b: models.build_resnet50(b, w, batch), feeds, ref_run, mode, table,
                        # the stem reads the space-to-depth copy of the image: 16 stored channels per
                        # 2x2 block (12 in fp32), i.e. 4 (3) per source pixel
                        conv_elements=models.resnet50_conv_elements(batch, cin_stored=3 if mode == "fp32" else 4))
    if family == "yolov3":
        my = pkg.models_yolo
        batch = batch or 16
        feeds = my.yolov3_input(batch)
        # head calibration: logits to unit std, bias so that ~1% of the scores pass 0.3
        w0 = my.yolov3_weights()
        hb = odla.HipBuilder(fp16=True)
        my.build_yolov3(hb, w0, 2, postprocess=False)
        s = hb.session()
        h = s.run(my.yolov3_input(2))
        s.close()
        hb.destroy()
        scales, bias = my.calibrate_heads([h["head%d" % i] for i in range(3)])
        w = my.yolov3_weights(head_bias=bias, head_scale=scales)
        macs = sum(co * ci * k * k * (416 // st) ** 2 for co, ci, k, st in yolo_conv_geometry(my))

        def ref_run(ref, n):
            rb = ref.RefBuilder(my.yolov3_input(n))
            my.build_yolov3(rb, w, n)
        return Workload(name, "images/s", batch, 2.0 * macs * batch,
                        "YOLOv3 %s NCHW [%d,3,416,416], Darknet-53 + FPN + 3 heads, sigmoid decode + batched NMS "
                        "(IoU 0.45, score 0.3, 80 classes)" % (mode, batch),
                        lambda b: my.build_yolov3(b, w, batch), feeds, ref_run, mode)
    if family == "bert":
        mb = pkg.models_bert
        batch = batch or 64
        seq = 128
        w = mb.bert_weights()
        feeds = mb.bert_input(batch, seq)

        def ref_run(ref, n):
            rb = ref.RefBuilder(mb.bert_input(n, seq))
            mb.build_bert(rb, w, n, seq)
        return Workload(name, "sequences/s", batch, mb.bert_gflop_per_sequence(seq) * 1e9 * batch,
                        "BERT-base encoder %s, batch %d x seq %d, 12 layers, hidden 768, 12 heads, FFN 3072"
                        % ({"bf16": "bf16 (BF16_PERFORMACE_MODE: every tensor bf16)",
                            "bf16acc": "bf16 (BF16_ACCURACY_MODE: fp32 tensors, bf16 Gemm operands)"}.get(mode, mode), batch, seq),
                        lambda b: mb.build_bert(b, w, batch, seq), feeds, ref_run, mode)
    if family == "mnist":
        batch = batch or 64
        w = models.mnist_weights()
        feeds = models.mnist_input(batch)

        def ref_run(ref, n):
            rb = ref.RefBuilder(models.mnist_input(n))
            models.build_mnist(rb, w, n)
        return Workload(name, "images/s", batch, 2.0 * 784 * 10 * batch,
                        "mnist_simple softmax regression fp32, Gemm+Add+Softmax, batch %d" % batch,
                        lambda b: models.build_mnist(b, w, batch), feeds, ref_run, mode)
    raise SystemExit("unknown workload %s" % name)


def yolo_conv_geometry(my):
    """(cout, cin, k, stride of the OUTPUT grid w.r.t. the input image) per convolution at width 1."""
    out = []
    stride = 1
    for name, cout, cin, k, s, act in my.yolov3_conv_specs():
        if name.startswith("d"):
            stride *= s
            out.append((cout, cin, k, stride))
        else:
            hi = int(name[1])
            out.append((cout, cin, k, {1: 32, 2: 16, 3: 8}[hi] * (2 if name.endswith(".lat") else 1)))
    return out


def calibrate_resnet_on_gpu(odla, models, w, batch=4, n_batches=32):
    """Activation ranges for the int8 plan: min/max of every named activation of
    the fp32 graph over 32 seeded N(0,1) batches (seeds 1000 .. 1031, 4 images
    each), computed by the fp32 plan of the library itself."""
    hb = odla.HipBuilder()
    taps = []
    models.build_resnet50(hb, w, batch, taps=taps, with_softmax=False)
    wanted = set(models.resnet50_quantized_values())
    for name, v in taps:
        if name in wanted and name != "input":
            hb.output(v, name)
    sess = hb.session()

    def run_taps(feeds):
        out = sess.run(feeds)
        out["input"] = feeds["input"]
        return out

    ranges = models.calibrate_ranges(run_taps, [models.resnet50_input(batch, seed=1000 + i) for i in range(n_batches)])
    sess.close()
    hb.destroy()
    return ranges


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="resnet50")
    ap.add_argument("--batch", type=int, default=0)
    ap.add_argument("--cpu-sample", type=int, default=-1,
                    help="units (images / sequences) timed on the CPU oracle; 0 = skip, -1 = per-workload default")
    ap.add_argument("--dump-steps", default=None, help="write the per-launch timing table to this file")
    ap.add_argument("--headline-only", action="store_true",
                    help="default workload: time the ResNet-50 int8 / fp16 plans only, not the other configurations")
    ap.add_argument("--e2e-steps", type=int, default=5,
                    help="executions timed with host buffers bound (the end_to_end block); 0 = skip")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this build has a single MI355X and the path "
              "shards by batch without any collective; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    pkg = entry.load()
    odla = pkg.odla
    L = odla.load_library()
    if args.workload.startswith("streaming_"):
        return streaming_bench(pkg, L, args)
    if args.workload == "resnet50":
        # the headline metric names both precisions: int8 (the optimisation target) on top, fp16 nested
        line = run_workload(pkg, L, "resnet50_int8", args, with_cpu=True)
        nested = ("value", "unit", "ms_per_step", "dtype", "config", "roofline", "end_to_end")
        fp16 = run_workload(pkg, L, "resnet50_fp16", args, with_cpu=False)
        line["fp16"] = {k: fp16[k] for k in nested}
        if not args.headline_only:
            for name in ("bert_bf16", "bert_bf16acc", "yolov3_fp16", "mnist_fp32"):
                sub = run_workload(pkg, L, name, args, with_cpu=False)
                line[name] = {k: sub[k] for k in nested}
    else:
        line = run_workload(pkg, L, args.workload, args, with_cpu=True)
    print(json.dumps(line))


def run_workload(pkg, L, name, args, with_cpu):
    """Builds the workload's computation, times args.steps executions after
    args.warmup and returns the fields of the result line."""
    odla = pkg.odla
    wl = make_workload(name, args.batch, pkg)
    mode = wl.mode

    hb = odla.HipBuilder(fp16=(mode == "fp16"), bf16={"bf16": "performance", "bf16acc": "accuracy"}.get(mode, False),
                         quant_table=wl.table)
    wl.build(hb)
    sess = hb.session(use_graph=True)
    sess.bind_device_io(wl.feeds)

    # the library says (at INFO level) when it runs a batch as two half-batch copies side by side
    said = []
    LOGCB = ctypes.CFUNCTYPE(None, ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p)
    cb = LOGCB(lambda f, line, fn_, lvl, msg: said.append(msg.decode(errors="replace")))
    L.odla_SetLogger(ctypes.cast(cb, ctypes.c_void_p))
    L.odla_SetLogLevel(4)
    try:
        # set-up, like the graph capture: the context's first sixteen executions measure whether
        # the batch runs whole (six) or as two half-batch copies (ten) and say which it keeps
        # (nothing to measure when ODLA_HIP_BATCH_SPLIT decides)
        for _ in range(0 if os.environ.get("ODLA_HIP_BATCH_SPLIT") else 16):
            sess.execute()
        for _ in range(args.warmup):
            sess.execute()
    finally:
        L.odla_SetLogLevel(2)
        L.odla_SetLogger(None)
    halves = any("two halves side by side" in m for m in said)
    uncaptured = any("run uncaptured" in m for m in said)
    for m in said:
        if "two halves" in m or "stays whole" in m:
            print("[%s] %s" % (name, m), file=sys.stderr)
    # odla_ExecuteComputation returns after the device is idle, so the wall
    # clock around K executions is the device-synchronised time of K steps.
    t0 = time.perf_counter()
    for _ in range(args.steps):
        sess.execute()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    per_s = wl.batch / (ms_per_step * 1e-3)

    e2e = end_to_end(hb, wl, args.e2e_steps) if args.e2e_steps > 0 else None

    dump = args.dump_steps
    if dump and args.workload == "resnet50":   # two plans in one run: one table each
        dump = "%s.%s" % (dump, name)
    roof = profile_roofline(L, sess, wl, dump)

    cpu = None
    sample = args.cpu_sample
    if sample < 0:
        sample = {"resnet50": 16, "yolov3": 1, "bert": 4, "mnist": 64}[name.rsplit("_", 1)[0]]
    if sample > 0 and with_cpu:
        cpu = cpu_baseline(wl, sample)

    line = {
        "metric": METRIC if wl.name.startswith("resnet50") else "%s, %s" % (wl.unit, wl.name),
        "value": round(per_s, 1), "unit": wl.unit, "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": DTYPE[mode], "data": "synthetic",
        "config": {"workload": wl.desc, "batch": wl.batch,
                   "executor": ("direct launches through odla_ExecuteComputation (fewer than six per execution: no hipGraph)"
                                if uncaptured else "hipGraph replay through odla_ExecuteComputation")
                               + (": two half-batch copies of the plan side by side on two streams" if halves else "")},
        "roofline": roof, "cpu_baseline": cpu, "end_to_end": e2e,
    }
    sess.close()
    hb.destroy()
    return line


def end_to_end(hb, wl, steps):
    """The same step with HOST buffers bound: odla_ExecuteComputation copies the arguments to the
    device, runs the graph and copies the results back before it returns
    [ref: python/halo/odla.py:172-175 times exactly that call].  Timed twice: with ordinary
    (pageable) numpy arrays, as the reference harness passes them, and with page-locked buffers
    from odla_AllocateHostMemory."""
    out = {"steps": steps, "unit": wl.unit,
           "host_bytes_per_step": int(sum(v.nbytes for v in wl.feeds.values()))}
    for kind, pinned in (("pageable", False), ("pinned", True)):
        sess = hb.session(use_graph=True)
        outs = sess.bind_host_io(wl.feeds, pinned=pinned)
        out["host_bytes_per_step"] = int(sum(v.nbytes for v in wl.feeds.values()) + sum(o.nbytes for o in outs.values()))
        # untimed: the captures, and the executions in which the context measures whether to
        # run the batch whole (six) or as two half-batch copies (ten)
        for _ in range(1 if os.environ.get("ODLA_HIP_BATCH_SPLIT") else 17):
            sess.execute()
        t0 = time.perf_counter()
        for _ in range(steps):
            sess.execute()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        out[kind] = {"value": round(wl.batch / (ms * 1e-3), 1), "ms_per_step": round(ms, 4)}
        sess.close()
    return out


class StepTime(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 64), ("ms", ctypes.c_float)]


def profile_steps(L, sess, iters=10):
    """[(launch name, mean ms)] of one execution, from odla_hip_ProfileSteps."""
    L.odla_hip_ProfileSteps.restype = ctypes.c_int32
    L.odla_hip_ProfileSteps.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(StepTime), ctypes.c_int32,
                                        ctypes.POINTER(ctypes.c_int32)]
    cap = 4096
    buf = (StepTime * cap)()
    n = ctypes.c_int32(0)
    if L.odla_hip_ProfileSteps(sess.ctx, iters, buf, cap, ctypes.byref(n)) != 0:
        return None
    return [(buf[i].name.decode(), float(buf[i].ms)) for i in range(n.value)]


def streaming_bench(pkg, L, args):
    """HBM roofline of the bandwidth-bound operators (one graph of independent
    branches at the shapes of the benchmark configurations)."""
    odla, ms = pkg.odla, pkg.models_streaming
    mode = args.workload.rsplit("_", 1)[1]
    es = 4 if mode == "fp32" else 2
    hb = odla.HipBuilder(fp16=(mode == "fp16"), bf16=(mode == "bf16"))
    ms.build_streaming(hb)
    sess = hb.session(use_graph=True)
    sess.bind_device_io(ms.streaming_input())
    for _ in range(max(args.warmup, 1)):
        sess.execute()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        sess.execute()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    steps = profile_steps(L, sess, 10) or []
    by_name = {}
    for name, t in steps:
        by_name[name] = by_name.get(name, 0.0) + t
    rows, tot_b, tot_ms = [], 0.0, 0.0
    for name, desc, nbytes in ms.streaming_cases(es):
        t = by_name.get(name)
        if t is None or t <= 0:
            continue
        gbs = nbytes / (t * 1e-3) / 1e9
        rows.append((name, desc, nbytes, t, gbs))
        tot_b += nbytes
        tot_ms += t
    if args.dump_steps:
        with open(args.dump_steps, "w") as f:
            f.write("%-26s %-62s %10s %9s %9s %6s\n" % ("launch", "operator", "MB", "us", "GB/s", "frac"))
            for name, desc, nbytes, t, gbs in rows:
                f.write("%-26s %-62s %10.1f %9.1f %9.0f %6.2f\n" % (name, desc, nbytes / 1e6, t * 1e3, gbs, gbs / 8000.0))
    agg = tot_b / (tot_ms * 1e-3) / 1e9 if tot_ms > 0 else 0.0
    worst = min(rows, key=lambda r: r[4]) if rows else None
    line = {
        "metric": "GB/s, streaming operators (%s)" % mode, "value": round(agg, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": DTYPE[mode], "data": "synthetic",
        "config": {"workload": "bandwidth-bound ODLA operators at benchmark shapes (%d launches priced)" % len(rows)},
        "roofline": {"bound": "hbm", "achieved": round(agg, 1), "peak": 8000.0, "unit": "GB/s",
                     "frac": round(agg / 8000.0, 4), "traffic": None,
                     "kernel": "all streaming launches, algorithmic bytes / summed launch time",
                     "slowest": None if worst is None else {"launch": worst[0], "GB/s": round(worst[4], 1)},
                     "per_op_frac": {r[0]: round(r[4] / 8000.0, 3) for r in rows}},
        "cpu_baseline": None,
    }
    print(json.dumps(line))
    sess.close()
    hb.destroy()


def profile_roofline(L, sess, wl, dump_path=None):
    """All conv / gemm launches of one step, each timed with a HIP event pair on
    the library's stream (odla_hip_ProfileSteps); algorithmic FLOPs = 2 x MACs."""
    class StepTime(ctypes.Structure):
        _fields_ = [("name", ctypes.c_char * 64), ("ms", ctypes.c_float)]

    L.odla_hip_ProfileSteps.restype = ctypes.c_int32
    L.odla_hip_ProfileSteps.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(StepTime), ctypes.c_int32,
                                        ctypes.POINTER(ctypes.c_int32)]
    cap = 4096
    buf = (StepTime * cap)()
    n = ctypes.c_int32(0)
    st = L.odla_hip_ProfileSteps(sess.ctx, 10, buf, cap, ctypes.byref(n))
    if st != 0:
        return None
    if dump_path:
        with open(dump_path, "w") as f:
            for i in range(n.value):
                f.write("%-40s %9.4f ms\n" % (buf[i].name.decode(), buf[i].ms))
    mm_ms = total_ms = 0.0
    launches = 0
    for i in range(n.value):
        name = buf[i].name.decode()
        total_ms += buf[i].ms
        if name.startswith("conv") or name.startswith("gemm"):
            mm_ms += buf[i].ms
            if not name.startswith("gemm.sum"):   # the reduction behind a split-K GEMM belongs to that GEMM
                launches += 1
    achieved = wl.flop / (mm_ms * 1e-3) / 1e12 if mm_ms > 0 else 0.0
    peak = PEAK[wl.mode]
    roof = {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak,
            "unit": "TOP/s" if wl.mode == "int8" else "TFLOP/s",
            "frac": round(achieved / peak, 4), "traffic": measured_traffic(wl.name),
            "kernel": "igemm_wreg_kernel / igemm_kernel / igemm_lean_kernel / igemm_taps_kernel / igemm_stream_q8_kernel / igemm_c3_kernel (all %d conv/gemm launches of one step, avg %.1f us, "
                      "avg %.2f GFLOP per launch)" % (launches, 1e3 * mm_ms / max(launches, 1),
                                                     wl.flop / 1e9 / max(launches, 1)),
            "mm_ms_per_step": round(mm_ms, 4), "all_kernels_ms_per_step": round(total_ms, 4),
            "launches_per_step": n.value}
    if wl.conv_elements is not None:
        # The same launches priced against both rooflines: per launch the bound is
        # max(FLOPs / MFMA peak, algorithmic bytes / 8 TB/s); most 1x1 layers of
        # this network at batch 256 sit on the HBM side.
        es = {"fp32": 4, "fp16": 2, "bf16": 2, "bf16acc": 2, "int8": 1}[wl.mode]
        t_by = {}
        for i in range(n.value):
            name = buf[i].name.decode()
            if name.startswith("conv"):
                key = name.split(":", 1)[1].replace(".relu", "").replace("out", "c3")
                t_by[key] = t_by.get(key, 0.0) + buf[i].ms
        bound_ms = meas_ms = nbytes = 0.0
        hbm_bound = 0
        # a launch that computes a second layer from the first layer's tiles ("a+b") is priced as
        # one launch: the operations and bytes of both, less the second layer's read of its input
        priced = {}
        for key in t_by:
            parts = key.split("+")
            if all(k in wl.conv_elements for k in parts):
                fl = sum(wl.conv_elements[k][0] for k in parts)
                act = sum(wl.conv_elements[k][1] for k in parts) - sum(wl.conv_elements[k][3] for k in parts[1:])
                wt = sum(wl.conv_elements[k][2] for k in parts)
                priced[key] = (fl, act, wt)
        for key, (fl, act, wt) in priced.items():
            by = (act + wt) * es
            t_m, t_h = fl / (peak * 1e12) * 1e3, by / 8e12 * 1e3
            hbm_bound += t_h > t_m
            bound_ms += max(t_m, t_h)
            meas_ms += t_by[key]
            nbytes += by
        if meas_ms > 0:
            roof["hbm"] = {"algorithmic_GB_per_step": round(nbytes / 1e9, 3),
                           "achieved_GBps": round(nbytes / (meas_ms * 1e-3) / 1e9, 1), "peak_GBps": 8000.0,
                           "frac": round(nbytes / (meas_ms * 1e-3) / 8e12, 4),
                           "launches_hbm_bound": int(hbm_bound), "launches_priced": len(priced)}
            roof["frac_of_per_launch_roofline"] = round(bound_ms / meas_ms, 4)
    return roof


def cpu_baseline(wl, sample):
    """The CPU oracle (a port of the reference CPU path's arithmetic, fp32) on
    `sample` units of the same workload, all host cores through OpenMP / BLAS."""
    ref = entry.load_oracle()
    wl.ref_run(ref, sample)      # warm-up (page in weights, spin up threads)
    passes, t0 = 0, time.perf_counter()
    while True:                  # about ten seconds of CPU work, whatever the host's speed
        wl.ref_run(ref, sample)
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= 10.0 or passes >= 64:
            break
    return {"value": round(sample * passes / dt, 2), "unit": wl.unit, "cores": ref.num_threads(), "kind": "port",
            "sample": "%d passes over %d %s of the same graph in fp32 (%.1f s) after one warm-up pass"
                      % (passes, sample, wl.unit.split("/")[0], dt)}


if __name__ == "__main__":
    main()
