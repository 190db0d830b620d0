#!/usr/bin/env python3
"""Throughput benchmark of the ODLA hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload resnet50_fp16|resnet50_int8|resnet50_fp32]
                  [--batch 256] [--cpu-sample N]

A step is one odla_ExecuteComputation of the whole graph on one batch of
synthetic input that is already resident in device memory (arguments and
outputs are bound to buffers from odla_AllocateDeviceMemory).  Prints ONE JSON
line with images/s, the roofline of the dominant kernel class (the
implicit-GEMM convolutions, measured live with HIP events around un-captured
launches on the library's stream) and the CPU oracle timed on a bounded sample.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

PEAK = {"fp16": 2500.0, "bf16": 2500.0, "int8": 5000.0, "fp32": 157.3}  # dense MFMA TFLOP/s (TOP/s)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="resnet50_fp16")
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--cpu-sample", type=int, default=4, help="images timed on the CPU oracle (0 = skip)")
    ap.add_argument("--dump-steps", default=None, help="write the per-launch timing table to this file")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this build has a single MI355X and the path "
              "shards by batch without any collective; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    pkg = entry.load()
    odla, models = pkg.odla, pkg.models
    L = odla.load_library()
    mode = args.workload.split("_")[1]
    if mode not in ("fp16", "fp32", "bf16", "int8"):
        print("unknown workload %s" % args.workload, file=sys.stderr)
        sys.exit(2)

    batch = args.batch
    w = models.resnet50_weights()
    feeds = models.resnet50_input(batch)
    table = None
    if mode == "int8":
        table = odla.quant_table(models.resnet50_quant_entries(w, calibrate_on_gpu(odla, models, w)))
    hb = odla.HipBuilder(fp16=(mode == "fp16"), bf16=(mode == "bf16"), quant_table=table)
    models.build_resnet50(hb, w, batch)
    sess = hb.session(use_graph=True)
    sess.bind_device_io(feeds)

    for _ in range(args.warmup):
        sess.execute()
    # odla_ExecuteComputation returns after the device is idle, so the wall
    # clock around K executions is the device-synchronised time of K steps.
    t0 = time.perf_counter()
    for _ in range(args.steps):
        sess.execute()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    images_per_s = batch / (ms_per_step * 1e-3)

    # Roofline of the convolution kernels: all conv + FC launches of one step,
    # timed with HIP events on the library's own stream (library entry point
    # odla_hip_ProfileSteps), algorithmic FLOPs = 2 * MACs of the layers.
    roof = None
    if hasattr(L, "odla_hip_ProfileSteps"):
        roof = profile_roofline(L, sess, hb, mode, batch, models, args.dump_steps)

    cpu = None
    if args.cpu_sample > 0:
        cpu = cpu_baseline(models, w, args.cpu_sample)

    line = {
        "metric": "images/sec at batch 256, ResNet-50 int8 & fp16; % MFMA peak / % HBM BW",
        "value": round(images_per_s, 1), "unit": "images/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": {"fp16": "f16", "bf16": "bf16", "fp32": "f32", "int8": "i8"}[mode],
        "data": "synthetic",
        "config": {"workload": "ResNet-50 v1.5 %s NCHW [%d,3,224,224], folded BN, random He-normal weights, "
                               "softmax head; inputs/outputs resident in HBM" % (mode, batch),
                   "batch": batch, "executor": "hipGraph replay through odla_ExecuteComputation"},
        "roofline": roof, "cpu_baseline": cpu,
    }
    print(json.dumps(line))
    sess.close()
    hb.destroy()


def calibrate_on_gpu(odla, models, w, batch=4, n_batches=8):
    """Activation ranges for the int8 plan: min/max of every named activation of
    the fp32 graph over 32 seeded N(0,1) images (8 batches of 4), computed by the
    fp32 plan of the library itself."""
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


def profile_roofline(L, sess, hb, mode, batch, models, dump_path=None):
    class StepTime(ctypes.Structure):
        _fields_ = [("name", ctypes.c_char * 64), ("ms", ctypes.c_float)]

    L.odla_hip_ProfileSteps.restype = ctypes.c_int32
    L.odla_hip_ProfileSteps.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(StepTime), ctypes.c_int32,
                                        ctypes.POINTER(ctypes.c_int32)]
    cap = 1024
    buf = (StepTime * cap)()
    n = ctypes.c_int32(0)
    st = L.odla_hip_ProfileSteps(sess.ctx, 10, buf, cap, ctypes.byref(n))
    if st != 0:
        return None
    if dump_path:
        with open(dump_path, "w") as f:
            for i in range(n.value):
                f.write("%-40s %9.4f ms\n" % (buf[i].name.decode(), buf[i].ms))
    conv_ms = 0.0
    total_ms = 0.0
    launches = 0
    for i in range(n.value):
        name = buf[i].name.decode()
        total_ms += buf[i].ms
        if name.startswith("conv") or name.startswith("gemm"):
            conv_ms += buf[i].ms
            launches += 1
    flop = models.RESNET50_GFLOP_PER_IMAGE * 1e9 * batch
    achieved = flop / (conv_ms * 1e-3) / 1e12 if conv_ms > 0 else 0.0
    peak = PEAK[mode]
    return {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
            "frac": round(achieved / peak, 4), "traffic": None,
            "kernel": "igemm_kernel (all %d conv/FC launches of one step)" % launches,
            "conv_ms_per_step": round(conv_ms, 4), "all_kernels_ms_per_step": round(total_ms, 4)}


def cpu_baseline(models, w, sample):
    """The CPU oracle (a port of the reference CPU path's arithmetic) on `sample`
    images of the same workload, all host cores through OpenMP."""
    ref = entry.load_oracle()
    feeds = models.resnet50_input(sample)
    rb = ref.RefBuilder(feeds)
    models.build_resnet50(rb, w, sample)      # warm-up (page in weights, spin up threads)
    t0 = time.perf_counter()
    rb = ref.RefBuilder(feeds)
    models.build_resnet50(rb, w, sample)
    dt = time.perf_counter() - t0
    return {"value": round(sample / dt, 2), "unit": "images/s", "cores": ref.num_threads(), "kind": "port",
            "sample": "%d images of the same ResNet-50 fp32 graph, one pass after one warm-up pass" % sample}


if __name__ == "__main__":
    main()
