"""Calibration on the GPU: the library's profiler mode (reference-named control
functions StartProfiling .. StopProfiling) against ranges computed from the
CPU oracle's activations, and the int8 plan built from the table it yields.
"""
import ctypes
import json
import os
import sys

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, run_hip

pytestmark = pytest.mark.gpu

sys.path.insert(0, os.path.join(entry.ROOT, "oracle"))

SMALL_STAGES = [(16, 2, 1), (32, 2, 2)]


def rng(seed):
    return np.random.default_rng(seed)


def test_profile_small_resnet_and_quantize(pkg, odla, models, ref, tmp_path):
    announce("calibration: small resnet, 4 runs")
    import resnet_q8_ref
    cal = pkg.calibration
    batch, hw, stem, classes = 4, 64, 16, 50
    w = models.resnet50_weights(seed=11, num_classes=classes, stages=SMALL_STAGES, stem=stem)
    for k in w:
        if k.endswith(".b") and k != "fc.b":
            w[k] = (rng(len(k)).standard_normal(w[k].shape) * 0.1).astype(np.float32)
    batches = [models.resnet50_input(batch, hw, seed=1000 + i) for i in range(4)]
    prof_path = str(tmp_path / "model.prof")

    with cal.Profiler(prof_path, channel_axis=1) as p:
        hb = odla.HipBuilder(fp16=True)   # the storage type asked for is ignored while profiling
        try:
            models.build_resnet50(hb, w, batch, hw, SMALL_STAGES, stem, classes)
            s = hb.session()
            try:
                for i, feeds in enumerate(batches):
                    with p.run("batch%d" % i):
                        s.run(feeds)
                s.run(batches[0])   # outside a run: not recorded
            finally:
                s.close()
        finally:
            hb.destroy()

    prof = cal.load_profile(prof_path)
    assert sorted(prof["ProfilingResults"]) == ["batch%d" % i for i in range(4)]
    merged = cal.consolidate(prof)

    # ranges of the fp32 oracle over the same batches
    def taps_of(feeds):
        rb = ref.RefBuilder(feeds)
        taps = []
        models.build_resnet50(rb, w, batch, hw, SMALL_STAGES, stem, classes, taps=taps)
        return dict(taps)

    ranges = models.calibrate_ranges(taps_of, batches)
    for name, (mn, mx) in ranges.items():
        rec = merged[name]
        scale = max(abs(mn), abs(mx), 1e-6)
        assert abs(rec["min_value"] - mn) <= 1e-4 * scale and abs(rec["max_value"] - mx) <= 1e-4 * scale, name
    # records carry the operator, the shape and the operands
    assert merged["stem"]["op_type"] == "odla_Conv" and merged["stem"]["shape"] == [batch, stem, hw // 2, hw // 2]
    assert merged["pool1"]["op_type"] == "odla_MaxPool" and merged["input"]["op_type"] == "odla_CreateArgument"
    assert prof["NetworkInfo"]["l1b0add"]["inputs"] == ["l1b0c3", "l1b0ds"]
    # per-channel ranges: activations along axis 1, kernels along their output channels (exact: same fp32 data)
    act = taps_of(batches[0])["l1b0out"]
    first = prof["ProfilingResults"]["batch0"]["l1b0out"]
    assert first["channels"] == act.shape[1]
    assert np.allclose(first["channels_max"], act.max(axis=(0, 2, 3)), rtol=0, atol=1e-4 * float(act.max()))
    for name, cout, cin, k, _, _ in models.resnet50_conv_specs(SMALL_STAGES, stem):
        rec, wt = merged[name + ".w"], w[name + ".w"].reshape(cout, -1)
        assert rec["op_type"] == "odla_CreateConstant" and rec["channels"] == cout
        # nine significant digits identify an fp32 value
        assert np.array_equal(np.array(rec["channels_min"], np.float32), wt.min(axis=1))
        assert np.array_equal(np.array(rec["channels_max"], np.float32), wt.max(axis=1))

    announce("calibration: int8 plan from the measured table")
    wanted = set(models.resnet50_quantized_values(SMALL_STAGES)) | {n + ".w" for n, *_ in models.resnet50_conv_specs(SMALL_STAGES, stem)}
    entries = [e for e in cal.table_entries(merged) if e[0] in wanted]
    assert len(entries) == len(wanted)
    qp = {e[0]: (np.float32(e[1]), e[2]) for e in entries if not e[0].endswith(".w")}
    feeds = models.resnet50_input(batch, hw, seed=1234)
    record = {}
    want = resnet_q8_ref.run(w, feeds, qp, SMALL_STAGES, stem, batch, hw, record)
    tap_names = [n for n in models.resnet50_quantized_values(SMALL_STAGES) if not n.endswith("c3") and n != "input"]

    def build(b):
        taps = []
        models.build_resnet50(b, w, batch, hw, SMALL_STAGES, stem, classes, taps=taps)
        d = dict(taps)
        for n in tap_names:
            b.output(d[n], n)

    got = run_hip(build, feeds, quant_table=odla.quant_table(entries))
    for n in tap_names:
        assert np.array_equal(got[n], ref.dequantize_act(record[n], *qp[n])), n
    assert np.array_equal(np.argmax(got["logits"], 1), np.argmax(want["logits"], 1))

    # the C table of the reference's driver
    n = cal.write_c_table(entries, str(tmp_path / "model.c"))
    text = open(str(tmp_path / "model.c")).read()
    assert "const int quant_infos_size = %d;" % n in text and text.count(".value_id") == n


def test_profile_interpret_mode(pkg, odla, tmp_path):
    """The reference's profiling flow: values with data, operators one by one."""
    announce("calibration: interpret mode")
    cal = pkg.calibration
    L = odla.load_library()
    path = str(tmp_path / "interp.prof")
    x = rng(5).standard_normal((2, 3, 4, 4)).astype(np.float32)
    with cal.Profiler(path) as p:
        comp = ctypes.c_void_p()
        assert L.odla_CreateComputation(ctypes.byref(comp)) == 0
        try:
            with p.run("only"):
                vx = L.odla_CreateValue(odla.make_type(np.float32, x.shape), b"x")
                assert L.odla_SetValueData(vx, x.ctypes.data_as(ctypes.c_void_p)) == 0
                y = L.odla_Relu(vx, b"y")
                z = L.odla_Neg(y, b"z")
                out = np.empty_like(x)
                assert L.odla_GetValueData(z, out.ctypes.data_as(ctypes.c_void_p), None) == 0
        finally:
            L.odla_DestroyComputation(comp)
    assert np.array_equal(out, -np.maximum(x, 0))
    run = json.load(open(path))["ProfilingResults"]["only"]
    assert run["x"]["op_type"] == "odla_SetValueData" and run["y"]["op_type"] == "odla_Relu"
    assert np.float32(run["x"]["min_value"]) == x.min() and np.float32(run["x"]["max_value"]) == x.max()
    assert run["y"]["min_value"] == 0.0 and np.float32(run["z"]["min_value"]) == -x.max()
    assert run["z"]["channels"] == 0 and run["z"]["channels_min"] == []
