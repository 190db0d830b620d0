"""BERT-base (batch 64 x 128, bf16) and YOLOv3 (batch 16 @ 416, fp16) at their benchmark
sizes, where the CPU oracle cannot follow the whole batch in test time: properties that
do not depend on the batch size for all of it, the first samples against the oracle.

  * samples of a batch do not influence each other: reversing the batch reverses the
    outputs bit for bit;
  * outputs are finite; YOLOv3 detections are well formed (valid indices, -1 padding
    only behind the selected rows) and, for all 16 images, identical to the oracle's
    selection rule applied to the boxes and scores the GPU decoded;
  * the first image's YOLOv3 heads agree with the fp32 oracle within 2e-2 absolute; the
    first eight BERT sequences, in both bf16 modes, within what the oracle's precision
    emulation shows the storage type to cost (see the comment above BERT_STATED_TOL); the
    measured differences are printed.
"""
import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, err_stats, run_hip, run_ref, run_ref_emulated

pytestmark = pytest.mark.gpu

# BERT-base in bf16.  The stated bound is 2e-2 absolute on the final hidden states (LayerNorm
# outputs of magnitude up to 5.2) against the fp32 oracle.  What the storage type itself costs is
# measured by the oracle's precision-emulating modes on the same inputs, and printed:
#   * "operands" (the reference's BF16_ACCURACY_MODE: only Conv / Gemm operands are rounded to
#     bf16): the floor of any matrix-unit implementation.  Over the first 8 sequences its largest
#     difference from fp32 is 2.2e-2 - already above the stated bound - with 99.9 % of the values
#     within 1.5e-2 and a mean of 3.5e-3.
#   * "stored" (every tensor bf16, BF16_PERFORMACE_MODE): 8.1e-2 / 4.7e-2 / 9.0e-3.
# A 12-layer network amplifies single rounding decisions (a value that sits on a bf16 rounding
# boundary flips with the summation order), so two correct implementations of one scheme differ
# from each other by about as much as each differs from fp32; what pins the GPU is therefore
# (a) its error statistics against fp32 within 1.25 x the emulated floor's - an implementation
# that loses twice the unavoidable precision fails - (b) its distance from the emulated oracle
# no larger than the floor, and (c) bit-level agreement after ONE encoder layer, where no such
# amplification has happened yet (test_bert_one_layer_bf16_vs_emulated).
BERT_STATED_TOL = 2e-2
FLOOR_SLACK = 1.25
YOLO_FP16_ABS_TOL = 2e-2


def _report(tag, st):
    announce("%-58s max %.3e  p99.9 %.3e  mean %.3e" % (tag, st[0], st[1], st[2]))


def test_bert_base_bf16_batch64():
    mb = entry.load().models_bert
    batch, seq, n_oracle = 64, 128, 8
    w = mb.bert_weights()
    feeds = mb.bert_input(batch, seq)
    feeds["attention_mask"][::3, 0, 0, 100:] = 0.0   # every third sequence is padded
    build = lambda b: mb.build_bert(b, w, batch, seq)
    got = {}
    for mode in ("accuracy", "performance"):
        announce("bert-base bf16 (%s mode) 64 x 128" % mode)
        got[mode] = run_hip(build, feeds, bf16=mode)["hidden"]
        assert got[mode].shape == (batch, seq, 768) and np.all(np.isfinite(got[mode]))
        announce("bert-base bf16 (%s mode), reversed batch" % mode)
        rev = run_hip(build, {k: np.ascontiguousarray(v[::-1]) for k, v in feeds.items()}, bf16=mode)["hidden"]
        assert np.array_equal(rev[::-1], got[mode])

    announce("bert-base oracle (fp32, operands-emulated, stored-emulated), %d sequences" % n_oracle)
    sub = {k: np.ascontiguousarray(v[:n_oracle]) for k, v in feeds.items()}
    build_n = lambda b: mb.build_bert(b, w, n_oracle, seq)
    want = run_ref(build_n, sub)["hidden"]
    emu_op = run_ref_emulated(build_n, sub, "operands", "bf16")["hidden"]
    emu_st = run_ref_emulated(build_n, sub, "stored", "bf16")["hidden"]
    acc, perf = got["accuracy"][:n_oracle], got["performance"][:n_oracle]
    floor_op, floor_st = err_stats(emu_op, want), err_stats(emu_st, want)
    e_acc, e_perf = err_stats(acc, want), err_stats(perf, want)
    d_acc, d_perf = err_stats(acc, emu_op), err_stats(perf, emu_st)
    announce("largest |hidden| = %.3f" % np.max(np.abs(want)))
    _report("floor, operands-emulated oracle vs fp32 oracle", floor_op)
    _report("GPU accuracy mode vs fp32 oracle", e_acc)
    _report("GPU accuracy mode vs operands-emulated oracle", d_acc)
    _report("floor, stored-emulated oracle vs fp32 oracle", floor_st)
    _report("GPU performance mode vs fp32 oracle", e_perf)
    _report("GPU performance mode vs stored-emulated oracle", d_perf)

    # accuracy mode: the stated bound wherever the floor allows it, the floor (with a little
    # room) where it does not
    assert e_acc[0] <= max(BERT_STATED_TOL, FLOOR_SLACK * floor_op[0])
    assert e_acc[1] <= BERT_STATED_TOL
    assert e_acc[2] <= FLOOR_SLACK * floor_op[2]
    assert d_acc[0] <= floor_op[0] and d_acc[2] <= floor_op[2]
    # performance mode: nothing beyond what bf16 storage of every tensor costs
    for k in range(3):
        assert e_perf[k] <= FLOOR_SLACK * floor_st[k], k
    assert d_perf[0] <= FLOOR_SLACK * floor_st[0] and d_perf[2] <= floor_st[2]


def test_bert_one_layer_bf16_vs_emulated():
    """One full-width encoder layer (embedding + LayerNorm, attention, feed-forward): here the
    GPU and the precision-emulating oracle round the same values, and they agree to about one
    unit of the last place of what they store.  (The stated 2e-2 against fp32 holds here in
    accuracy mode; in performance mode the bf16 rounding of the result itself, magnitude up to
    5, already costs up to 1.6e-2.)"""
    mb = entry.load().models_bert
    cfg = dict(mb.BERT_BASE, layers=1)
    batch, seq = 8, 128
    w = mb.bert_weights(cfg)
    feeds = mb.bert_input(batch, seq, cfg)
    feeds["attention_mask"][::3, 0, 0, 100:] = 0.0
    build = lambda b: mb.build_bert(b, w, batch, seq, cfg)
    want = run_ref(build, feeds)["hidden"]
    for mode, emu in (("accuracy", "operands"), ("performance", "stored")):
        announce("bert one layer, bf16 %s mode" % mode)
        got = run_hip(build, feeds, bf16=mode)["hidden"]
        exp = run_ref_emulated(build, feeds, emu, "bf16")["hidden"]
        floor, e, d = err_stats(exp, want), err_stats(got, want), err_stats(got, exp)
        _report("one layer, %s-emulated oracle vs fp32 oracle" % emu, floor)
        _report("one layer, GPU %s mode vs fp32 oracle" % mode, e)
        _report("one layer, GPU %s mode vs %s-emulated oracle" % (mode, emu), d)
        for k in range(3):
            assert e[k] <= FLOOR_SLACK * floor[k], k
        if mode == "accuracy":
            assert e[0] <= BERT_STATED_TOL
            # fp32 results: the only differences are operand roundings that fell the other way
            # (measured: largest 2.8e-3, mean 1.2e-4)
            assert d[0] <= 6e-3 and d[2] <= 3e-4
        else:
            # bf16 results of magnitude < 8, where one unit of the last place is 2^-5 at most
            # (measured: largest difference one unit, 2^-6, at magnitude 2 .. 4; mean 4.5e-5)
            assert d[0] <= 2.0 ** -5 and d[2] <= 2e-4
            assert float(np.mean(got == exp)) >= 0.95


def test_yolov3_fp16_batch16():
    announce("yolov3 fp16 batch 16 @ 416: head calibration")
    my = entry.load().models_yolo
    ref = entry.load_oracle()
    batch = 16
    feeds = my.yolov3_input(batch)
    # head logits to unit spread and a bias that lets about 1 % of the scores pass 0.3
    w0 = my.yolov3_weights()
    h = run_hip(lambda b: my.build_yolov3(b, w0, 2, postprocess=False), my.yolov3_input(2), fp16=True)
    scales, bias = my.calibrate_heads([h["head%d" % i] for i in range(3)])
    w = my.yolov3_weights(head_bias=bias, head_scale=scales)

    announce("yolov3 fp16 batch 16 @ 416")
    build = lambda b: my.build_yolov3(b, w, batch, postprocess=False)
    got = run_hip(build, feeds, fp16=True)
    for k, v in got.items():
        assert np.all(np.isfinite(v)), k

    announce("yolov3 fp16, reversed batch")
    rev = run_hip(build, {"input": np.ascontiguousarray(feeds["input"][::-1])}, fp16=True)
    for k in got:
        assert np.array_equal(rev[k][::-1], got[k]), k

    announce("yolov3 fp32 oracle, 1 image")
    want = run_ref(lambda b: my.build_yolov3(b, w, 1, postprocess=False), {"input": feeds["input"][:1]})
    for k in want:
        d = np.abs(got[k][:1] - want[k])
        announce("yolov3 fp16 vs fp32 oracle, %s: max |d| = %.3e, mean = %.3e, largest |value| = %.3f"
                 % (k, d.max(), d.mean(), np.max(np.abs(want[k]))))
        assert d.max() <= YOLO_FP16_ABS_TOL, k

    announce("yolov3 fp16 with decode + NMS")
    full = run_hip(lambda b: my.build_yolov3(b, w, batch), feeds, fp16=True)
    det = full["detections"].reshape(batch, -1, 3)
    for n in range(batch):
        rows = det[n]
        valid = rows[:, 0] >= 0
        k = int(valid.sum())
        assert np.all(valid[:k]) and not np.any(valid[k:])          # -1 padding only at the end
        assert np.all(rows[:k, 0] == n) and np.all(rows[:k, 1] >= 0) and np.all(rows[:k, 1] < my.NUM_CLASSES)
    # The selection itself on bit-identical inputs: the oracle's rule applied to the boxes and
    # scores the GPU decoded must pick the same (image, class, box) rows for all 16 images.
    announce("yolov3: oracle NMS on the GPU's decoded boxes and scores, %d images" % batch)
    want_det = ref.nms(full["boxes"], full["scores"], 100, 0.45, 0.3)
    n_det = int((want_det[:, 2] >= 0).sum())
    passed = float((full["scores"] > 0.3).mean())
    announce("yolov3: %d detections over %d images, %.2f %% of the scores pass 0.3" % (n_det, batch, 100 * passed))
    assert n_det >= batch, "head calibration produced too few detections"
    assert np.array_equal(full["detections"], want_det)
