"""BERT-base (batch 64 x 128, bf16) and YOLOv3 (batch 16 @ 416, fp16) at their benchmark
sizes, where the CPU oracle cannot follow the whole batch in test time: properties that
do not depend on the batch size for all of it, the first samples against the oracle.

  * samples of a batch do not influence each other: reversing the batch reverses the
    outputs bit for bit;
  * outputs are finite; YOLOv3 detections are well formed (valid indices, -1 padding
    only behind the selected rows);
  * the first two sequences / the first image agree with the fp32 oracle within the
    storage type's tolerance.
"""
import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, run_hip, run_ref

pytestmark = pytest.mark.gpu


def test_bert_base_bf16_batch64():
    announce("bert-base bf16 64 x 128")
    mb = entry.load().models_bert
    batch, seq, n_oracle = 64, 128, 2
    w = mb.bert_weights()
    feeds = mb.bert_input(batch, seq)
    feeds["attention_mask"][::3, 0, 0, 100:] = 0.0   # every third sequence is padded
    build = lambda b: mb.build_bert(b, w, batch, seq)
    got = run_hip(build, feeds, bf16=True)["hidden"]
    assert got.shape == (batch, seq, 768) and np.all(np.isfinite(got))

    announce("bert-base bf16, reversed batch")
    rev = run_hip(build, {k: np.ascontiguousarray(v[::-1]) for k, v in feeds.items()}, bf16=True)["hidden"]
    assert np.array_equal(rev[::-1], got)

    announce("bert-base fp32 oracle, %d sequences" % n_oracle)
    sub = {k: np.ascontiguousarray(v[:n_oracle]) for k, v in feeds.items()}
    want = run_ref(lambda b: mb.build_bert(b, w, n_oracle, seq), sub)["hidden"]
    # twelve layers of bf16 storage (8 significant bits) on O(1) LayerNorm outputs
    assert np.max(np.abs(got[:n_oracle] - want)) <= 6e-2 * max(1.0, float(np.max(np.abs(want))))
    assert float(np.mean(np.abs(got[:n_oracle] - want))) <= 1e-2


def test_yolov3_fp16_batch16():
    announce("yolov3 fp16 batch 16 @ 416")
    my = entry.load().models_yolo
    batch = 16
    w = my.yolov3_weights()
    feeds = my.yolov3_input(batch)
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
        scale = max(1.0, float(np.max(np.abs(want[k]))))
        assert np.max(np.abs(got[k][:1] - want[k])) <= 3e-2 * scale, k

    announce("yolov3 fp16 with decode + NMS")
    full = run_hip(lambda b: my.build_yolov3(b, w, batch), feeds, fp16=True)
    det = full["detections"].reshape(batch, -1, 3)
    for n in range(batch):
        rows = det[n]
        valid = rows[:, 0] >= 0
        k = int(valid.sum())
        assert np.all(valid[:k]) and not np.any(valid[k:])          # -1 padding only at the end
        assert np.all(rows[:k, 0] == n) and np.all(rows[:k, 1] >= 0) and np.all(rows[:k, 1] < my.NUM_CLASSES)
