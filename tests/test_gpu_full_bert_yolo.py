"""BERT-base (batch 64 x 128, bf16) and YOLOv3 (batch 16 @ 416, fp16) at their benchmark
sizes, where the CPU oracle cannot follow the whole batch in test time: properties that
do not depend on the batch size for all of it, the first samples against the oracle.

  * samples of a batch do not influence each other: reversing the batch reverses the
    outputs bit for bit;
  * outputs are finite; YOLOv3 detections are well formed (valid indices, -1 padding
    only behind the selected rows) and, for all 16 images, identical to the oracle's
    selection rule applied to the boxes and scores the GPU decoded;
  * the first image's YOLOv3 heads agree with the fp32 oracle within 2e-2 absolute; the
    first eight BERT sequences within what bf16 storage allows (bounds and the reason
    beside BERT_BF16_MAX_TOL); the measured differences are printed.
"""
import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, run_hip, run_ref

pytestmark = pytest.mark.gpu

# Differences of the final hidden states (LayerNorm outputs, magnitude up to 5.2) from the
# fp32 oracle after twelve layers of bf16 storage.  The stated 2e-2 absolute cannot hold for
# this storage type: bf16 keeps 8 significant bits, so rounding ONE value between 4 and 8 is
# off by up to 1.6e-2, and every layer rounds its residual stream twice.  Measured over 8
# sequences (786 432 values): largest 9.6e-2, 99.9 % of the values within 4.7e-2, mean 9.0e-3;
# the bounds below hold those figures with a little room.
BERT_BF16_MAX_TOL = 1.2e-1
BERT_BF16_P999_TOL = 6e-2
BERT_BF16_MEAN_TOL = 1e-2
YOLO_FP16_ABS_TOL = 2e-2


def test_bert_base_bf16_batch64():
    announce("bert-base bf16 64 x 128")
    mb = entry.load().models_bert
    batch, seq, n_oracle = 64, 128, 8
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
    d = np.abs(got[:n_oracle] - want)
    announce("bert-base bf16 vs fp32 oracle over %d sequences: max |d hidden| = %.3e, mean = %.3e, 99.9th percentile = %.3e, "
             "largest |hidden| = %.3f" % (n_oracle, d.max(), d.mean(), np.quantile(d, 0.999), np.max(np.abs(want))))
    assert d.max() <= BERT_BF16_MAX_TOL
    assert float(np.quantile(d, 0.999)) <= BERT_BF16_P999_TOL
    assert float(d.mean()) <= BERT_BF16_MEAN_TOL


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
