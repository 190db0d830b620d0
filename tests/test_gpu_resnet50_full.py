"""Full-size ResNet-50 v1.5 at the benchmark batch (256 x 3 x 224 x 224), where
the CPU oracle cannot follow in test time.  The whole batch is checked through
properties that do not depend on its size, and a few images of it against the
oracle:

  * fp16: probabilities are finite and sum to 1; the images of the batch do not
    influence each other (reversing the batch reverses the outputs bit for bit);
    the first images agree with the fp32 oracle within the fp16 tolerance (2e-2
    of the largest logit) with the same top-1 class.
  * int8: the first images of the batch-256 run equal, bit for bit, the same
    images run at batch 4, and those equal the integer oracle's activations.
"""
import os
import sys

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, run_hip, run_ref

pytestmark = pytest.mark.gpu

sys.path.insert(0, os.path.join(entry.ROOT, "oracle"))

BATCH = 256
N_ORACLE = 2


def test_resnet50_fp16_batch256(models):
    announce("resnet50 fp16 batch 256")
    w = models.resnet50_weights()
    feeds = models.resnet50_input(BATCH)
    build = lambda b: models.build_resnet50(b, w, BATCH)
    got = run_hip(build, feeds, fp16=True)
    prob, logits = got["prob"], got["logits"]
    assert prob.shape == (BATCH, 1000) and logits.shape == (BATCH, 1000)
    assert np.all(np.isfinite(logits)) and np.all(np.isfinite(prob))
    assert np.max(np.abs(prob.sum(axis=1) - 1.0)) <= 1e-3
    assert np.all(prob >= 0)

    announce("resnet50 fp16 batch 256, reversed batch")
    rev = run_hip(build, {"input": np.ascontiguousarray(feeds["input"][::-1])}, fp16=True)
    assert np.array_equal(rev["logits"][::-1], logits)

    announce("resnet50 fp32 oracle, %d images" % N_ORACLE)
    sub = {"input": np.ascontiguousarray(feeds["input"][:N_ORACLE])}
    want = run_ref(lambda b: models.build_resnet50(b, w, N_ORACLE), sub)
    scale = max(1.0, float(np.max(np.abs(want["logits"]))))
    assert np.max(np.abs(logits[:N_ORACLE] - want["logits"])) <= 2e-2 * scale
    assert np.array_equal(np.argmax(logits[:N_ORACLE], 1), np.argmax(want["logits"], 1))


def test_resnet50_int8_batch256(models, odla, ref):
    announce("resnet50 int8: calibration on the oracle")
    import resnet_q8_ref
    w = models.resnet50_weights()
    small = 4

    def taps_of(feeds):
        rb = ref.RefBuilder(feeds)
        taps = []
        models.build_resnet50(rb, w, 2, taps=taps)
        return dict(taps)

    ranges = models.calibrate_ranges(taps_of, [models.resnet50_input(2, seed=2000 + i) for i in range(2)])
    entries = models.resnet50_quant_entries(w, ranges)
    qp = {e[0]: (e[1], e[2]) for e in entries if e[5] is None}
    qp["pool1"] = qp["stem.relu"]   # max pooling works on levels and keeps its input's scale / zero point
    feeds = models.resnet50_input(BATCH)
    sub = {"input": np.ascontiguousarray(feeds["input"][:small])}
    tap_names = ["pool1", "l1b2out", "l2b3out", "l3b5out", "l4b2out"]

    def build_n(n):
        def build(b):
            taps = []
            models.build_resnet50(b, w, n, taps=taps)
            d = dict(taps)
            for t in tap_names:
                b.output(d[t], t)
        return build

    announce("resnet50 int8 batch 256")
    big = run_hip(build_n(BATCH), feeds, quant_table=odla.quant_table(entries))
    announce("resnet50 int8 batch %d" % small)
    few = run_hip(build_n(small), sub, quant_table=odla.quant_table(entries))
    for t in tap_names + ["logits"]:
        assert np.array_equal(big[t][:small], few[t]), t

    announce("resnet50 int8 oracle, %d images" % small)
    record = {}
    want = resnet_q8_ref.run(w, sub, qp, models.RESNET50_STAGES, 64, small, 224, record)
    for t in tap_names:
        assert np.array_equal(few[t], ref.dequantize_act(record[t], *qp[t])), t
    assert np.max(np.abs(few["logits"] - want["logits"])) <= 1e-4 * max(1.0, float(np.max(np.abs(want["logits"]))))
