"""Full-size ResNet-50 v1.5 at the benchmark batch (256 x 3 x 224 x 224).

  * fp16: probabilities are finite and sum to 1; the images of the batch do not
    influence each other (reversing the batch reverses the outputs bit for bit);
    EVERY image of the batch is compared with two oracles:
      - the precision-emulating oracle (the fp32 graph with every stored tensor
        rounded to fp16 where the fp16 plan stores one): every logit within two
        fp16 units of the last place of the image's largest logit (measured: at
        most one, half of the logits bit-equal), and the GPU's differences from
        fp32 - largest, 99.9th percentile, mean - within 1.25 x those of the
        emulated oracle, so an implementation that lost twice what the storage
        type costs would fail;
      - the fp32 oracle: same top-1 class on all 256, and the largest difference
        of the logits within 1e-3 of the largest logit.  The stated bound, 2e-2
        absolute, presumes logits of the usual magnitude (about 20, where it is
        the same 1e-3): the random He-normal weights of this configuration, with
        identity batch norms, give logits up to 3.7e3, where neighbouring fp16
        numbers are 2.0 apart.  The floor is printed beside the measurement: the
        emulated oracles (operands only / every stored tensor) differ from fp32
        by 2.3 / 2.7 on the first 32 images, the GPU by 2.6.
  * int8: ALL 256 images are compared with the integer oracle: the 8-bit
    activations behind the first pooling and behind every stage bit for bit, the
    fp32 logits to 1e-4 of their scale, top-1 equal on 256 / 256; the same
    images run at batch 4 give the same bits as in the batch of 256.
    Activation ranges come from 32 seeded N(0,1) batches (seeds 1000 .. 1031,
    one image each) run through the fp32 oracle.
"""
import os
import sys

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, err_stats, run_hip, run_ref, run_ref_emulated

pytestmark = pytest.mark.gpu

sys.path.insert(0, os.path.join(entry.ROOT, "oracle"))

BATCH = 256
ORACLE_CHUNK = 32    # images per oracle pass (bounds the oracle's memory)
FP16_ABS_TOL = 2e-2  # on the logits, absolute, for logits of magnitude up to 20
FP16_REL_TOL = 1e-3  # ... and this fraction of the largest logit beyond


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

    want = np.empty_like(logits)
    emu = np.empty_like(logits)
    floor_op = None
    for i0 in range(0, BATCH, ORACLE_CHUNK):
        announce("resnet50 fp32 and fp16-emulating oracle, images %d .. %d" % (i0, i0 + ORACLE_CHUNK - 1))
        sub = {"input": np.ascontiguousarray(feeds["input"][i0:i0 + ORACLE_CHUNK])}
        build_c = lambda b: models.build_resnet50(b, w, ORACLE_CHUNK)
        want[i0:i0 + ORACLE_CHUNK] = run_ref(build_c, sub)["logits"]
        emu[i0:i0 + ORACLE_CHUNK] = run_ref_emulated(build_c, sub, "stored", "fp16")["logits"]
        if i0 == 0:   # what rounding the Conv / Gemm operands alone costs (first chunk)
            floor_op = err_stats(run_ref_emulated(build_c, sub, "operands", "fp16")["logits"], want[:ORACLE_CHUNK])
    err = np.max(np.abs(logits - want), axis=1)
    top_ok = np.argmax(logits, 1) == np.argmax(want, 1)
    srt = np.sort(want, axis=1)
    announce("resnet50 fp16 vs fp32 oracle over %d images: max |d logits| = %.3e (mean of per-image maxima %.3e), "
             "largest |logit| = %.3f, top-1 equal on %d / %d, smallest top-1 margin of the oracle = %.3e"
             % (BATCH, err.max(), err.mean(), np.max(np.abs(want)), int(top_ok.sum()), BATCH,
                float(np.min(srt[:, -1] - srt[:, -2]))))
    announce("floor: operands-emulated oracle vs fp32 (first %d images)  max %.3e  p99.9 %.3e  mean %.3e" % ((ORACLE_CHUNK,) + floor_op))
    announce("floor: stored-emulated oracle vs fp32 (all images)         max %.3e  p99.9 %.3e  mean %.3e" % err_stats(emu, want))
    announce("GPU fp16 vs fp32 oracle                                     max %.3e  p99.9 %.3e  mean %.3e" % err_stats(logits, want))
    # Against the emulated oracle.  A logit is a sum of 2048 products that largely cancel, so its
    # error has the scale of the image's largest logits, not its own: the unit is one fp16 unit
    # of the last place of the row's largest magnitude (2.0 for logits beyond 2048).
    row_max = np.max(np.maximum(np.abs(logits), np.abs(emu)), axis=1, keepdims=True)
    ulp = 2.0 ** (np.floor(np.log2(row_max)) - 10)
    d_ulp = np.abs(logits - emu) / ulp
    floor_st, e_gpu, d_emu = err_stats(emu, want), err_stats(logits, want), err_stats(logits, emu)
    announce("GPU fp16 vs stored-emulated oracle: max %.3e (%.2f units of the last place of the row's largest logit)  "
             "p99.9 %.3e  mean %.3e, %.1f %% of the logits bit-equal"
             % (d_emu[0], d_ulp.max(), d_emu[1], d_emu[2], 100.0 * np.mean(logits == emu)))
    assert d_ulp.max() <= 2.0 and d_emu[2] <= floor_st[2]
    assert np.mean(logits == emu) >= 0.3
    for k in range(3):   # nothing beyond what fp16 storage costs (twice that would fail)
        assert e_gpu[k] <= 1.25 * floor_st[k], k
    assert err.max() <= max(FP16_ABS_TOL, FP16_REL_TOL * float(np.max(np.abs(want))))
    assert np.all(top_ok)


def test_resnet50_int8_batch256(models, odla, ref):
    announce("resnet50 int8: calibration on the oracle")
    import resnet_q8_ref
    w = models.resnet50_weights()
    small = 4

    def taps_of(feeds):
        rb = ref.RefBuilder(feeds)
        taps = []
        models.build_resnet50(rb, w, 1, taps=taps)
        return dict(taps)

    ranges = models.calibrate_ranges(taps_of, [models.resnet50_input(1, seed=1000 + i) for i in range(32)])
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

    top_equal = 0
    for i0 in range(0, BATCH, ORACLE_CHUNK):
        announce("resnet50 int8 oracle, images %d .. %d" % (i0, i0 + ORACLE_CHUNK - 1))
        chunk = {"input": np.ascontiguousarray(feeds["input"][i0:i0 + ORACLE_CHUNK])}
        record = {}
        want = resnet_q8_ref.run(w, chunk, qp, models.RESNET50_STAGES, 64, ORACLE_CHUNK, 224, record)
        for t in tap_names:
            assert np.array_equal(big[t][i0:i0 + ORACLE_CHUNK], ref.dequantize_act(record[t], *qp[t])), (t, i0)
        got_l = big["logits"][i0:i0 + ORACLE_CHUNK]
        assert np.max(np.abs(got_l - want["logits"])) <= 1e-4 * max(1.0, float(np.max(np.abs(want["logits"]))))
        top_equal += int(np.sum(np.argmax(got_l, 1) == np.argmax(want["logits"], 1)))
    announce("resnet50 int8 vs integer oracle over %d images: %d taps bit-equal, top-1 equal on %d / %d"
             % (BATCH, len(tap_names), top_equal, BATCH))
    assert top_equal == BATCH
