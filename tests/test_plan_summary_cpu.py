"""odla_hip_PlanSummary lowers a recorded graph on the host, so the planner -
operator fusion, layout choices, arena assignment - is exercised here without
a GPU: launch counts and device-memory needs of the benchmark graphs and the
element-wise group fusion (the decode of
a detection head collapses to a handful of launches).
"""
import ctypes

import numpy as np
import pytest


def summary_of(odla, build, **kw):
    hb = odla.HipBuilder(**kw)
    try:
        build(hb)
        first = hb.plan_summary()
        assert hb.plan_summary() == first   # lowering leaves the recording unchanged
        return first
    finally:
        hb.destroy()


def test_resnet50_fp16_plan(pkg, odla, models):
    w = models.resnet50_weights()
    s = summary_of(odla, lambda b: models.build_resnet50(b, w, 8), fp16=True)
    # 53 convolutions + classifier, the input relayout, two pools, softmax, output cast;
    # BatchNorm, ReLU and the residual adds ride in the convolution epilogues
    assert 55 <= s["launches"] <= 70, s
    assert 50e6 < s["constant_bytes"] < 120e6, s    # 25.5 M weights in fp16, packed rows plus the MFMA-fragment copies
    assert 0 < s["arena_bytes"] < 200e6, s


def test_resnet50_arena_scales_with_batch(pkg, odla, models):
    w = models.resnet50_weights(stages=((1, 16, 1), (1, 32, 2)), stem=16, num_classes=10)
    one = summary_of(odla, lambda b: models.build_resnet50(b, w, 2, hw=64, stages=((1, 16, 1), (1, 32, 2)), stem=16,
                                                             num_classes=10), fp16=True)
    two = summary_of(odla, lambda b: models.build_resnet50(b, w, 8, hw=64, stages=((1, 16, 1), (1, 32, 2)), stem=16,
                                                             num_classes=10), fp16=True)
    assert one["launches"] == two["launches"]
    assert one["constant_bytes"] == two["constant_bytes"]
    assert 3.0 < two["arena_bytes"] / one["arena_bytes"] < 4.5


def test_bert_plan_has_no_head_transposes(pkg, odla):
    mb = pkg.models_bert
    cfg = dict(mb.BERT_BASE)
    cfg.update(layers=2)
    w = mb.bert_weights(cfg)
    s = summary_of(odla, lambda b: mb.build_bert(b, w, 4, 128, cfg), bf16=True)
    # per layer: merged QKV, scores, softmax, context, projection, LayerNorm, two FFN GEMMs, LayerNorm
    assert s["launches"] <= 2 * 10 + 12, s


def test_yolo_decode_is_fused(pkg, odla):
    my = pkg.models_yolo
    s = summary_of(odla, lambda b: my.build_yolo_postprocess(b, 4), fp16=True)
    # per head: layout change, transpose, one launch for the boxes, one for the scores;
    # then the two concatenations over the heads and the NMS
    assert s["launches"] <= 3 * 4 + 6 + 6, s


def test_plan_summary_rejects_bad_arguments(odla):
    L = odla.load_library()
    ps = odla.PlanSummary()
    assert L.odla_hip_PlanSummary(None, ctypes.byref(ps)) != 0
    hb = odla.HipBuilder()
    try:
        x = hb.arg("x", (2, 3))
        hb.output(hb.relu(x, name="y"), "y")
        assert L.odla_hip_PlanSummary(hb.comp, None) != 0
        s = hb.plan_summary()
        assert s["launches"] >= 1 and s["arena_bytes"] >= 2 * 3 * 4
    finally:
        hb.destroy()
