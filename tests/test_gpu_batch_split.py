"""One execution as two half-batch copies side by side (a context measures both ways and keeps
the faster; ODLA_HIP_BATCH_SPLIT = n forces halves from batch n on, 0 forbids them): each half is a copy of the recording at
half the batch, planned like any computation, with its own arena, stream and hipGraph, on its
half of the caller's buffers.  The results must be those of the whole batch; graphs that do not
keep the images' rows apart (batches joined end to end, one scale per row) and
executions whose results are not all bound to buffers run as one batch.
[function: odla_ExecuteComputation, ODLA/platforms/dnnl/odla_dnnl.cc:417-478 in the reference]"""
import numpy as np
import pytest

import __graft_entry__ as entry
from test_gpu_dynamic_batch import build_cnn, cnn_weights
from test_gpu_taps_kernel import run_logged
from util import announce, max_rel_err, run_hip, run_ref

pytestmark = pytest.mark.gpu

HALVES = "runs as two halves side by side"


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
@pytest.mark.parametrize("use_graph", [True, False])
def test_cnn_in_two_halves_equals_the_whole_batch(mode, use_graph, monkeypatch):
    w = cnn_weights(11)
    B = 8
    x = np.random.default_rng(12).standard_normal((B, 3, 20, 20)).astype(np.float32)
    build = build_cnn(w, B)
    kw = {"fp16": mode == "fp16"}
    announce("batch halves cnn %s graph=%s" % (mode, use_graph))
    monkeypatch.setenv("ODLA_HIP_BATCH_SPLIT", "0")
    whole, seen0 = run_logged(lambda: run_hip(build, {"x": x}, use_graph=use_graph, repeats=2, **kw))
    assert not any(HALVES in m for m in seen0)
    monkeypatch.setenv("ODLA_HIP_BATCH_SPLIT", "2")
    halves, seen = run_logged(lambda: run_hip(build, {"x": x}, use_graph=use_graph, repeats=3, **kw))
    assert any(HALVES in m for m in seen), [m for m in seen if "halves" in m]
    want = run_ref(build, {"x": x})
    for k in want:
        assert halves[k].shape == want[k].shape == whole[k].shape
        if mode == "fp32":
            assert max_rel_err(halves[k], want[k]) <= 1e-4, k
        else:
            assert np.max(np.abs(halves[k] - want[k])) <= 2e-2 * max(1.0, float(np.max(np.abs(want[k])))), k
        # every image's rows are where the whole batch puts them (a swapped or shifted half would
        # differ by the values' own size, rounding differs by far less)
        assert np.max(np.abs(halves[k] - whole[k])) <= (1e-5 if mode == "fp32" else 2e-2) * max(1.0, float(np.max(np.abs(want[k])))), k


def test_a_context_measures_and_keeps_the_faster_way(monkeypatch):
    """Without ODLA_HIP_BATCH_SPLIT a context runs six times whole, eight times in halves, then says
    which way it keeps; every one of these executions gives the whole batch's results."""
    odla = entry.load().odla
    B = 8
    r = np.random.default_rng(22)
    x = r.standard_normal((B, 16, 12, 12)).astype(np.float32)
    ws = [(r.standard_normal((16, 16, 3, 3)) * 0.12).astype(np.float32) for _ in range(9)]

    def build(b):   # (a plan of 18 launches and more: shorter ones are not tried)
        v = b.arg("x", (B, 16, 12, 12))
        for i, wi in enumerate(ws):
            c = b.conv(v, b.const("w%d" % i, wi), None, (1, 1), (1, 1, 1, 1), name="c%d" % i)
            v = b.tanh(b.add(c, v, name="s%d" % i), name="t%d" % i)
        b.output(v, "y")

    want = run_ref(build, {"x": x})
    monkeypatch.delenv("ODLA_HIP_BATCH_SPLIT", raising=False)
    announce("batch halves: measured choice")
    hb = odla.HipBuilder()
    try:
        build(hb)
        s = hb.session(True)
        try:
            def go():
                outs = []
                for _ in range(18):
                    outs.append(s.run({"x": x}))
                return outs
            outs, seen = run_logged(go)
        finally:
            s.close()
    finally:
        hb.destroy()
    verdicts = [m for m in seen if "runs as two halves side by side (" in m or "stays whole (" in m]
    assert len(verdicts) == 1, [m for m in seen if "halves" in m or "whole" in m]
    for got in outs:
        for k in want:
            assert max_rel_err(got[k], want[k]) <= 1e-4, k


def test_device_buffers_are_split_in_place(monkeypatch):
    """Arguments and results resident in device memory: each half reads and writes its half of
    the caller's buffers in place."""
    odla = entry.load().odla
    w = cnn_weights(13)
    B = 6
    x = np.random.default_rng(14).standard_normal((B, 3, 20, 20)).astype(np.float32)
    build = build_cnn(w, B)
    monkeypatch.setenv("ODLA_HIP_BATCH_SPLIT", "2")
    announce("batch halves device buffers")
    hb = odla.HipBuilder()
    try:
        build(hb)
        s = hb.session(True)
        try:
            def go():
                s.bind_device_io({"x": x})
                for _ in range(3):
                    s.execute()
                return s.fetch_device_outputs()
            got, seen = run_logged(go)
            # odla_GetValueData after such an execution collects the rows from both halves
            import ctypes
            L = odla.load_library()
            for name, (h, shape, dt) in hb.outs.items():
                again = np.empty(shape, dt)
                assert L.odla_GetValueData(h, again.ctypes.data_as(ctypes.c_void_p), s.ctx) == 0
                assert np.array_equal(again, got[name]), name
        finally:
            s.close()
    finally:
        hb.destroy()
    assert any(HALVES in m for m in seen)
    want = run_ref(build, {"x": x})
    for k in want:
        assert max_rel_err(got[k], want[k]) <= 1e-4, k


@pytest.mark.parametrize("B", [2, 6])
def test_detections_keep_the_numbers_of_the_whole_batch(B, monkeypatch):
    """NonMaxSuppression lists (image, class, box) triples, max_num_outputs rows per image: the
    second half writes its images' rows with the numbers they have in the whole batch."""
    r = np.random.default_rng(15 + B)
    N, C = 64, 3
    xy = r.uniform(0, 40, (B, N, 2)).astype(np.float32)
    wh = r.uniform(4, 16, (B, N, 2)).astype(np.float32)
    boxes = np.concatenate([xy, xy + wh], axis=2)
    scores = r.uniform(0, 1, (B, C, N)).astype(np.float32)

    def build(b):
        bx = b.arg("boxes", (B, N, 4))
        sc = b.arg("scores", (B, C, N))
        b.output(b.nms(bx, sc, 10, 0.5, 0.3, name="keep"), "keep")

    monkeypatch.setenv("ODLA_HIP_BATCH_SPLIT", "2")
    announce("batch halves: nms, batch %d" % B)
    got, seen = run_logged(lambda: run_hip(build, {"boxes": boxes, "scores": scores}))
    assert any(HALVES in m for m in seen)
    want = run_ref(build, {"boxes": boxes, "scores": scores})
    assert np.array_equal(got["keep"], want["keep"])
    assert set(np.unique(want["keep"][:, 0])) >= set(range(B))   # every image has detections, under its own number


def test_batches_joined_end_to_end_run_as_one_batch(monkeypatch):
    B = 4
    r = np.random.default_rng(16)
    a = r.standard_normal((B, 5, 3)).astype(np.float32)
    c = r.standard_normal((B, 5, 3)).astype(np.float32)

    def build(b):
        x = b.arg("a", (B, 5, 3))
        y = b.arg("c", (B, 5, 3))
        b.output(b.relu(b.concat([x, y], 0, name="joined"), name="out"), "out")

    monkeypatch.setenv("ODLA_HIP_BATCH_SPLIT", "2")
    announce("batch halves refused: concat along the batch")
    got, seen = run_logged(lambda: run_hip(build, {"a": a, "c": c}))
    assert not any(HALVES in m for m in seen)
    assert np.array_equal(got["out"], np.maximum(np.concatenate([a, c], 0), 0))
