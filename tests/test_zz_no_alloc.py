"""odla_hip_ExecuteComputationStatic: the execution entry point that allocates no
device memory (the plan's temporaries live in the library's static device
scratch, launches are issued un-captured).  Its results must equal, bit for
bit, those of odla_ExecuteComputation on the same bound device buffers - on two
calls in a row, the second with a smaller input - and the device's used-memory
figure must not move across the calls.
"""
import ctypes

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce

pytestmark = pytest.mark.gpu

STAGES = [(8, 1, 1), (16, 1, 2)]


def small_net(odla, models, batch, mode, seed=7):
    """(builder, session with device-resident I/O) of a small ResNet-shaped network."""
    w = models.resnet50_weights(seed=seed, num_classes=10, stages=STAGES, stem=8)
    hb = odla.HipBuilder(fp16=(mode == "fp16"))
    models.build_resnet50(hb, w, batch, 32, STAGES, 8, 10)
    s = hb.session(True)
    s.bind_device_io(models.resnet50_input(batch, 32, seed=seed + batch))
    return hb, s


def both_ways(s):
    """Outputs of the ordinary and of the static execution of one session."""
    s.execute()
    want = s.fetch_device_outputs()
    # poison the result buffers so that a static call that wrote nothing cannot pass
    for name, (p, shape, dt) in s.dev_out.items():
        junk = np.full(shape, 123, dt)
        assert s.L.odla_CopyMemory(p, junk.ctypes.data_as(ctypes.c_void_p), junk.nbytes, 1) == 0
    assert s.execute_static() == 0
    got = s.fetch_device_outputs()
    return got, want


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_static_execution_equals_ordinary_execution_twice_in_a_row(odla, models, mode):
    announce("static execution, %s, batch 8 then batch 3" % mode)
    hb8, s8 = small_net(odla, models, 8, mode)
    hb3, s3 = small_net(odla, models, 3, mode)
    try:
        got8, want8 = both_ways(s8)
        for k in want8:
            assert got8[k].shape[0] == 8 and np.array_equal(got8[k], want8[k]), k
        # a second call right behind it, on a smaller input: the scratch still holds batch 8's temporaries
        got3, want3 = both_ways(s3)
        for k in want3:
            assert got3[k].shape[0] == 3 and np.array_equal(got3[k], want3[k]), k
        assert np.all(np.isfinite(want3["logits"])) and np.max(np.abs(want3["logits"])) > 0
        # and back: what the smaller call left behind does not matter either
        used0 = odla.used_device_memory()
        for _ in range(3):
            assert s8.execute_static() == 0
            assert s3.execute_static() == 0
        assert odla.used_device_memory() == used0          # nothing was allocated by the calls
        again8 = s8.fetch_device_outputs()
        for k in want8:
            assert np.array_equal(again8[k], want8[k]), k
    finally:
        s8.close(); s3.close()
        hb8.destroy(); hb3.destroy()


def test_static_execution_int8_plan(odla, models, ref):
    """The quantised plan (requantising epilogues, 8-bit temporaries) through the static entry point."""
    announce("static execution, int8")
    stages, stem = [(16, 1, 1), (32, 2, 2)], 16      # 8-bit tensors want channel counts that are multiples of 16
    w = models.resnet50_weights(seed=11, num_classes=10, stages=stages, stem=stem)

    def taps_of(feeds):
        rb = ref.RefBuilder(feeds)
        taps = []
        models.build_resnet50(rb, w, 2, 32, stages, stem, 10, taps=taps)
        return dict(taps)

    ranges = models.calibrate_ranges(taps_of, [models.resnet50_input(2, 32, seed=50 + i) for i in range(2)])
    table = odla.quant_table(models.resnet50_quant_entries(w, ranges, stages, stem))
    hb = odla.HipBuilder(quant_table=table)
    models.build_resnet50(hb, w, 4, 32, stages, stem, 10)
    s = hb.session(True)
    try:
        s.bind_device_io(models.resnet50_input(4, 32, seed=60))
        got, want = both_ways(s)
        for k in want:
            assert np.array_equal(got[k], want[k]), k
    finally:
        s.close()
        hb.destroy()


def test_static_execution_refuses_what_it_cannot_hold(odla):
    announce("static execution: limits")
    # temporaries beyond the static scratch (64 MiB): a 128 MiB tensor through two launches
    hb = odla.HipBuilder()
    x = hb.arg("x", (32, 1 << 20))
    hb.output(hb.relu(hb.exp(x, name="e"), name="y"), "y")
    s = hb.session(True)
    try:
        xin = np.zeros((32, 1 << 20), np.float32)
        s.bind_device_io({"x": xin})
        hb.L.odla_SetLogLevel(0)
        assert s.execute_static() == 4          # ODLA_MEM_ERROR
        hb.L.odla_SetLogLevel(2)
        s.execute()                             # the ordinary entry point still runs it
        assert np.array_equal(s.fetch_device_outputs()["y"], np.ones_like(xin))
    finally:
        s.close()
        hb.destroy()
    # another run-time batch than the recorded one would have to plan (and allocate) a copy
    hb = odla.HipBuilder(max_batch=4)
    x = hb.arg("x", (-1, 16))
    hb.output(hb.relu(x, name="y"), "y")
    s = hb.session(True)
    try:
        s.set_batch(2)
        hb.L.odla_SetLogLevel(0)
        assert s.execute_static() == 7          # ODLA_UNSUPPORTED_OP
        hb.L.odla_SetLogLevel(2)
    finally:
        s.close()
        hb.destroy()
    assert hb.L.odla_hip_ExecuteComputationStatic(None, None, 1, None) == odla.ODLA_INVALID_PARAM
