"""Arguments bound to device memory.  When only layout conversions read an
argument's staging tensor, odla_ExecuteComputation lets them read the caller's
buffer where it is (no copy into the arena); the captured launch sequence then
holds that address, so other buffers bring another graph.  Every case is
checked against the CPU oracle on the same data.

Tolerance: fp32 graphs, 1e-4 of the largest expected magnitude (convolutions).
"""
import ctypes

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, run_ref

pytestmark = pytest.mark.gpu


def small_net(b, N, s2d):
    r = np.random.default_rng(5)
    x = b.arg("x", (N, 3, 20, 20))
    if s2d:   # 7x7 stride 2 on three channels: the space-to-depth conversion reads the argument
        w = (r.standard_normal((8, 3, 7, 7)) * 0.1).astype(np.float32)
        y = b.conv(x, b.const("w", w), stride=(2, 2), pad=(3, 3, 3, 3), name="stem")
    else:     # 3x3 stride 1: the channels-last conversion reads it
        w = (r.standard_normal((8, 3, 3, 3)) * 0.2).astype(np.float32)
        y = b.conv(x, b.const("w", w), pad=(1, 1, 1, 1), name="stem")
    b.output(b.relu(y, name="act"), "y")


class DeviceBuffers:
    def __init__(self, odla, L):
        self.odla, self.L, self.ptrs = odla, L, []

    def put(self, a, offset=0):
        p = ctypes.c_void_p()
        assert self.L.odla_AllocateDeviceMemory(ctypes.byref(p), a.nbytes + offset) == 0
        self.ptrs.append(p)
        q = ctypes.c_void_p(p.value + offset)
        assert self.L.odla_CopyMemory(q, a.ctypes.data_as(ctypes.c_void_p), a.nbytes, self.odla.ODLA_MEMCPY_H2D) == 0
        return q

    def free(self):
        for p in self.ptrs:
            self.L.odla_FreeDeviceMemory(p)


def capture_log(L, seen):
    CB = ctypes.CFUNCTYPE(None, ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p)
    cb = CB(lambda f, line, fn, lvl, msg: seen.append(msg.decode()))
    L.odla_SetLogger(ctypes.cast(cb, ctypes.c_void_p))
    L.odla_SetLogLevel(5)
    return cb


@pytest.mark.parametrize("s2d", [False, True])
@pytest.mark.parametrize("use_graph", [True, False])
def test_device_arguments_are_read_in_place(s2d, use_graph):
    announce("device arguments s2d=%s graph=%s" % (s2d, use_graph))
    pkg = entry.load()
    odla = pkg.odla
    L = odla.load_library()
    N = 3
    r = np.random.default_rng(17)
    datas = [r.standard_normal((N, 3, 20, 20)).astype(np.float32) for _ in range(6)]
    wants = [run_ref(lambda b: small_net(b, N, s2d), {"x": d})["y"] for d in datas]
    hb = odla.HipBuilder()
    bufs = DeviceBuffers(odla, L)
    seen = []
    cb = capture_log(L, seen)
    try:
        small_net(hb, N, s2d)
        s = hb.session(use_graph)
        h = hb.args["x"][0]
        oh, oshape, odt = hb.outs["y"]
        out = np.empty(oshape, odt)
        assert L.odla_BindToOutput(oh, out.ctypes.data_as(ctypes.c_void_p), s.ctx) == 0

        def run_with(ptr, want):
            assert L.odla_BindToArgument(h, ptr, s.ctx) == 0
            s.execute()
            assert float(np.max(np.abs(out - want))) <= 1e-4 * max(1.0, float(np.max(np.abs(want))))

        dev = [bufs.put(d) for d in datas]
        # the same buffer twice (replay), then others (each captures), then back (the set-aside graphs)
        for k in (0, 0, 1, 2, 0, 1, 3, 4, 5, 0):
            run_with(dev[k], wants[k])
        assert any("'x' is read in place" in m for m in seen), seen[-5:]
        # new contents in a buffer the graph already holds
        assert L.odla_CopyMemory(dev[0], datas[3].ctypes.data_as(ctypes.c_void_p), datas[3].nbytes, odla.ODLA_MEMCPY_H2D) == 0
        run_with(dev[0], wants[3])
        # a buffer that is only 4-byte aligned: the conversions fall back to narrower loads
        run_with(bufs.put(datas[2], offset=4), wants[2])
        # host memory goes through the staging copy, as before
        seen.clear()
        run_with(datas[4].ctypes.data_as(ctypes.c_void_p), wants[4])
        assert not any("read in place" in m for m in seen), seen
        run_with(dev[1], wants[1])
        s.close()
    finally:
        L.odla_SetLogLevel(2)
        L.odla_SetLogger(None)
        bufs.free()
        hb.destroy()


def test_argument_with_other_readers_is_copied():
    """An argument that a GEMM reads directly (no layout conversion in between) keeps
    its copy into the arena: the GEMM's loads rely on the arena's alignment."""
    announce("device argument read by a GEMM")
    pkg = entry.load()
    odla = pkg.odla
    L = odla.load_library()
    r = np.random.default_rng(18)
    x = r.standard_normal((5, 37)).astype(np.float32)
    w = (r.standard_normal((37, 11)) * 0.3).astype(np.float32)

    def build(b):
        b.output(b.gemm(b.arg("x", x.shape), b.const("w", w), name="mm"), "y")

    want = run_ref(build, {"x": x})["y"]
    hb = odla.HipBuilder()
    bufs = DeviceBuffers(odla, L)
    seen = []
    cb = capture_log(L, seen)
    try:
        build(hb)
        s = hb.session(True)
        out = np.empty(want.shape, np.float32)
        assert L.odla_BindToOutput(hb.outs["y"][0], out.ctypes.data_as(ctypes.c_void_p), s.ctx) == 0
        assert L.odla_BindToArgument(hb.args["x"][0], bufs.put(x, offset=4), s.ctx) == 0
        s.execute()
        assert float(np.max(np.abs(out - want))) <= 1e-4 * max(1.0, float(np.max(np.abs(want))))
        assert not any("read in place" in m for m in seen), seen
        s.close()
    finally:
        L.odla_SetLogLevel(2)
        L.odla_SetLogger(None)
        bufs.free()
        hb.destroy()


def test_device_results_are_written_in_place():
    """fp16 storage: the conversion of the result to its declared fp32 writes the
    caller's device buffer.  Checked against the oracle at 2e-2 absolute on O(1) data
    (fp16 storage), and exactly against the same execution through a host buffer."""
    announce("device results in place")
    pkg = entry.load()
    odla = pkg.odla
    L = odla.load_library()
    N = 2
    x = np.random.default_rng(19).standard_normal((N, 3, 20, 20)).astype(np.float32)
    want = run_ref(lambda b: small_net(b, N, False), {"x": x})["y"]
    hb = odla.HipBuilder(fp16=True)
    bufs = DeviceBuffers(odla, L)
    seen = []
    cb = capture_log(L, seen)
    try:
        small_net(hb, N, False)
        s = hb.session(True)
        oh, oshape, odt = hb.outs["y"]
        host_out = np.empty(oshape, odt)
        assert L.odla_BindToArgument(hb.args["x"][0], x.ctypes.data_as(ctypes.c_void_p), s.ctx) == 0
        assert L.odla_BindToOutput(oh, host_out.ctypes.data_as(ctypes.c_void_p), s.ctx) == 0
        s.execute()
        assert float(np.max(np.abs(host_out - want))) <= 2e-2
        assert not any("written in place" in m for m in seen), seen

        def fetch(p):
            o = np.empty(oshape, odt)
            assert L.odla_CopyMemory(o.ctypes.data_as(ctypes.c_void_p), p, o.nbytes, odla.ODLA_MEMCPY_D2H) == 0
            return o

        for rep in range(3):   # capture, replay, replay
            d_out = bufs.put(np.zeros(oshape, odt)) if rep < 2 else d_out
            assert L.odla_BindToOutput(oh, d_out, s.ctx) == 0
            s.execute()
            assert np.array_equal(fetch(d_out), host_out)
        assert any("'act' is written in place" in m for m in seen), seen[-5:]
        again = np.empty(oshape, odt)
        assert L.odla_GetValueData(oh, again.ctypes.data_as(ctypes.c_void_p), s.ctx) == 0
        assert np.array_equal(again, host_out)
        # argument and result in one device allocation, overlapping: the result keeps its copy
        both = bufs.put(np.zeros(x.nbytes + host_out.nbytes, np.uint8))
        assert L.odla_CopyMemory(both, x.ctypes.data_as(ctypes.c_void_p), x.nbytes, odla.ODLA_MEMCPY_H2D) == 0
        assert L.odla_BindToArgument(hb.args["x"][0], both, s.ctx) == 0
        seen.clear()
        assert L.odla_BindToOutput(oh, ctypes.c_void_p(both.value + 64), s.ctx) == 0
        s.execute()
        assert not any("written in place" in m for m in seen), seen
        assert np.array_equal(fetch(ctypes.c_void_p(both.value + 64)), host_out)
        s.close()
    finally:
        L.odla_SetLogLevel(2)
        L.odla_SetLogger(None)
        bufs.free()
        hb.destroy()


def test_new_buffer_every_call_goes_back_to_copies(monkeypatch):
    """Twelve executions, each with another device buffer: after eight captures in a
    row the context stages the argument again and replays one graph."""
    announce("device arguments, a new buffer every call")
    monkeypatch.setenv("ODLA_HIP_BATCH_SPLIT", "0")   # (the messages counted below are one context's)
    pkg = entry.load()
    odla = pkg.odla
    L = odla.load_library()
    N = 2
    r = np.random.default_rng(20)
    hb = odla.HipBuilder()
    bufs = DeviceBuffers(odla, L)
    seen = []
    cb = capture_log(L, seen)
    try:
        small_net(hb, N, True)
        s = hb.session(True)
        oh, oshape, odt = hb.outs["y"]
        out = np.empty(oshape, odt)
        assert L.odla_BindToOutput(oh, out.ctypes.data_as(ctypes.c_void_p), s.ctx) == 0
        for k in range(12):
            x = r.standard_normal((N, 3, 20, 20)).astype(np.float32)
            want = run_ref(lambda b: small_net(b, N, True), {"x": x})["y"]
            assert L.odla_BindToArgument(hb.args["x"][0], bufs.put(x), s.ctx) == 0
            s.execute()
            assert float(np.max(np.abs(out - want))) <= 1e-4 * max(1.0, float(np.max(np.abs(want)))), k
        assert any("copied from now on" in m for m in seen)
        assert sum("read in place" in m for m in seen) <= 9
        s.close()
    finally:
        L.odla_SetLogLevel(2)
        L.odla_SetLogger(None)
        bufs.free()
        hb.destroy()


def test_short_launch_sequences_run_uncaptured(monkeypatch):
    """Without ODLA_HIP_GRAPH_MIN_STEPS a plan of fewer than six launches is not captured: the
    library says so once, a new device buffer every call needs no new graph, and the results are
    those of the oracle; a plan of six launches or more is captured as before."""
    announce("short launch sequences")
    monkeypatch.delenv("ODLA_HIP_GRAPH_MIN_STEPS", raising=False)
    monkeypatch.setenv("ODLA_HIP_BATCH_SPLIT", "0")   # (the messages counted below are one context's)
    pkg = entry.load()
    odla = pkg.odla
    L = odla.load_library()
    r = np.random.default_rng(21)
    x0 = r.standard_normal((4, 24)).astype(np.float32)

    def chain(b, n):
        v = b.arg("x", x0.shape)
        for i in range(n):
            v = b.softmax(v, -1, name="s%d" % i)
        b.output(v, "y")

    for n, captured in ((2, False), (7, True)):
        hb = odla.HipBuilder()
        bufs = DeviceBuffers(odla, L)
        seen = []
        cb = capture_log(L, seen)
        try:
            chain(hb, n)
            s = hb.session(True)
            oh, oshape, odt = hb.outs["y"]
            out = np.empty(oshape, odt)
            assert L.odla_BindToOutput(oh, out.ctypes.data_as(ctypes.c_void_p), s.ctx) == 0
            for k in range(3):
                x = r.standard_normal(x0.shape).astype(np.float32)
                want = run_ref(lambda b: chain(b, n), {"x": x})["y"]
                assert L.odla_BindToArgument(hb.args["x"][0], bufs.put(x), s.ctx) == 0
                s.execute()
                assert float(np.max(np.abs(out - want))) <= 1e-5, (n, k)
            assert any("run uncaptured" in m for m in seen) == (not captured), (n, seen[-5:])
            assert sum("run uncaptured" in m for m in seen) <= 1
            s.close()
        finally:
            L.odla_SetLogLevel(2)
            L.odla_SetLogger(None)
            bufs.free()
            hb.destroy()
        del cb
