"""Element-wise group fusion: chains of unary / binary operators on values of
rank <= 3, with Slices in front and a Concat or Transpose behind, run as one
launch.  Every case is checked against the CPU oracle, and the launch list of
the plan (odla_hip_ProfileSteps) shows that the fusion took place - or, for
the shapes it must leave alone, that it did not.

Tolerance: fp32 graphs 1e-5 of the largest expected magnitude (the group keeps
fp32 between its operators, as the separate launches do); fp16 storage 2e-2
absolute on O(1) data.
"""
import ctypes

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, run_ref

pytestmark = pytest.mark.gpu


def run_with_steps(build_fn, feeds, **kw):
    """(outputs, names of the launches of one execution)."""
    pkg = entry.load()
    odla = pkg.odla
    L = odla.load_library()

    class StepTime(ctypes.Structure):
        _fields_ = [("name", ctypes.c_char * 64), ("ms", ctypes.c_float)]

    L.odla_hip_ProfileSteps.restype = ctypes.c_int32
    L.odla_hip_ProfileSteps.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(StepTime), ctypes.c_int32,
                                        ctypes.POINTER(ctypes.c_int32)]
    hb = odla.HipBuilder(**kw)
    try:
        build_fn(hb)
        s = hb.session(True)
        try:
            out = s.run(feeds)
            out2 = s.run(feeds)   # graph replay
            for k in out:
                assert np.array_equal(out[k], out2[k]), k
            buf = (StepTime * 512)()
            n = ctypes.c_int32()
            assert L.odla_hip_ProfileSteps(s.ctx, 1, buf, 512, ctypes.byref(n)) == 0
            return out, [buf[i].name.decode() for i in range(n.value)]
        finally:
            s.close()
    finally:
        hb.destroy()


def check(got, want, tol):
    for k in want:
        assert got[k].shape == want[k].shape, k
        scale = max(1.0, float(np.max(np.abs(want[k]))))
        assert float(np.max(np.abs(got[k].astype(np.float64) - want[k]))) <= tol * scale, k


def fused(steps):
    return [s for s in steps if s.startswith("fused:")]


def yolo_like(b, N, nb, C):
    t = b.arg("t", (N, nb, 5 + C))
    gx = b.const("gx", np.arange(nb, dtype=np.float32).reshape(1, nb, 1))
    aw = b.const("aw", np.linspace(0.1, 0.9, nb, dtype=np.float32).reshape(1, nb, 1))
    half = b.const("half", np.full((1,), 0.5, np.float32))
    ig = b.const("ig", np.full((1,), 1.0 / 13.0, np.float32))

    def comp(k0, k1, nm):
        return b.slice(t, (0, 0, k0), (N, nb, k1), name=nm)

    cx = b.mul(b.add(b.sigmoid(comp(0, 1, "tx"), name="sx"), gx, name="ax"), ig, name="cx")
    cy = b.mul(b.add(b.sigmoid(comp(1, 2, "ty"), name="sy"), gx, name="ay"), ig, name="cy")
    bw = b.mul(b.exp(comp(2, 3, "tw"), name="ew"), aw, name="bw")
    bh = b.mul(b.exp(comp(3, 4, "th"), name="eh"), aw, name="bh")
    hw, hh = b.mul(bw, half, name="hw"), b.mul(bh, half, name="hh")
    box = b.concat([b.sub(cy, hh, name="y1"), b.sub(cx, hw, name="x1"), b.add(cy, hh, name="y2"),
                    b.add(cx, hw, name="x2")], 2, name="box")
    obj = b.sigmoid(comp(4, 5, "to"), name="obj")
    cls = b.sigmoid(comp(5, 5 + C, "tc"), name="cls")
    sc = b.mul(cls, obj, name="score")
    b.output(box, "box")
    b.output(b.transpose(sc, (0, 2, 1), name="score_t"), "score_t")


@pytest.mark.parametrize("mode,shape", [("fp32", (2, 48, 7)), ("fp16", (3, 507, 80)), ("fp32", (1, 5, 1))])
def test_box_decode_is_two_launches(mode, shape):
    """The decode of a detection head (Slices, Sigmoid / Exp, broadcast constants,
    scalar constants, Concat of four one-column results, Transpose of the class
    scores) becomes one launch for the boxes and one for the scores."""
    N, nb, C = shape
    announce("fused box decode %s %s" % (mode, shape))
    x = np.random.default_rng(7).standard_normal((N, nb, 5 + C)).astype(np.float32)
    build = lambda b: yolo_like(b, N, nb, C)
    got, steps = run_with_steps(build, {"t": x}, fp16=(mode == "fp16"))
    want = run_ref(build, {"t": x})
    check(got, want, 1e-5 if mode == "fp32" else 2e-2)
    assert len(fused(steps)) == 2, steps
    assert not [s for s in steps if s.startswith(("slice:", "unary:", "binary:", "concat:", "transpose:"))], steps


def test_group_with_several_results_and_shared_operands():
    """Results used outside the group are stored as well; an operand read twice is
    loaded once; both operand orders of a scalar constant are honoured."""
    announce("fused group, several results")
    r = np.random.default_rng(8)
    x = r.standard_normal((4, 33, 17)).astype(np.float32)
    y = r.standard_normal((4, 33, 17)).astype(np.float32)
    row = r.standard_normal((17,)).astype(np.float32)

    def build(b):
        a, c = b.arg("x", x.shape), b.arg("y", y.shape)
        two = b.const("two", np.full((1,), 2.0, np.float32))
        d = b.sub(two, a, name="d")                       # scalar on the left
        e = b.div(d, two, name="e")                       # scalar on the right
        f = b.mul(b.add(e, c, name="ec"), b.const("row", row), name="f")   # row broadcast
        g = b.tanh(b.mul(f, f, name="ff"), name="g")      # the same value twice
        h = b.max(g, a, name="h")
        b.output(e, "e")
        b.output(g, "g")
        b.output(h, "h")

    got, steps = run_with_steps(build, {"x": x, "y": y})
    want = run_ref(build, {"x": x, "y": y})
    check(got, want, 1e-5)
    assert len(fused(steps)) == 1 and not [s for s in steps if s.startswith(("unary:", "binary:"))], steps


def test_group_results_feed_other_operators():
    """A group in front of and behind operators that are not element-wise."""
    announce("fused group between other operators")
    r = np.random.default_rng(9)
    x = r.standard_normal((6, 40)).astype(np.float32)
    w = (r.standard_normal((40, 24)) * 0.2).astype(np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        pre = b.tanh(b.mul(a, b.const("k", np.full((1,), 0.5, np.float32)), name="half"), name="pre")
        m = b.gemm(pre, b.const("w", w), name="mm")
        post = b.exp(b.neg(b.abs(m, name="abs"), name="neg"), name="post")
        b.output(b.softmax(post, -1, name="sm"), "sm")
        b.output(pre, "pre")

    got, steps = run_with_steps(build, {"x": x})
    want = run_ref(build, {"x": x})
    check(got, want, 1e-4)
    assert len(fused(steps)) >= 1, steps


def test_shapes_left_to_the_ordinary_path():
    """Rank-4 values (channels-last on the device, fused into convolution
    epilogues) and single operators stay as they were."""
    announce("fused group: exclusions")
    r = np.random.default_rng(10)
    x = r.standard_normal((2, 8, 6, 6)).astype(np.float32)
    v = r.standard_normal((5, 9)).astype(np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        b.output(b.sigmoid(b.neg(a, name="n4"), name="s4"), "s4")
        c = b.arg("v", v.shape)
        b.output(b.tanh(c, name="single"), "single")

    got, steps = run_with_steps(build, {"x": x, "v": v})
    want = run_ref(build, {"x": x, "v": v})
    check(got, want, 1e-5)
    assert not fused(steps), steps


def test_broadcast_member_and_smaller_result_give_up_cleanly():
    """A result that leaves the group with a shape smaller than the group's
    iteration space cannot be stored by every thread: the planner falls back to
    separate launches, with the same values."""
    announce("fused group: fallback")
    r = np.random.default_rng(11)
    x = r.standard_normal((3, 20, 1)).astype(np.float32)
    y = r.standard_normal((3, 20, 16)).astype(np.float32)

    def build(b):
        a, c = b.arg("x", x.shape), b.arg("y", y.shape)
        s = b.sigmoid(a, name="s")            # [3,20,1], also an output
        b.output(s, "s")
        b.output(b.mul(c, s, name="m"), "m")   # [3,20,16]

    got, steps = run_with_steps(build, {"x": x, "y": y})
    want = run_ref(build, {"x": x, "y": y})
    check(got, want, 1e-5)
