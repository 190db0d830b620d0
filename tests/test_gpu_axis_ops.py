"""GatherElements, CumSum, Hardmax, Compress and Shift: libodla_hip.so through the ODLA C
ABI against the CPU oracle on identical seeded inputs, and on the operator examples the
reference's tests name.  Index, integer and one-hot results bit-exact; CumSum in fp32
within 1e-4 of the largest expected magnitude (bit-exact where one thread adds a line in
the oracle's order), fp16 storage 2e-2.
"""
import numpy as np
import pytest

from util import announce, max_rel_err, run_both, run_hip

pytestmark = pytest.mark.gpu


def rng(seed):
    return np.random.default_rng(seed)


def test_operator_examples():
    announce("axis ops: operator examples")
    d2 = np.array([[1, 2], [3, 4]], np.float32)
    d3 = np.arange(1, 10, dtype=np.float32).reshape(3, 3)
    x5 = np.arange(1, 6, dtype=np.float32)
    hm = np.array([[3, 0, 1, 2], [2, 5, 1, 0], [0, 1, 3, 2], [0, 1, 2, 3]], np.float32)
    cx = np.array([[1, 2], [3, 4], [5, 6]], np.float32)
    sx, sy = np.array([16, 4, 1], np.uint8), np.array([1, 2, 3], np.uint8)

    def build(b):
        v2, v3, v5 = b.arg("d2", d2.shape), b.arg("d3", d3.shape), b.arg("x5", x5.shape)
        b.output(b.gather_elements(v2, b.const("i0", np.array([[0, 0], [1, 0]], np.int64)), 1, name="ge0"), "ge0")
        b.output(b.gather_elements(v3, b.const("i1", np.array([[1, 2, 0], [2, 0, 0]], np.int32)), 0, name="ge1"), "ge1")
        b.output(b.gather_elements(v3, b.const("i2", np.array([[-1, -2, 0], [-2, 0, 0]], np.int64)), 0, name="ge2"), "ge2")
        b.output(b.cumsum(v5, 0, name="cs"), "cs")
        b.output(b.cumsum(v5, 0, exclusive=True, name="cse"), "cse")
        b.output(b.cumsum(v5, 0, reverse=True, name="csr"), "csr")
        b.output(b.cumsum(v5, 0, exclusive=True, reverse=True, name="cser"), "cser")
        b.output(b.hardmax(b.arg("hm", hm.shape), -1, name="hmx"), "hmx")
        b.output(b.hardmax(b.const("tie", np.array([[3, 3, 3, 1]], np.float32)), 1, name="tiex"), "tiex")
        vc = b.arg("cx", cx.shape)
        b.output(b.compress(vc, b.const("c0", np.array([0, 1, 1], np.bool_)), 0, (3, 2), name="cp0"), "cp0")
        b.output(b.compress(vc, b.const("c1", np.array([0, 1], np.bool_)), 1, (3, 2), name="cp1"), "cp1")
        b.output(b.compress(vc, b.const("c2", np.array([0, 1, 0, 0, 1], np.bool_)), None, (5,), name="cp2"), "cp2")
        vs, va = b.arg("sx", sx.shape, np.uint8), b.arg("sy", sy.shape, np.uint8)
        b.output(b.shift(vs, va, True, name="shl"), "shl")
        b.output(b.shift(vs, va, False, name="shr"), "shr")

    got = run_hip(build, {"d2": d2, "d3": d3, "x5": x5, "hm": hm, "cx": cx, "sx": sx, "sy": sy})
    assert np.array_equal(got["ge0"], [[1, 1], [4, 3]])
    assert np.array_equal(got["ge1"], [[4, 8, 3], [7, 2, 3]])
    assert np.array_equal(got["ge2"], [[7, 5, 3], [4, 2, 3]])
    assert np.array_equal(got["cs"], [1, 3, 6, 10, 15])
    assert np.array_equal(got["cse"], [0, 1, 3, 6, 10])
    assert np.array_equal(got["csr"], [15, 14, 12, 9, 5])
    assert np.array_equal(got["cser"], [14, 12, 9, 5, 0])
    assert np.array_equal(got["hmx"], np.eye(4, dtype=np.float32))
    assert np.array_equal(got["tiex"], [[1, 0, 0, 0]])
    assert np.array_equal(got["cp0"].reshape(-1), [3, 4, 5, 6, 0, 0])
    assert np.array_equal(got["cp1"].reshape(-1), [2, 4, 6, 0, 0, 0])
    assert np.array_equal(got["cp2"], [2, 5, 0, 0, 0])
    assert np.array_equal(got["shl"], [32, 16, 8])
    assert np.array_equal(got["shr"], [8, 1, 0])


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_gather_elements_and_hardmax(mode):
    announce("gather elements / hardmax %s" % mode)
    r = rng(301)
    d = r.standard_normal((5, 37, 9)).astype(np.float32)
    di = r.integers(-1000, 1000, (6, 11)).astype(np.int32)
    idx = {ax: r.integers(-d.shape[ax], d.shape[ax], [13 if i == ax else n for i, n in enumerate(d.shape)]) for ax in range(3)}
    small = r.integers(0, 37, (3, 50, 9)).astype(np.int32)      # fewer leading slices than the input
    ii = r.integers(-11, 11, (6, 4)).astype(np.int64)
    hx = np.round(r.standard_normal((4, 19, 33)) * 2).astype(np.float32)   # rounded: equal maxima occur

    def build(b):
        v = b.arg("d", d.shape)
        for ax in range(3):
            b.output(b.gather_elements(v, b.const("idx%d" % ax, idx[ax].astype(np.int64 if ax else np.int32)), ax, name="g%d" % ax), "g%d" % ax)
        b.output(b.gather_elements(v, b.arg("small", small.shape, np.int32), 1, name="gs"), "gs")
        b.output(b.gather_elements(b.arg("di", di.shape, np.int32), b.const("ii", ii), -1, name="gi"), "gi")
        h = b.arg("hx", hx.shape)
        for ax in (0, 1, 2, -2):
            b.output(b.hardmax(h, ax, name="h%d" % (ax % 3 + (3 if ax < 0 else 0))), "h%d" % (ax % 3 + (3 if ax < 0 else 0)))

    got, want = run_both(build, {"d": d, "small": small, "di": di, "hx": hx}, fp16=mode == "fp16")
    for k in want:
        if k[0] == "h":
            if mode == "fp32":
                assert np.array_equal(got[k], want[k]), k
            else:   # operands rounded to fp16 may create new ties; the result is still one-hot at a maximum
                ax = {"h0": 0, "h1": 1, "h2": 2, "h4": 1}[k]
                assert np.array_equal(got[k].sum(axis=ax), np.ones_like(got[k].sum(axis=ax))), k
                h16 = hx.astype(np.float16).astype(np.float32)
                assert np.array_equal(np.max(h16, axis=ax), np.sum(got[k] * h16, axis=ax)), k
        elif k == "gi" or mode == "fp32":
            assert np.array_equal(got[k], want[k]), k
        else:
            assert np.array_equal(got[k], want[k].astype(np.float16).astype(np.float32)), k


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_cumsum(mode):
    announce("cumsum %s" % mode)
    r = rng(302)
    x = r.standard_normal((3, 70, 40)).astype(np.float32)
    long_rows = r.standard_normal((5, 3000)).astype(np.float32)   # contiguous axis: one wavefront per line

    def build(b):
        v, w = b.arg("x", x.shape), b.arg("long", long_rows.shape)
        for ax in range(3):
            for ex in (0, 1):
                for rv in (0, 1):
                    n = "c%d%d%d" % (ax, ex, rv)
                    b.output(b.cumsum(v, ax, bool(ex), bool(rv), name=n), n)
        b.output(b.cumsum(w, 1, name="l"), "l")
        b.output(b.cumsum(w, -1, True, True, name="ler"), "ler")
        b.output(b.cumsum(w, 0, name="l0"), "l0")

    got, want = run_both(build, {"x": x, "long": long_rows}, fp16=mode == "fp16")
    for k in want:
        if mode == "fp32":
            if k not in ("l", "ler"):
                assert np.array_equal(got[k], want[k]), k       # the oracle's order of additions
            assert max_rel_err(got[k], want[k]) <= 1e-4, (k, max_rel_err(got[k], want[k]))
        else:
            # fp16 storage of sums of up to 3000 values of magnitude 1: two units of the last place of the largest sum
            scale = max(1.0, float(np.max(np.abs(want[k]))))
            assert np.max(np.abs(got[k] - want[k])) <= 2e-2 * scale, k


def test_compress_and_shift():
    announce("compress / shift")
    r = rng(303)
    x = r.standard_normal((6, 300, 7)).astype(np.float32)
    xi = r.integers(-99, 99, (40, 5)).astype(np.int32)
    conds = {0: r.random(6) < 0.5, 1: r.random(300) < 0.3, 2: r.random(5) < 0.6}   # the last is shorter than its axis
    flat = r.random(xi.size) < 0.2
    none = np.zeros(300, np.bool_)
    u8 = r.integers(0, 256, (7, 33)).astype(np.uint8)
    s8 = r.integers(0, 10, (33,)).astype(np.uint8)
    u32 = r.integers(0, 2 ** 32, (50,), dtype=np.uint64).astype(np.uint32)
    s32 = r.integers(0, 35, (50,)).astype(np.uint32)
    u64 = r.integers(0, 2 ** 63, (50,), dtype=np.uint64) * np.uint64(2) + np.uint64(1)
    s64 = r.integers(0, 67, (50,)).astype(np.uint64)

    def build(b):
        v, vi = b.arg("x", x.shape), b.arg("xi", xi.shape, np.int32)
        for ax in range(3):
            b.output(b.compress(v, b.arg("cond%d" % ax, conds[ax].shape, np.bool_), ax, x.shape, name="p%d" % ax), "p%d" % ax)
        b.output(b.compress(v, b.const("none", none), 1, x.shape, name="pn"), "pn")
        b.output(b.compress(vi, b.const("flat", flat), None, (xi.size,), name="pf"), "pf")
        a8, b8 = b.arg("u8", u8.shape, np.uint8), b.arg("s8", s8.shape, np.uint8)
        a32, b32 = b.arg("u32", u32.shape, np.uint32), b.arg("s32", s32.shape, np.uint32)
        a64, b64 = b.arg("u64", u64.shape, np.uint64), b.arg("s64", s64.shape, np.uint64)
        for left in (True, False):
            t = "l" if left else "r"
            b.output(b.shift(a8, b8, left, name="s8" + t), "s8" + t)
            b.output(b.shift(a32, b32, left, name="s32" + t), "s32" + t)
            b.output(b.shift(a64, b64, left, name="s64" + t), "s64" + t)

    feeds = {"x": x, "xi": xi, "u8": u8, "s8": s8, "u32": u32, "s32": s32, "u64": u64, "s64": s64}
    feeds.update({"cond%d" % ax: conds[ax] for ax in range(3)})
    got, want = run_both(build, feeds)
    for k in want:
        assert got[k].dtype == want[k].dtype and np.array_equal(got[k], want[k]), k
    assert not np.any(got["pn"])
    kept = int(conds[1].sum())
    assert np.array_equal(got["p1"].reshape(-1)[:6 * kept * 7].reshape(6, kept, 7), x[:, conds[1], :])
