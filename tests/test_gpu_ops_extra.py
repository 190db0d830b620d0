"""Parity of the wider operator surface: libodla_hip.so through the ODLA C ABI
against the CPU oracle on identical seeded inputs.  fp32 graphs within 1e-4 of
the largest expected magnitude (transcendentals: 2e-4 absolute where the
function is steep), fp16 storage 2e-2; integer, boolean and index results
bit-exact.
"""
import numpy as np
import pytest

from util import announce, max_rel_err, run_both

pytestmark = pytest.mark.gpu

F32_TOL = 1e-4


def rng(seed):
    return np.random.default_rng(seed)


def check(got, want, mode="fp32", tol=None):
    for k in want:
        g, w = got[k], want[k]
        assert g.shape == w.shape, (k, g.shape, w.shape)
        if w.dtype.kind in "biu":
            assert np.array_equal(g, w), k
        elif mode == "fp32":
            assert max_rel_err(g, w) <= (tol or F32_TOL), (k, max_rel_err(g, w))
        else:
            assert np.max(np.abs(g.astype(np.float64) - w)) <= 2e-2 * max(1.0, float(np.max(np.abs(w)))), k


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_unary_family(mode):
    announce("extra unary %s" % mode)
    r = rng(101)
    x = (r.standard_normal((3, 5, 37)) * 2).astype(np.float32)
    u = (r.random((3, 5, 37)) * 1.8 - 0.9).astype(np.float32)   # (-0.9, 0.9)
    g = (r.random((3, 5, 37)) * 4 + 1.05).astype(np.float32)    # > 1

    def build(b):
        a, un, ge = b.arg("x", x.shape), b.arg("u", u.shape), b.arg("g", g.shape)
        for name in ("ceil", "floor", "sign", "sin", "cos", "atan", "sinh", "cosh", "asinh", "softplus", "softsign"):
            b.output(getattr(b, name)(a, name=name), name)
        for name in ("tan", "asin", "acos", "atanh"):
            b.output(getattr(b, name)(un, name=name), name)
        b.output(b.acosh(ge, name="acosh"), "acosh")
        b.output(b.reciprocal(ge, name="reciprocal"), "reciprocal")
        b.output(b.elu(a, 0.7, name="elu"), "elu")
        b.output(b.selu(a, 1.6732632, 1.050701, name="selu"), "selu")
        b.output(b.celu(a, 1.3, name="celu"), "celu")
        b.output(b.hard_sigmoid(a, 0.2, 0.5, name="hsig"), "hsig")
        b.output(b.thresholded_relu(a, 0.8, name="trelu"), "trelu")
        b.output(b.shrink(a, 0.3, 0.6, name="shrink"), "shrink")

    got, want = run_both(build, {"x": x, "u": u, "g": g}, fp16=(mode == "fp16"))
    if mode == "fp16":
        # ceil / floor / sign / threshold decisions are taken on the fp16-rounded input
        xr = x.astype(np.float16).astype(np.float32)
        for k, f in (("ceil", np.ceil), ("floor", np.floor), ("sign", np.sign)):
            assert np.array_equal(got.pop(k), f(xr)), k
            want.pop(k)
        for k in ("trelu", "shrink"):
            got.pop(k), want.pop(k)
    check(got, want, mode)


def test_integer_arithmetic_and_mod():
    announce("integer binary ops")
    r = rng(102)
    a = r.integers(-50, 50, (4, 1, 9)).astype(np.int32)
    c = r.integers(1, 9, (6, 9)).astype(np.int32) * r.choice([-1, 1], (6, 9)).astype(np.int32)
    p = r.integers(0, 4, (6, 9)).astype(np.int32)
    l64 = r.integers(-2 ** 40, 2 ** 40, (5, 3)).astype(np.int64)
    r64 = r.integers(1, 2 ** 20, (3,)).astype(np.int64)
    fa = (r.standard_normal((4, 6, 9)) * 5).astype(np.float32)
    fb = ((r.random((6, 9)) + 0.5) * r.choice([-1, 1], (6, 9))).astype(np.float32)

    def build(b):
        va, vc, vp = b.arg("a", a.shape, np.int32), b.arg("c", c.shape, np.int32), b.arg("p", p.shape, np.int32)
        v64, w64 = b.arg("l64", l64.shape, np.int64), b.arg("r64", r64.shape, np.int64)
        vf, wf = b.arg("fa", fa.shape), b.arg("fb", fb.shape)
        b.output(b.add(va, vc, name="add"), "add")
        b.output(b.sub(va, vc, name="sub"), "sub")
        b.output(b.mul(va, vc, name="mul"), "mul")
        b.output(b.max(va, vc, name="max"), "max")
        b.output(b.min(va, vc, name="min"), "min")
        b.output(b.mod(va, vc, name="mod"), "mod")
        b.output(b.mod(va, vc, fmod=True, name="fmod"), "fmod")
        b.output(b.pow(va, vp, name="ipow"), "ipow")
        b.output(b.squared_difference(va, vc, name="sqd"), "sqd")
        b.output(b.add(v64, w64, name="add64"), "add64")
        b.output(b.mod(v64, w64, name="mod64"), "mod64")
        b.output(b.mod(vf, wf, name="modf"), "modf")
        b.output(b.mod(vf, wf, fmod=True, name="fmodf"), "fmodf")

    got, want = run_both(build, {"a": a, "c": c, "p": p, "l64": l64, "r64": r64, "fa": fa, "fb": fb})
    for k in ("modf", "fmodf"):
        assert np.array_equal(got.pop(k), want.pop(k)), k   # same float operations in the same order
    check(got, want)


def test_float_binary_extras():
    announce("pow / prelu / squared difference / mean")
    r = rng(103)
    base = (r.random((2, 5, 7)) * 3 + 0.1).astype(np.float32)
    ex = (r.standard_normal((5, 7)) * 1.5).astype(np.float32)
    x = r.standard_normal((2, 6, 5, 7)).astype(np.float32)
    slope = r.random((6, 1, 1)).astype(np.float32)

    def build(b):
        vb, ve, vx = b.arg("base", base.shape), b.arg("ex", ex.shape), b.arg("x", x.shape)
        b.output(b.pow(vb, ve, name="pow"), "pow")
        b.output(b.prelu(vx, b.const("slope", slope), name="prelu"), "prelu")
        b.output(b.squared_difference(vb, ve, name="sqd"), "sqd")
        b.output(b.mean([vb, b.relu(vb), b.neg(vb)], name="mean"), "mean")

    got, want = run_both(build, {"base": base, "ex": ex, "x": x})
    check(got, want)


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_compare_logic_select(mode):
    announce("compare / logic / select %s" % mode)
    r = rng(104)
    a = r.integers(-3, 4, (3, 4, 11)).astype(np.float32)    # small integers: exact in fp16, many ties
    c = r.integers(-3, 4, (4, 11)).astype(np.float32)
    ia = r.integers(-3, 4, (3, 4, 11)).astype(np.int32)
    ic = r.integers(-3, 4, (11,)).astype(np.int32)
    special = np.array([0.0, np.inf, -np.inf, np.nan, 1.0, -2.0, np.inf, np.nan], np.float32)

    def build(b):
        va, vc = b.arg("a", a.shape), b.arg("c", c.shape)
        wa, wc = b.arg("ia", ia.shape, np.int32), b.arg("ic", ic.shape, np.int32)
        sp = b.arg("special", special.shape)
        cmp = {}
        for name in ("equal", "not_equal", "less", "less_equal", "greater", "greater_equal"):
            cmp[name] = getattr(b, name)(va, vc, name=name)
            b.output(cmp[name], name)
            b.output(getattr(b, name)(wa, wc, name="i" + name), "i" + name)
        b.output(b.logical_and(cmp["less"], cmp["not_equal"], name="and"), "and")
        b.output(b.logical_or(cmp["less"], cmp["equal"], name="or"), "or")
        b.output(b.logical_xor(cmp["less_equal"], cmp["greater_equal"], name="xor"), "xor")
        b.output(b.logical_not(cmp["equal"], name="not"), "not")
        b.output(b.select(cmp["greater"], va, vc, name="sel"), "sel")
        b.output(b.select(cmp["greater"], wa, b.sub(wa, wc, name="wd"), name="isel"), "isel")
        b.output(b.isnan(sp, name="isnan"), "isnan")
        b.output(b.isinf(sp, True, True, name="isinf"), "isinf")
        b.output(b.isinf(sp, True, False, name="isinf_pos"), "isinf_pos")
        b.output(b.isinf(sp, False, True, name="isinf_neg"), "isinf_neg")

    got, want = run_both(build, {"a": a, "c": c, "ia": ia, "ic": ic, "special": special}, fp16=(mode == "fp16"))
    for k in want:
        assert got[k].dtype == want[k].dtype, k
        assert np.array_equal(got[k], want[k]), k


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_reduce_family(mode):
    announce("extra reductions %s" % mode)
    r = rng(105)
    x = (r.random((3, 6, 40)) + 0.25).astype(np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        for axes, keep in (([2], True), ([1], False), ([1, 2], True), ([0], False)):
            tag = "_%s_%d" % ("".join(str(v) for v in axes), keep)
            b.output(b.reduce_min(a, axes, keep, name="min" + tag), "min" + tag)
            b.output(b.reduce_prod(a, axes, keep, name="prod" + tag), "prod" + tag)
            b.output(b.reduce_sum_square(a, axes, keep, name="ssq" + tag), "ssq" + tag)
            b.output(b.reduce_l1(a, axes, keep, 0.25, name="l1" + tag), "l1" + tag)
            b.output(b.reduce_l2(a, axes, keep, 0.5, name="l2" + tag), "l2" + tag)
            b.output(b.reduce_log_sum(a, axes, keep, name="ls" + tag), "ls" + tag)
            b.output(b.reduce_log_sum_exp(a, axes, keep, name="lse" + tag), "lse" + tag)

    got, want = run_both(build, {"x": x}, fp16=(mode == "fp16"))
    if mode == "fp16":
        for k in list(want):   # long products underflow / lose precision in half storage
            if k.startswith("prod"):
                got.pop(k), want.pop(k)
    check(got, want, mode)


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_argmax_argmin_topk(mode):
    announce("argmax / argmin / topk %s" % mode)
    r = rng(106)
    ties = r.integers(0, 5, (4, 9, 6)).astype(np.float32)
    distinct = r.permutation(4 * 300 * 3).reshape(4, 300, 3).astype(np.float32) / 8.0   # exact in fp16 up to 2048/8
    if mode == "fp16":
        distinct = r.permutation(2 * 300 * 3).reshape(2, 300, 3).astype(np.float32)
    rows = r.standard_normal((5, 1000)).astype(np.float32)

    def build(b):
        t, d, w = b.arg("ties", ties.shape), b.arg("distinct", distinct.shape), b.arg("rows", rows.shape)
        for axis in (0, 1, 2):
            for last in (False, True):
                tag = "_%d_%d" % (axis, last)
                b.output(b.argmax(t, axis, True, last, name="amax" + tag), "amax" + tag)
                b.output(b.argmin(t, axis, False, last, np.int64, name="amin" + tag), "amin" + tag)
        for largest in (True, False):
            v, i = b.topk(d, 7, 1, largest, names=("tv%d" % largest, "ti%d" % largest))
            b.output(v, "tv%d" % largest)
            b.output(i, "ti%d" % largest)
            v, i = b.topk(t, 9, 1, largest, np.int64, names=("sv%d" % largest, "si%d" % largest))   # full sort with ties
            b.output(v, "sv%d" % largest)
            b.output(i, "si%d" % largest)
        if mode == "fp32":
            v, i = b.topk(w, 20, 1, True, names=("rv", "ri"))
            b.output(v, "rv")
            b.output(i, "ri")

    got, want = run_both(build, {"ties": ties, "distinct": distinct, "rows": rows}, fp16=(mode == "fp16"))
    for k in want:
        assert got[k].dtype == want[k].dtype, k
        assert np.array_equal(got[k], want[k]), k


def test_pad_tile_broadcast_squeeze_stack():
    announce("pad / tile / broadcast / squeeze / stack")
    r = rng(107)
    x = r.standard_normal((2, 3, 5, 8)).astype(np.float32)
    idx = r.integers(0, 100, (3, 4)).astype(np.int32)

    def build(b):
        a, i = b.arg("x", x.shape), b.arg("idx", idx.shape, np.int32)
        b.output(b.pad(a, [0, 1, 2, 3], [1, 0, 1, 5], name="pad"), "pad")
        b.output(b.pad(a, [0, 0, 1, 1], [0, 0, 1, 1], name="pad_hw"), "pad_hw")
        b.output(b.pad(i, [1, 2], [0, 1], name="ipad"), "ipad")
        b.output(b.tile(a, [2, 1, 3, 2], name="tile"), "tile")
        b.output(b.tile(i, [3, 2], name="itile"), "itile")
        row = b.slice(a, [0, 0, 0, 0], [2, 1, 5, 8], name="row")
        b.output(b.broadcast_to(row, (2, 4, 5, 8), name="bcast"), "bcast")
        b.output(b.broadcast_to(i, (2, 3, 4), name="ibcast"), "ibcast")
        b.output(b.squeeze(row, [1], name="squeeze"), "squeeze")
        b.output(b.stack([a, b.relu(a), b.neg(a)], 2, name="stack"), "stack")
        b.output(b.stack([i, i], 0, name="istack"), "istack")

    got, want = run_both(build, {"x": x, "idx": idx})
    for k in want:
        assert got[k].shape == want[k].shape, k
        assert np.array_equal(got[k], want[k]), k


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_lrn_instance_norm(mode):
    announce("lrn / instance norm %s" % mode)
    r = rng(108)
    x = r.standard_normal((2, 9, 13, 11)).astype(np.float32)
    big = r.standard_normal((1, 3, 70, 64)).astype(np.float32)   # rows longer than one pass of the workgroup
    g, o = (r.random(9) + 0.5).astype(np.float32), r.standard_normal(9).astype(np.float32)

    def build(b):
        a, c = b.arg("x", x.shape), b.arg("big", big.shape)
        b.output(b.lrn(a, 5, 1e-2, 0.75, 1.5, name="lrn5"), "lrn5")
        b.output(b.lrn(a, 3, 0.5, 0.5, 1.0, name="lrn3"), "lrn3")
        b.output(b.instance_norm(a, 1e-5, b.const("g", g), b.const("o", o), name="inorm"), "inorm")
        b.output(b.instance_norm(c, 1e-3, None, None, 2.0, -1.0, name="inorm_scalar"), "inorm_scalar")

    got, want = run_both(build, {"x": x, "big": big}, fp16=(mode == "fp16"))
    check(got, want, mode)


DECONV_CASES = [
    # N, Cin, H, W, Cout/group, k, stride, pad, group, output padding
    (2, 4, 5, 4, 3, 3, 2, 1, 1, 0),
    (2, 4, 5, 4, 3, 3, 2, 1, 2, 1),
    (1, 6, 7, 7, 2, 4, 2, 1, 3, 0),
    (3, 3, 6, 5, 5, 2, 1, 0, 1, 0),
    (1, 2, 4, 4, 2, 5, 3, 2, 1, 2),
    (2, 64, 14, 14, 32, 2, 2, 0, 1, 0),     # upsampling block of a decoder
    (1, 32, 16, 16, 128, 4, 2, 1, 1, 0),
]


@pytest.mark.parametrize("case", DECONV_CASES)
@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_deconv(case, mode):
    announce("deconv %s %s" % (case, mode))
    N, Cin, H, W, Og, k, s, p, grp, op = case
    r = rng(109)
    x = r.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (r.standard_normal((Cin, Og, k, k)) / np.sqrt(Cin * k * k / (s * s))).astype(np.float32)
    bias = r.standard_normal(Og * grp).astype(np.float32)
    out_hw = None
    if op:
        out_hw = ((H - 1) * s - 2 * p + k + op, (W - 1) * s - 2 * p + k + op)

    def build(b):
        a = b.arg("x", x.shape)
        y = b.deconv(a, b.const("w", w), b.const("bias", bias), (s, s), (p, p, p, p), grp, out_hw, name="y")
        b.output(y, "y")
        b.output(b.relu(b.deconv(a, b.const("w2", w), None, (s, s), (p, p, p, p), grp, out_hw, name="y2"), name="y2r"), "y2r")

    got, want = run_both(build, {"x": x}, fp16=(mode == "fp16"))
    check(got, want, mode)


@pytest.mark.parametrize("case", [(2, 32, 14, 32, 32, 3, 1, 1), (1, 24, 9, 48, 12, 3, 2, 1), (2, 12, 8, 6, 3, 1, 1, 0)])
@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_grouped_conv_few_channels_per_group(case, mode):
    """Depthwise and narrow groups (fewer channels per group than one 16-byte K vector)."""
    announce("grouped conv %s %s" % (case, mode))
    N, C, H, O, G, k, s, p = case
    r = rng(110)
    x = r.standard_normal((N, C, H, H)).astype(np.float32)
    w = (r.standard_normal((O, C // G, k, k)) / np.sqrt(C // G * k * k)).astype(np.float32)
    bias = r.standard_normal(O).astype(np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        y = b.conv(a, b.const("w", w), b.const("b", bias), (s, s), (p, p, p, p), (1, 1), G, name="y")
        b.output(b.relu(y, name="yr"), "yr")

    got, want = run_both(build, {"x": x}, fp16=(mode == "fp16"))
    check(got, want, mode)
