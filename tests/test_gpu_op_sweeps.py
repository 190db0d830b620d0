"""Seeded random sweeps of the non-convolution operators against the oracle.  Every
rank-4 case runs twice: on a graph argument (row-major in the plan) and behind a 1x1
convolution, whose result the plan keeps channels-last - the operator then has to
honour a layout it did not choose.  fp32 results within 1e-4 of the largest expected
magnitude, fp16 plans within 2e-2; pure data movement is exact."""
import os
import tempfile
import zlib

import numpy as np
import pytest

from util import announce, max_rel_err, run_hip, run_hip_stored, run_ref

pytestmark = pytest.mark.gpu

# ODLA_SWEEP_SEED=<n> shifts every seed below: other random cases, same code (default 0)
SEED0 = int(__import__("os").environ.get("ODLA_SWEEP_SEED", "0"))


def source(b, name, shape, behind_conv, seed, mix=0.05):
    """A value of `shape`: the argument itself, or a 1x1 convolution of it (identity
    weights plus a little mixing), which the planner stores channels-last.  The
    weights depend on `seed` alone: the oracle and the library build the same graph."""
    v = b.arg(name, shape)
    if not behind_conv or len(shape) != 4:
        return v
    C = shape[1]
    r = np.random.default_rng(seed)
    w = (np.eye(C, dtype=np.float32) + mix * r.standard_normal((C, C)).astype(np.float32)).reshape(C, C, 1, 1)
    return b.conv(v, b.const(name + ".w", w), None, (1, 1), (0, 0, 0, 0), name=name + ".conv")


def check(build, feeds, exact=False, modes=("fp32", "fp16"), tag=""):
    want = run_ref(build, feeds)
    for mode in modes:
        got = run_hip(build, feeds, fp16=(mode == "fp16"))
        if zlib.crc32(tag.encode()) % 4 == 0:
            # every fourth case also goes through a stored file: same bits expected
            with tempfile.TemporaryDirectory() as d:
                again = run_hip_stored(build, feeds, os.path.join(d, "case.odla"), fp16=(mode == "fp16"))
            for k in got:
                assert np.array_equal(again[k], got[k], equal_nan=True), (tag, mode, k, "stored")
        for k in want:
            assert got[k].shape == want[k].shape, (tag, mode, k, got[k].shape, want[k].shape)
            if want[k].dtype.kind in "iub":
                assert np.array_equal(got[k], want[k]), (tag, mode, k)
            elif mode == "fp32":
                if exact:
                    assert np.array_equal(got[k], want[k]), (tag, mode, k)
                else:
                    assert max_rel_err(got[k], want[k]) <= 1e-4, (tag, mode, k)
            else:
                scale = max(1.0, float(np.max(np.abs(want[k]))))
                assert float(np.max(np.abs(got[k] - want[k]))) <= 2e-2 * scale, (tag, mode, k)


def rand_shape4(r):
    return (int(r.integers(1, 4)), int(r.choice([3, 8, 16, 24, 40])), int(r.integers(3, 12)), int(r.integers(3, 12)))


@pytest.mark.parametrize("behind_conv", [False, True])
def test_movement_sweep(behind_conv):
    r = np.random.default_rng(SEED0 + 31 + behind_conv)
    for i in range(40):
        shape = rand_shape4(r)
        kind = str(r.choice(["transpose", "slice", "concat", "pad", "tile", "resize", "reshape_transpose", "strided_slice"]))
        tag = "move %s #%d %s conv=%s" % (kind, i, shape, behind_conv)
        announce(tag)
        wr = 1000 + i
        perm = tuple(int(v) for v in r.permutation(4))
        start = [int(r.integers(0, d)) for d in shape]
        end = [int(r.integers(s + 1, d + 1)) for s, d in zip(start, shape)]
        step = [int(r.integers(1, 3)) for _ in shape]
        axis = int(r.integers(0, 4))
        front = [int(r.integers(0, 3)) for _ in shape]
        back = [int(r.integers(0, 3)) for _ in shape]
        rep = [int(r.integers(1, 3)) for _ in shape]
        up = (shape[2] * int(r.integers(1, 4)), shape[3] * int(r.integers(1, 4)))

        def build(b):
            x = source(b, "x", shape, behind_conv, wr)
            if kind == "transpose":
                y = b.transpose(x, perm, name="y")
            elif kind == "slice":
                y = b.slice(x, start, end, name="y")
            elif kind == "strided_slice":
                y = b.slice(x, start, end, step, name="y")
            elif kind == "concat":
                other = source(b, "x2", shape, behind_conv and axis != 1, wr + 500)
                y = b.concat([x, b.relu(other, name="o"), x], axis, name="y")
            elif kind == "pad":
                y = b.pad(x, front, back, name="y")
            elif kind == "tile":
                y = b.tile(x, rep, name="y")
            elif kind == "resize":
                y = b.resize_nearest(x, up, name="y")
            else:
                t = b.reshape(x, (shape[0], shape[1], shape[2] * shape[3]), name="r")
                y = b.transpose(t, (0, 2, 1), name="y")
            b.output(y, "y")

        x = r.standard_normal(shape).astype(np.float32)
        feeds = {"x": x}
        if kind == "concat":
            feeds["x2"] = r.standard_normal(shape).astype(np.float32)
        check(build, feeds, exact=not behind_conv, tag=tag)


@pytest.mark.parametrize("behind_conv", [False, True])
def test_reduction_and_normalisation_sweep(behind_conv):
    r = np.random.default_rng(SEED0 + 41 + behind_conv)
    kinds = ["reduce_mean", "reduce_sum", "reduce_max", "reduce_min", "reduce_sum_square", "reduce_log_sum_exp",
             "softmax", "log_softmax", "layernorm", "batchnorm", "maxpool", "avgpool", "argmax", "instance_norm", "lrn"]
    for i in range(60):
        shape = rand_shape4(r)
        kind = kinds[i % len(kinds)]
        tag = "reduce %s #%d %s conv=%s" % (kind, i, shape, behind_conv)
        announce(tag)
        wr = 2000 + i
        n_ax = int(r.integers(1, 4))
        axes = sorted(int(v) for v in r.choice(4, n_ax, replace=False))
        keep = bool(r.random() < 0.6)
        axis = int(r.integers(0, 4))
        C = shape[1]
        mean, var = r.standard_normal(C).astype(np.float32), (r.random(C) + 0.5).astype(np.float32)
        gam, bet = r.standard_normal(C).astype(np.float32), r.standard_normal(C).astype(np.float32)
        ln_axes = int(r.integers(1, 4))
        ln_shape = shape[4 - ln_axes:]
        lg, lb = r.standard_normal(ln_shape).astype(np.float32), r.standard_normal(ln_shape).astype(np.float32)
        win = (int(r.integers(1, min(4, shape[2]) + 1)), int(r.integers(1, min(4, shape[3]) + 1)))
        st = (int(r.integers(1, 3)), int(r.integers(1, 3)))
        pd = (int(r.integers(0, (win[0] + 1) // 2 + 0)), int(r.integers(0, (win[1] + 1) // 2 + 0)))
        pd = (min(pd[0], win[0] - 1), min(pd[1], win[1] - 1))
        pads = (pd[0], pd[1], pd[0], pd[1])
        incl = bool(r.random() < 0.5)

        def build(b):
            x = source(b, "x", shape, behind_conv, wr)
            if kind.startswith("reduce_"):
                y = getattr(b, kind)(x, axes, keep, name="y")
            elif kind == "softmax":
                y = b.softmax(x, axis, name="y")
            elif kind == "log_softmax":
                y = b.softmax(x, axis, log=True, name="y")
            elif kind == "layernorm":
                y = b.layernorm(x, ln_axes, 1e-5, b.const("g", lg), b.const("be", lb), name="y")
            elif kind == "batchnorm":
                y = b.batchnorm(x, b.const("m", mean), b.const("v", var), 1e-5, b.const("g", gam), b.const("be", bet), name="y")
            elif kind == "maxpool":
                y = b.maxpool(x, win, st, pads, name="y")
            elif kind == "avgpool":
                y = b.avgpool(x, win, st, pads, incl, name="y")
            elif kind == "argmax":
                y = b.argmax(x, axis, keep, name="y")
            elif kind == "instance_norm":
                y = b.instance_norm(x, 1e-5, b.const("g", gam), b.const("be", bet), name="y")
            else:
                y = b.lrn(x, 3, 1e-3, 0.75, 1.0, name="y")
            b.output(y, "y")

        x = r.standard_normal(shape).astype(np.float32)
        # arg-extreme results are compared exactly: keep the candidates apart (and, in
        # fp16 plans, representable, so that rounding cannot reorder them)
        modes = ("fp32", "fp16")
        if kind == "argmax":
            x = r.permutation(x.size).reshape(shape).astype(np.float32) / 8.0
            # k / 8 is exact in fp16 only up to k = 2048: beyond that rounding makes ties
            modes = ("fp32",) if behind_conv or x.size > 2048 else modes
        if kind in ("reduce_sum", "reduce_sum_square", "reduce_log_sum_exp"):
            modes = ("fp32",) if np.prod([shape[a] for a in axes]) > 512 else modes
        check(build, {"x": x}, tag=tag, modes=modes)


def test_gemm_sweep():
    r = np.random.default_rng(SEED0 + 51)
    for i in range(50):
        M, K, N = int(r.integers(1, 200)), int(r.choice([1, 7, 16, 64, 100, 256, 777])), int(r.choice([1, 5, 10, 64, 130, 256]))
        ta, tb = bool(r.random() < 0.3), bool(r.random() < 0.4)
        batch = () if r.random() < 0.6 else (int(r.integers(1, 5)),)
        if len(batch) and r.random() < 0.3:
            batch = batch + (int(r.integers(1, 4)),)
        const_b = bool(r.random() < 0.6) and not batch
        alpha = float(r.choice([1.0, 1.0, 0.5, -2.0]))
        bias_kind = str(r.choice(["none", "row", "full", "scalar"]))
        beta = float(r.choice([1.0, 1.0, 0.25]))
        tag = "gemm #%d M%d K%d N%d ta%d tb%d batch%s constB%d alpha%g beta%g bias=%s" % (i, M, K, N, ta, tb, batch, const_b, alpha, beta, bias_kind)
        announce(tag)
        a_shape = batch + ((K, M) if ta else (M, K))
        b_shape = batch + ((N, K) if tb else (K, N))
        A = r.standard_normal(a_shape).astype(np.float32)
        B = (r.standard_normal(b_shape) / np.sqrt(K)).astype(np.float32)
        Cb = {"none": None, "row": r.standard_normal((1, N)).astype(np.float32) if not batch else r.standard_normal((N,)).astype(np.float32),
              "full": r.standard_normal(batch + (M, N)).astype(np.float32), "scalar": r.standard_normal((1,)).astype(np.float32)}[bias_kind]

        def build(b):
            a = b.arg("a", a_shape)
            bb = b.const("b", B) if const_b else b.arg("b", b_shape)
            c = b.const("c", Cb) if Cb is not None else None
            b.output(b.gemm(a, bb, c, ta, tb, alpha, beta, name="y"), "y")

        feeds = {"a": A}
        if not const_b:
            feeds["b"] = B
        check(build, feeds, tag=tag)


def test_binary_broadcast_sweep():
    r = np.random.default_rng(SEED0 + 61)
    ops = ["add", "sub", "mul", "div", "max", "min", "pow", "squared_difference", "less", "equal"]
    for i in range(60):
        rank = int(r.integers(1, 5))
        full = tuple(int(r.integers(1, 9)) for _ in range(rank))
        def sub_shape():
            s = tuple(d if r.random() < 0.6 else 1 for d in full)
            cut = int(r.integers(0, rank))            # leading dimensions may be missing altogether
            return s[cut:] if r.random() < 0.4 else s
        sa, sb = sub_shape(), sub_shape()
        if r.random() < 0.5:
            sa = full
        op = ops[i % len(ops)]
        behind = len(sa) == 4 and r.random() < 0.5
        tag = "binary %s #%d %s %s conv=%s" % (op, i, sa, sb, behind)
        announce(tag)
        wr = 3000 + i
        const_rhs = bool(r.random() < 0.4)
        A = r.standard_normal(sa).astype(np.float32)
        B = r.standard_normal(sb).astype(np.float32)
        if op == "pow":
            A, B = np.abs(A) + 0.5, np.clip(B, -2, 2)
        if op == "div":
            B = np.where(np.abs(B) < 0.3, np.float32(0.7), B)
        if op == "equal":
            B = np.where(r.random(sb) < 0.5, np.broadcast_to(A, np.broadcast_shapes(sa, sb))[tuple(slice(0, d) for d in sb)] if False else B, B)

        def build(b):
            # pow needs a positive base: no mixing in the convolution in front of it
            x = source(b, "a", sa, behind, wr, mix=0.0 if op == "pow" else 0.05)
            y = b.const("b", B) if const_rhs else b.arg("b", sb)
            b.output(getattr(b, op)(x, y, name="y"), "y")

        try:
            want_shape = np.broadcast_shapes(sa, sb)
        except ValueError:
            continue
        # the reference aligns a lower-rank operand by sliding it along the other's
        # dimensions; keep to the cases where that coincides with numpy's rule
        if len(sa) != len(sb):
            lo, hi = (sa, sb) if len(sa) < len(sb) else (sb, sa)
            if any(hi[len(hi) - len(lo) + k] != lo[k] and lo[k] != 1 and hi[len(hi) - len(lo) + k] != 1 for k in range(len(lo))):
                continue
        feeds = {"a": A}
        if not const_rhs:
            feeds["b"] = B
        modes = ("fp32",) if op in ("less", "equal") and behind else ("fp32", "fp16")
        if op in ("less", "equal"):
            # comparisons of fp16-rounded operands may differ from fp32 ones: compare on representable data
            feeds = {k: v.astype(np.float16).astype(np.float32) for k, v in feeds.items()}
            B = B.astype(np.float16).astype(np.float32)
        check(build, feeds, tag=tag, modes=modes)
        assert tuple(want_shape) is not None


def test_gather_cast_sweep():
    r = np.random.default_rng(SEED0 + 71)
    for i in range(20):
        rank = int(r.integers(1, 4))
        shape = tuple(int(r.integers(2, 12)) for _ in range(rank))
        axis = int(r.integers(0, rank))
        ishape = tuple(int(r.integers(1, 6)) for _ in range(int(r.integers(1, 3))))
        idx = r.integers(0, shape[axis], ishape).astype(np.int64 if i % 2 else np.int32)
        tag = "gather #%d %s axis %d idx %s %s" % (i, shape, axis, ishape, idx.dtype)
        announce(tag)
        X = r.standard_normal(shape).astype(np.float32)
        const_table = bool(i % 3 == 0)

        def build(b):
            x = b.const("x", X) if const_table else b.arg("x", shape)
            ids = b.arg("i", ishape, idx.dtype)
            b.output(b.gather(x, ids, axis, name="y"), "y")

        feeds = {"i": idx}
        if not const_table:
            feeds["x"] = X
        check(build, feeds, exact=True, tag=tag, modes=("fp32",))


UNARY = {
    # name -> (call, input transform)
    "relu": (lambda b, x, n: b.relu(x, name=n), None), "sigmoid": (lambda b, x, n: b.sigmoid(x, name=n), None),
    "tanh": (lambda b, x, n: b.tanh(x, name=n), None), "exp": (lambda b, x, n: b.exp(x, name=n), None),
    "log": (lambda b, x, n: b.log(x, name=n), "pos"), "sqrt": (lambda b, x, n: b.sqrt(x, name=n), "pos"),
    "rsqrt": (lambda b, x, n: b.rsqrt(x, name=n), "pos"), "erf": (lambda b, x, n: b.erf(x, name=n), None),
    "abs": (lambda b, x, n: b.abs(x, name=n), None), "neg": (lambda b, x, n: b.neg(x, name=n), None),
    "reciprocal": (lambda b, x, n: b.reciprocal(x, name=n), "pos"),
    "sin": (lambda b, x, n: b.sin(x, name=n), None), "cos": (lambda b, x, n: b.cos(x, name=n), None),
    "atan": (lambda b, x, n: b.atan(x, name=n), None), "asin": (lambda b, x, n: b.asin(x, name=n), "unit"),
    "sinh": (lambda b, x, n: b.sinh(x, name=n), None), "asinh": (lambda b, x, n: b.asinh(x, name=n), None),
    "softplus": (lambda b, x, n: b.softplus(x, name=n), None), "softsign": (lambda b, x, n: b.softsign(x, name=n), None),
    "gelu": (lambda b, x, n: b.gelu(x, name=n), None), "gelu_tanh": (lambda b, x, n: b.gelu(x, True, name=n), None),
    "leaky": (lambda b, x, n: b.leaky_relu(x, 0.2, name=n), None), "clamp": (lambda b, x, n: b.clamp(x, -0.3, 0.8, name=n), None),
    "elu": (lambda b, x, n: b.elu(x, 1.3, name=n), None), "selu": (lambda b, x, n: b.selu(x, 1.67, 1.05, name=n), None),
    "celu": (lambda b, x, n: b.celu(x, 0.8, name=n), None),
    "hard_sigmoid": (lambda b, x, n: b.hard_sigmoid(x, 0.2, 0.5, name=n), None),
    "thresholded_relu": (lambda b, x, n: b.thresholded_relu(x, 0.4, name=n), "grid"),
    "shrink": (lambda b, x, n: b.shrink(x, 0.1, 0.5, name=n), "grid"),
    "ceil": (lambda b, x, n: b.ceil(x, name=n), "grid"), "floor": (lambda b, x, n: b.floor(x, name=n), "grid"),
    "round": (lambda b, x, n: b.round(x, name=n), "grid"), "sign": (lambda b, x, n: b.sign(x, name=n), "grid"),
}


@pytest.mark.parametrize("behind_conv", [False, True])
def test_unary_sweep(behind_conv):
    r = np.random.default_rng(SEED0 + 81 + behind_conv)
    for i, (name, (call, dom)) in enumerate(sorted(UNARY.items())):
        rank = 4 if behind_conv else int(r.integers(1, 5))
        shape = rand_shape4(r) if rank == 4 else tuple(int(r.integers(1, 40)) for _ in range(rank))
        tag = "unary %s %s conv=%s" % (name, shape, behind_conv)
        announce(tag)
        x = r.standard_normal(shape).astype(np.float32)
        if dom == "pos":
            x = np.abs(x) + 0.25
        elif dom == "unit":
            x = np.clip(x * 0.4, -0.95, 0.95)
        elif dom == "grid":
            # step functions: values a safe distance from every step, exact in fp16
            x = (np.round(x * 4) / 4 + 0.125).astype(np.float32)
        x = x.astype(np.float16).astype(np.float32) if dom is not None else x

        def build(b):
            # restricted domains survive only an identity convolution
            v = source(b, "x", shape, behind_conv, 4000 + i, mix=0.05 if dom is None else 0.0)
            b.output(call(b, v, "y"), "y")

        check(build, {"x": x.astype(np.float32)}, tag=tag)


def test_compare_select_logic_sweep():
    r = np.random.default_rng(SEED0 + 91)
    for i in range(30):
        rank = int(r.integers(1, 5))
        shape = tuple(int(r.integers(1, 10)) for _ in range(rank))
        bshape = tuple(d if r.random() < 0.6 else 1 for d in shape)
        tag = "select #%d %s %s" % (i, shape, bshape)
        announce(tag)
        A = (np.round(r.standard_normal(shape) * 2) / 2).astype(np.float32)
        B = (np.round(r.standard_normal(bshape) * 2) / 2).astype(np.float32)
        cmp = ["less", "less_equal", "greater", "greater_equal", "equal", "not_equal"][i % 6]
        logic = ["logical_and", "logical_or", "logical_xor"][i % 3]

        def build(b):
            a, bb = b.arg("a", shape), b.arg("b", bshape)
            c1 = getattr(b, cmp)(a, bb, name="c1")
            c2 = b.greater(a, b.const("z", np.zeros((1,), np.float32)), name="c2")
            m = getattr(b, logic)(c1, c2, name="m")
            b.output(c1, "c1")
            b.output(b.logical_not(m, name="nm"), "nm")
            b.output(b.select(m, a, b.neg(a, name="na"), name="sel"), "sel")

        check(build, {"a": A, "b": B}, exact=True, tag=tag, modes=("fp32", "fp16"))


def test_topk_stack_squeeze_sweep():
    r = np.random.default_rng(SEED0 + 101)
    for i in range(24):
        rank = int(r.integers(1, 4))
        shape = tuple(int(r.integers(2, 30)) for _ in range(rank))
        axis = int(r.integers(0, rank))
        k = int(r.integers(1, shape[axis] + 1))
        largest = bool(i % 2)
        tag = "topk #%d %s axis %d k %d largest %s" % (i, shape, axis, k, largest)
        announce(tag)
        X = r.permutation(int(np.prod(shape))).reshape(shape).astype(np.float32) / 4.0   # distinct, exact in fp16 up to 8k elements

        def build(b):
            x = b.arg("x", shape)
            v, idx = b.topk(x, k, axis, largest, np.int64 if i % 3 == 0 else np.int32, names=("v", "i"))
            b.output(v, "v")
            b.output(idx, "i")
            s = b.stack([x, b.neg(x, name="n")], int(r.integers(0, rank + 1)) if False else axis, name="s")
            b.output(s, "s")

        check(build, {"x": X}, exact=True, tag=tag, modes=("fp32",) if X.size > 2048 else ("fp32", "fp16"))


def test_deconv_sweep():
    r = np.random.default_rng(SEED0 + 111)
    for i in range(16):
        N, C, O = int(r.integers(1, 3)), int(r.choice([4, 8, 16])), int(r.choice([3, 8, 16]))
        H, W = int(r.integers(3, 9)), int(r.integers(3, 9))
        k = int(r.choice([2, 3, 4]))
        s = int(r.choice([1, 2]))
        p = int(r.integers(0, min(k - 1, 1) + 1))
        tag = "deconv #%d N%d C%d O%d %dx%d k%d s%d p%d" % (i, N, C, O, H, W, k, s, p)
        announce(tag)
        Wt = (r.standard_normal((C, O, k, k)) * np.sqrt(1.0 / (C * k * k))).astype(np.float32)
        bias = r.standard_normal(O).astype(np.float32) if i % 2 else None
        X = r.standard_normal((N, C, H, W)).astype(np.float32)

        def build(b):
            x = b.arg("x", X.shape)
            y = b.deconv(x, b.const("w", Wt), b.const("b", bias) if bias is not None else None, (s, s), (p, p, p, p), name="y")
            b.output(y, "y")

        check(build, {"x": X}, tag=tag)


def test_quantize_dequantize_sweep():
    r = np.random.default_rng(SEED0 + 121)
    for i in range(20):
        rank = int(r.integers(1, 5))
        shape = tuple(int(r.integers(1, 12)) for _ in range(rank))
        axis = int(r.integers(0, rank))
        per_axis = bool(i % 2)
        n = shape[axis] if per_axis else 1
        scale = (r.random(n) * 0.1 + 0.01).astype(np.float32)
        signed = bool(i % 3 == 0)
        zp = r.integers(-20, 20, n).astype(np.int8) if signed else r.integers(100, 150, n).astype(np.uint8)
        tag = "qdq #%d %s axis %d per_axis %s signed %s" % (i, shape, axis, per_axis, signed)
        announce(tag)
        X = (r.standard_normal(shape) * 3).astype(np.float32)

        def build(b):
            x = b.arg("x", shape)
            q = b.quantize(x, scale, zp, axis, signed, name="q")
            b.output(q, "q")
            b.output(b.dequantize(q, scale, zp, axis, name="d", zp_dtype=zp.dtype), "d")

        check(build, {"x": X}, tag=tag, modes=("fp32",))
