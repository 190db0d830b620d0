"""The HIP path on the committed golden vectors (tests/golden/sn_rt_vectors.npz:
inputs and outputs of the reference's own generic CPU kernels for Conv, MaxPool,
Gemm and Softmax), through the ODLA C ABI, without the oracle in between."""
import os

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, run_hip

pytestmark = pytest.mark.gpu

GOLD = np.load(os.path.join(entry.ROOT, "tests", "golden", "sn_rt_vectors.npz"))
TOL = 1e-4   # fp32 path: relative to the largest expected magnitude


def close(got, want):
    return np.max(np.abs(got - want)) <= TOL * max(float(np.max(np.abs(want))), 1e-30)


@pytest.mark.parametrize("i", range(5))
def test_conv_golden(i):
    announce("golden conv %d" % i)
    x, w, want = GOLD["conv%d_x" % i], GOLD["conv%d_w" % i], GOLD["conv%d_y" % i]
    s, p = (int(v) for v in GOLD["conv%d_attr" % i])

    def build(b):
        b.output(b.conv(b.arg("x", x.shape), b.const("w", w), None, (s, s), (p, p, p, p), name="y"), "y")

    got = run_hip(build, {"x": x})["y"]
    assert got.shape == want.shape and close(got, want)


@pytest.mark.parametrize("i", range(3))
def test_maxpool_golden(i):
    announce("golden maxpool %d" % i)
    x, want = GOLD["pool%d_x" % i], GOLD["pool%d_y" % i]
    k, s, p = (int(v) for v in GOLD["pool%d_attr" % i])

    def build(b):
        b.output(b.maxpool(b.arg("x", x.shape), (k, k), (s, s), (p, p, p, p), name="y"), "y")

    got = run_hip(build, {"x": x})["y"]
    assert np.array_equal(got, want)


@pytest.mark.parametrize("i", range(3))
def test_gemm_golden(i):
    announce("golden gemm %d" % i)
    a, bm, c, want = GOLD["gemm%d_a" % i], GOLD["gemm%d_b" % i], GOLD["gemm%d_c" % i], GOLD["gemm%d_y" % i]
    ta, tb, alpha, beta = GOLD["gemm%d_attr" % i]

    def build(b):
        y = b.gemm(b.arg("a", a.shape), b.const("b", bm), b.const("c", c.reshape(1, -1)), bool(ta), bool(tb),
                   float(alpha), float(beta), name="y")
        b.output(y, "y")

    got = run_hip(build, {"a": a})["y"]
    assert got.shape == want.shape and close(got, want)


@pytest.mark.parametrize("i", range(2))
def test_softmax_golden(i):
    announce("golden softmax %d" % i)
    x, want = GOLD["softmax%d_x" % i], GOLD["softmax%d_y" % i]

    def build(b):
        b.output(b.softmax(b.arg("x", x.shape), -1, name="y"), "y")

    got = run_hip(build, {"x": x})["y"]
    assert np.max(np.abs(got - want)) <= 1e-6
