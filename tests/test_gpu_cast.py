"""odla_Cast and odla_BatchMatMul through the C ABI on the GPU.

odla_Cast is a oneDNN reorder in the reference
[ref: ODLA/platforms/dnnl/odla_dnnl_cast.cc:232-258]: float -> integer rounds to
nearest even and saturates, integer -> narrower integer saturates.  The expected
values are hand-listed (the same lists pin the oracle) or come from numpy's
IEEE conversions (fp16 round-to-nearest-even); random data goes through the
oracle.  Integer and bool results must be equal, floating-point results
bit-equal (a cast has no arithmetic to disagree on).
"""
import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, max_rel_err, run_both, run_hip

pytestmark = pytest.mark.gpu

TIES = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 2.4999, 126.5, 127.5, 300.0, -128.5, -129.5, -1000.0, 254.5, 255.5],
                np.float32)
TIES_WANT = {
    np.int8: [0, 2, 2, 0, -2, -2, 2, 126, 127, 127, -128, -128, -128, 127, 127],
    np.uint8: [0, 2, 2, 0, 0, 0, 2, 126, 128, 255, 0, 0, 0, 254, 255],
    np.int32: [0, 2, 2, 0, -2, -2, 2, 126, 128, 300, -128, -130, -1000, 254, 256],
    np.int64: [0, 2, 2, 0, -2, -2, 2, 126, 128, 300, -128, -130, -1000, 254, 256],
}


def cast_graph(x, dst, name="y"):
    def build(b):
        b.output(b.cast(b.arg("x", x.shape, x.dtype), dst, name=name), name)
    return build


@pytest.mark.parametrize("dst", [np.int8, np.uint8, np.int32, np.int64])
def test_cast_float_to_integer_hand_listed(dst):
    announce("cast f32 -> %s, ties and saturation" % np.dtype(dst).name)
    got = run_hip(cast_graph(TIES, dst), {"x": TIES})["y"]
    assert got.dtype == np.dtype(dst)
    assert got.tolist() == TIES_WANT[dst]


def test_cast_float_to_int32_ends():
    announce("cast f32 -> int32 at the ends of the range")
    x = np.array([3e9, -3e9, 2147483520.0, -2147483648.0, 16777217.0, 1e20, -1e20], np.float32)
    got = run_hip(cast_graph(x, np.int32), {"x": x})["y"]
    assert got.tolist() == [2147483520, -2147483648, 2147483520, -2147483648, 16777216, 2147483520, -2147483648]


@pytest.mark.parametrize("src,dst", [(np.int32, np.int8), (np.int32, np.uint8), (np.int64, np.int32), (np.int8, np.uint8),
                                     (np.uint8, np.int8), (np.int8, np.int32), (np.uint8, np.int64)])
def test_cast_integer_to_integer_saturates(src, dst, ref):
    announce("cast %s -> %s" % (np.dtype(src).name, np.dtype(dst).name))
    si, di = np.iinfo(src), np.iinfo(dst)
    edge = [si.min, si.min + 1, -70000, -129, -128, -1, 0, 1, 127, 128, 255, 256, 70000, si.max - 1, si.max,
            di.min, di.max]
    x = np.array([v for v in edge if si.min <= v <= si.max], src)
    got = run_hip(cast_graph(x, dst), {"x": x})["y"]
    want = np.clip(x.astype(np.int64), di.min, di.max).astype(dst)
    assert got.dtype == np.dtype(dst) and np.array_equal(got, want)
    assert np.array_equal(ref.cast_like_reference(x, dst), want)


@pytest.mark.parametrize("src", [np.int8, np.uint8, np.int32, np.int64, np.bool_])
def test_cast_integer_to_float(src):
    announce("cast %s -> f32" % np.dtype(src).name)
    r = np.random.default_rng(5)
    if src == np.bool_:
        x = r.integers(0, 2, 4099).astype(np.bool_)
    else:
        info = np.iinfo(src)
        x = r.integers(max(info.min, -2 ** 40), min(info.max, 2 ** 40), 4099, dtype=np.int64).astype(src)
        x[:4] = [info.min if abs(info.min) < 2 ** 41 else -2 ** 40, 0, 1, info.max if info.max < 2 ** 41 else 2 ** 40]
    got = run_hip(cast_graph(x, np.float32), {"x": x})["y"]
    assert got.dtype == np.float32 and np.array_equal(got, x.astype(np.float32))   # numpy: IEEE round to nearest even
    if src == np.int32:   # 2^24 + 1 and 2^24 + 3 are ties in float32: to the even neighbour
        t = np.array([16777217, 16777219], np.int32)
        assert run_hip(cast_graph(t, np.float32), {"x": t})["y"].tolist() == [16777216.0, 16777220.0]


def test_cast_to_bool_and_back():
    announce("cast f32 -> bool -> int32")
    x = np.array([0.0, -0.0, 0.25, -3.0, 1e-30, np.inf], np.float32)

    def build(b):
        m = b.cast(b.arg("x", x.shape), np.bool_, name="m")
        b.output(m, "m")
        b.output(b.cast(m, np.int32, name="i"), "i")
    got = run_hip(build, {"x": x})
    assert got["m"].tolist() == [False, False, True, True, True, True]
    assert got["i"].tolist() == [0, 0, 1, 1, 1, 1]


@pytest.mark.parametrize("half", [np.float16, "bf16"])
def test_cast_float_to_half_and_back_rounds_to_even(half, ref):
    """f32 -> fp16 / bf16 -> f32: equal, bit for bit, to the IEEE round-to-nearest-even
    conversion (numpy's for fp16, the integer formula for bf16), ties and overflow included."""
    announce("cast f32 -> %s -> f32" % half)
    r = np.random.default_rng(6)
    x = np.concatenate([r.standard_normal(5000).astype(np.float32) * 100,
                        np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65504.0, 65519.0, 65520.0, 1e-8, -1e-8,
                                  1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 3.3895314e38], np.float32)])
    if half == "bf16":
        u = x.view(np.uint32).astype(np.uint64)
        u = (u + 0x7fff + ((u >> 16) & 1)) >> 16 << 16
        want = (u & 0xffffffff).astype(np.uint32).view(np.float32)
        odla = entry.load().odla

        def build(b):
            h = b._ret(b.L.odla_Cast(b.arg("x", x.shape), odla.ODLA_BFLOAT16, None), "odla_Cast")
            b.output(b.cast(h, np.float32, name="y"), "y")
    else:
        want = x.astype(np.float16).astype(np.float32)

        def build(b):
            b.output(b.cast(b.cast(b.arg("x", x.shape), np.float16), np.float32, name="y"), "y")
    with np.errstate(over="ignore"):
        got = run_hip(build, {"x": x})["y"]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_cast_random_against_oracle_behind_arithmetic():
    """Casts inside a graph: a scaled tensor to int32 and int8 (results feed integer
    arithmetic), indices from int64 to int32 into a Gather."""
    announce("cast inside a graph")
    r = np.random.default_rng(7)
    x = (r.standard_normal((6, 37)) * 90).astype(np.float32)
    idx = r.integers(0, 6, (5,)).astype(np.int64)

    def build(b):
        xv = b.arg("x", x.shape)
        i32 = b.cast(xv, np.int32, name="i32")
        b.output(i32, "i32")
        b.output(b.cast(xv, np.int8, name="i8"), "i8")
        b.output(b.cast(b.cast(xv, np.uint8), np.float32, name="u8f"), "u8f")
        rows = b.gather(xv, b.cast(b.arg("idx", idx.shape, np.int64), np.int32), axis=0, name="rows")
        b.output(rows, "rows")
    got, want = run_both(build, {"x": x, "idx": idx})
    for k in ("i32", "i8", "u8f", "rows"):
        assert got[k].dtype == want[k].dtype and np.array_equal(got[k], want[k]), k


def test_cast_in_fp16_mode_reads_half_storage():
    """Under ODLA_FP16_MODE the FLOAT32 value is stored as fp16; the cast reads that storage."""
    announce("cast from fp16 storage")
    x = np.array([0.5, 1.5, 2.5, -2.5, 100.25, 300.0, -300.0, 1000.0], np.float32)   # all exact in fp16

    def build(b):
        s = b.mul(b.arg("x", x.shape), b.const("one", np.ones((1,), np.float32)))   # a half-precision temporary
        b.output(b.cast(s, np.int8, name="i8"), "i8")
        b.output(b.cast(s, np.int32, name="i32"), "i32")
    got = run_hip(build, {"x": x}, fp16=True)
    assert got["i8"].tolist() == [0, 2, 2, -2, 100, 127, -128, 127]
    assert got["i32"].tolist() == [0, 2, 2, -2, 100, 300, -300, 1000]


def test_batch_matmul_entry_point():
    """odla_BatchMatMul itself (not odla_Gemm): batched operands, both transposes."""
    announce("odla_BatchMatMul")
    r = np.random.default_rng(8)
    a = r.standard_normal((3, 4, 24, 40)).astype(np.float32)
    bt = r.standard_normal((3, 4, 56, 40)).astype(np.float32)   # B transposed
    at = r.standard_normal((3, 4, 40, 24)).astype(np.float32)   # A transposed
    b2 = r.standard_normal((3, 4, 40, 56)).astype(np.float32)

    def build(b):
        av, btv = b.arg("a", a.shape), b.arg("bt", bt.shape)
        atv, b2v = b.arg("at", at.shape), b.arg("b2", b2.shape)
        b.output(b.batch_matmul(av, btv, False, True, name="y0"), "y0")
        b.output(b.batch_matmul(atv, b2v, True, False, name="y1"), "y1")
        b.output(b.batch_matmul(av, b2v, name="y2"), "y2")
    got, want = run_both(build, {"a": a, "bt": bt, "at": at, "b2": b2})
    for k in ("y0", "y1", "y2"):
        assert got[k].shape == (3, 4, 24, 56)
        assert max_rel_err(got[k], want[k]) <= 1e-4, k
