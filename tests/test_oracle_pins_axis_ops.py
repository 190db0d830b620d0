"""Pins of the oracle's GatherElements, CumSum, Hardmax, Compress and Shift (no GPU
needed).  The reference tests these operators with the operator-standard node examples
(tests/unittests/lit_cases/test_dnnl/test_{gather_elements_*, cumsum_*, hardmax_*,
compress_*, bitshift_*}_dnnl.cc; the data files they load are not part of the reference
tree): the small examples below are those cases, written out.  Beyond them every function
is compared with an independent numpy formulation on random inputs, chosen so that a wrong
axis, a swapped extent or an off-by-one in the exclusive / reverse forms fails.
"""
import numpy as np
import pytest


def rng(seed):
    return np.random.default_rng(seed)


def test_gather_elements_examples(ref):
    d = np.array([[1, 2], [3, 4]], np.float32)
    assert np.array_equal(ref.gather_elements(d, np.array([[0, 0], [1, 0]], np.int64), 1), [[1, 1], [4, 3]])
    d = np.arange(1, 10, dtype=np.float32).reshape(3, 3)
    assert np.array_equal(ref.gather_elements(d, np.array([[1, 2, 0], [2, 0, 0]], np.int32), 0), [[4, 8, 3], [7, 2, 3]])
    assert np.array_equal(ref.gather_elements(d, np.array([[-1, -2, 0], [-2, 0, 0]], np.int64), 0), [[7, 5, 3], [4, 2, 3]])


@pytest.mark.parametrize("axis", [0, 1, 2, -1])
def test_gather_elements_against_take_along_axis(ref, axis):
    r = rng(5 + axis)
    d = r.standard_normal((4, 5, 6)).astype(np.float32)
    shp = list(d.shape)
    shp[axis] = 7          # more picks than the axis is long; extents differ, so a swapped one shows
    idx = r.integers(-d.shape[axis], d.shape[axis], shp).astype(np.int64)
    want = np.take_along_axis(d, np.where(idx < 0, idx + d.shape[axis], idx), axis=axis)
    assert np.array_equal(ref.gather_elements(d, idx, axis), want)
    # a smaller leading extent of the indices picks from the leading slices only
    if axis % 3 != 0:
        assert np.array_equal(ref.gather_elements(d, idx[:2], axis), want[:2])


def test_cumsum_examples(ref):
    x = np.arange(1, 6, dtype=np.float32)
    assert np.array_equal(ref.cumsum(x, 0), [1, 3, 6, 10, 15])
    assert np.array_equal(ref.cumsum(x, 0, exclusive=True), [0, 1, 3, 6, 10])
    assert np.array_equal(ref.cumsum(x, 0, reverse=True), [15, 14, 12, 9, 5])
    assert np.array_equal(ref.cumsum(x, 0, exclusive=True, reverse=True), [14, 12, 9, 5, 0])
    m = np.arange(1, 7, dtype=np.float32).reshape(2, 3)
    assert np.array_equal(ref.cumsum(m, 0), [[1, 2, 3], [5, 7, 9]])
    assert np.array_equal(ref.cumsum(m, 1), [[1, 3, 6], [4, 9, 15]])
    assert np.array_equal(ref.cumsum(m, -1), [[1, 3, 6], [4, 9, 15]])


@pytest.mark.parametrize("axis", [0, 1, 2])
@pytest.mark.parametrize("exclusive", [False, True])
@pytest.mark.parametrize("reverse", [False, True])
def test_cumsum_against_numpy(ref, axis, exclusive, reverse):
    x = rng(11).standard_normal((3, 17, 5)).astype(np.float32)
    v = np.flip(x, axis) if reverse else x
    want = np.cumsum(v.astype(np.float64), axis=axis)
    if exclusive:
        want = want - v
    if reverse:
        want = np.flip(want, axis)
    got = ref.cumsum(x, axis, exclusive, reverse)
    assert got.dtype == np.float32 and np.max(np.abs(got - want)) <= 1e-5
    # the sum over the whole axis is the last (first) inclusive element
    if not exclusive:
        edge = np.take(got, 0 if reverse else -1, axis=axis)
        assert np.max(np.abs(edge - x.sum(axis=axis, dtype=np.float64))) <= 1e-5


def test_hardmax_examples(ref):
    x = np.array([[3, 0, 1, 2], [2, 5, 1, 0], [0, 1, 3, 2], [0, 1, 2, 3]], np.float32)
    assert np.array_equal(ref.hardmax(x, -1), np.eye(4, dtype=np.float32))
    # equal maxima: the first one
    assert np.array_equal(ref.hardmax(np.array([[3, 3, 3, 1]], np.float32), 1), [[1, 0, 0, 0]])


@pytest.mark.parametrize("axis", [0, 1, 2, -1])
def test_hardmax_against_argmax(ref, axis):
    x = np.round(rng(21).standard_normal((3, 4, 5)) * 2).astype(np.float32)   # rounded: ties occur
    got = ref.hardmax(x, axis)
    assert np.array_equal(got.sum(axis=axis), np.ones_like(got.sum(axis=axis)))
    assert np.array_equal(np.argmax(got, axis=axis), np.argmax(x, axis=axis))   # numpy: first occurrence too


def test_compress_examples(ref):
    x = np.array([[1, 2], [3, 4], [5, 6]], np.float32)
    assert np.array_equal(ref.compress(x, [0, 1, 1], 0, (2, 2)), [[3, 4], [5, 6]])
    assert np.array_equal(ref.compress(x, [0, 1], 1, (3, 1)), [[2], [4], [6]])
    assert np.array_equal(ref.compress(x, [0, 1], -1, (3, 1)), [[2], [4], [6]])
    # flat form; the declared maximum holds one element per condition
    assert np.array_equal(ref.compress(x, [0, 1, 0, 0, 1], None, (5,)), [2, 5, 0, 0, 0])


@pytest.mark.parametrize("axis", [0, 1, 2, None])
def test_compress_against_numpy(ref, axis):
    r = rng(31)
    x = r.standard_normal((4, 6, 5)).astype(np.float32)
    n = x.size if axis is None else x.shape[axis]
    cond = r.random(n) < 0.4
    want = np.compress(cond, x, axis=axis)
    # the declared maximum: as if every condition were set
    max_shape = (x.size,) if axis is None else x.shape
    got = ref.compress(x, cond, axis, max_shape)
    assert got.shape == tuple(max_shape)
    flat = got.reshape(-1)
    assert np.array_equal(flat[:want.size], want.reshape(-1))     # dense, in the order of the true shape
    assert not np.any(flat[want.size:])
    # a condition shorter than the axis only looks at the leading slices
    short = cond[: n // 2]
    want2 = np.compress(short, x, axis=axis)
    assert np.array_equal(ref.compress(x, short, axis, max_shape).reshape(-1)[:want2.size], want2.reshape(-1))


def test_shift_examples(ref):
    for dt in (np.uint8, np.uint32, np.uint64):
        x, y = np.array([16, 4, 1], dt), np.array([1, 2, 3], dt)
        assert np.array_equal(ref.shift(x, y, True), [32, 16, 8])
        assert np.array_equal(ref.shift(x, y, False), [8, 1, 0])


def test_shift_against_python_integers(ref):
    r = rng(41)
    for dt, bits in ((np.uint8, 8), (np.uint32, 32), (np.uint64, 64)):
        x = r.integers(0, 2 ** bits, 200, dtype=np.uint64).astype(dt)
        s = r.integers(0, bits + 3, 200).astype(dt)      # also shifts by the width and more
        for left in (True, False):
            got = ref.shift(x, s, left)
            want = [((int(a) << int(b)) % 2 ** bits if left else int(a) >> int(b)) if int(b) < bits else 0 for a, b in zip(x, s)]
            assert got.dtype == dt and [int(v) for v in got] == want
