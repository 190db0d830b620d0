"""Pins of the CPU oracle (no GPU needed).

Before the oracle is trusted as the checker of the GPU library, each of its
functions is checked against something that does not come from this
repository's own formulas: known-answer vectors the reference's tests hold,
vectors produced by the reference's own fp32 kernels (tests/golden/
sn_rt_vectors.npz, and live against oracle/_ref/libsn_rt.so when it is built),
published ONNX operator examples, float64 / int64 brute force, and closed forms
from the standard library.
"""
import math
import os

import numpy as np
import pytest

import __graft_entry__ as entry

GOLD = np.load(os.path.join(entry.ROOT, "tests", "golden", "sn_rt_vectors.npz"))


def rng(seed):
    return np.random.default_rng(seed)


# ------------------------------------------------------------------ conv ----
def test_conv_kat_from_reference_doctest(ref):
    """odla_popart/test/odla_ops_nn_test.cc:147-200 of the reference tree."""
    x = np.arange(25, dtype=np.float32).reshape(1, 1, 5, 5)
    w = np.ones((1, 1, 3, 3), np.float32)
    y = ref.conv2d(x, w, None, (1, 1), (1, 1, 1, 1))
    assert y.reshape(-1).tolist() == [12, 21, 27, 33, 24, 33, 54, 63, 72, 51, 63, 99, 108, 117, 81, 93, 144, 153,
                                      162, 111, 72, 111, 117, 123, 84]


@pytest.mark.parametrize("i", range(5))
def test_conv_against_reference_kernel_vectors(ref, i):
    x, w = GOLD["conv%d_x" % i], GOLD["conv%d_w" % i]
    s, p = (int(v) for v in GOLD["conv%d_attr" % i])
    y = ref.conv2d(x, w, None, (s, s), (p, p, p, p))
    want = GOLD["conv%d_y" % i]
    assert y.shape == want.shape
    assert np.max(np.abs(y - want)) <= 1e-5 * np.max(np.abs(want))


def brute_conv(x, w, b, stride, pad, dil, group):
    N, C, H, W = x.shape
    O, I, R, S = w.shape
    Ho = (H + pad[0] + pad[2] - ((R - 1) * dil[0] + 1)) // stride[0] + 1
    Wo = (W + pad[1] + pad[3] - ((S - 1) * dil[1] + 1)) // stride[1] + 1
    y = np.zeros((N, O, Ho, Wo), np.float64)
    og = O // group
    for n in range(N):
        for o in range(O):
            g = o // og
            for ho in range(Ho):
                for wo in range(Wo):
                    acc = 0.0 if b is None else float(b[o])
                    for c in range(I):
                        for r in range(R):
                            for s in range(S):
                                hi = ho * stride[0] - pad[0] + r * dil[0]
                                wi = wo * stride[1] - pad[1] + s * dil[1]
                                if 0 <= hi < H and 0 <= wi < W:
                                    acc += float(x[n, g * I + c, hi, wi]) * float(w[o, c, r, s])
                    y[n, o, ho, wo] = acc
    return y


@pytest.mark.parametrize("case", [
    (1, 4, 6, 7, 6, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1),
    (2, 4, 7, 6, 4, 3, (2, 1), (0, 1, 2, 0), (1, 1), 2),   # asymmetric pad, groups, mixed stride
    (1, 2, 9, 9, 3, 3, (1, 1), (2, 2, 2, 2), (2, 2), 1),   # dilation
    (1, 3, 8, 8, 2, 5, (2, 2), (2, 2, 2, 2), (1, 1), 1),
])
def test_conv_against_float64_brute_force(ref, case):
    N, C, H, W, O, k, st, pad, dil, g = case
    r = rng(3)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = r.standard_normal((O, C // g, k, k)).astype(np.float32)
    b = r.standard_normal(O).astype(np.float32)
    y = ref.conv2d(x, w, b, st, pad, dil, g)
    want = brute_conv(x, w, b, st, pad, dil, g)
    assert y.shape == want.shape
    assert np.max(np.abs(y - want)) <= 1e-5 * np.max(np.abs(want))


def test_conv_identities(ref):
    """1x1 convolution is a matrix product; a delta kernel is a shifted copy."""
    r = rng(4)
    x = r.standard_normal((2, 5, 4, 4)).astype(np.float32)
    w = r.standard_normal((3, 5, 1, 1)).astype(np.float32)
    y = ref.conv2d(x, w)
    want = np.einsum("nchw,oc->nohw", x.astype(np.float64), w[:, :, 0, 0].astype(np.float64))
    assert np.max(np.abs(y - want)) <= 1e-5
    d = np.zeros((1, 1, 3, 3), np.float32)
    d[0, 0, 0, 2] = 1.0  # picks x[h-1, w+1]
    x1 = r.standard_normal((1, 1, 5, 5)).astype(np.float32)
    y = ref.conv2d(x1, d, None, (1, 1), (1, 1, 1, 1))
    want = np.zeros_like(x1)
    want[0, 0, 1:, :-1] = x1[0, 0, :-1, 1:]
    assert np.array_equal(y, want)


# ---------------------------------------------------------------- pooling ----
def test_pool_kats_from_reference_doctest(ref):
    """odla_ops_nn_test.cc:38-78 and :523-560."""
    x = np.arange(1, 17, dtype=np.float32).reshape(1, 1, 4, 4)
    assert ref.pool2d(x, (3, 3), (1, 1), (0, 0, 0, 0), None, False).reshape(-1).tolist() == [6, 7, 10, 11]
    assert ref.pool2d(x, (3, 3), (1, 1), (0, 0, 0, 0), None, True).reshape(-1).tolist() == [11, 12, 15, 16]


@pytest.mark.parametrize("i", range(3))
def test_maxpool_against_reference_kernel_vectors(ref, i):
    x = GOLD["pool%d_x" % i]
    k, s, p = (int(v) for v in GOLD["pool%d_attr" % i])
    y = ref.pool2d(x, (k, k), (s, s), (p, p, p, p), None, True)
    assert np.array_equal(y, GOLD["pool%d_y" % i])


def test_avgpool_padding_rules(ref):
    """ONNX averagepool_2d_pads (exclude padding, passes on the reference CPU
    backend) and count_include_pad, on a constant image where both are closed forms."""
    x = np.ones((1, 1, 4, 4), np.float32)
    ex = ref.pool2d(x, (3, 3), (1, 1), (1, 1, 1, 1), None, False, False)
    assert np.allclose(ex, 1.0)
    inc = ref.pool2d(x, (3, 3), (1, 1), (1, 1, 1, 1), None, False, True)
    assert np.isclose(inc[0, 0, 0, 0], 4.0 / 9.0) and np.isclose(inc[0, 0, 0, 1], 6.0 / 9.0) and np.isclose(inc[0, 0, 1, 1], 1.0)


def test_maxpool_ceil_mode_shape(ref):
    """odla_dnnl.cc:1411-1429: an output one larger than the floor formula is served by extra back padding."""
    x = rng(5).standard_normal((1, 1, 6, 6)).astype(np.float32)
    y = ref.pool2d(x, (3, 3), (2, 2), (0, 0, 0, 0), (3, 3), True)
    assert y.shape == (1, 1, 3, 3)
    assert y[0, 0, 2, 2] == x[0, 0, 4:, 4:].max()


# ------------------------------------------------------------ gemm/softmax ----
@pytest.mark.parametrize("i", range(3))
def test_gemm_against_reference_kernel_vectors(ref, i):
    a, b, c = GOLD["gemm%d_a" % i], GOLD["gemm%d_b" % i], GOLD["gemm%d_c" % i]
    ta, tb, alpha, beta = GOLD["gemm%d_attr" % i]
    rb = ref.RefBuilder({})
    y = rb.gemm(a, b, c.reshape(1, -1), bool(ta), bool(tb), float(alpha), float(beta))
    want = GOLD["gemm%d_y" % i]
    assert np.max(np.abs(y - want)) <= 1e-5 * np.max(np.abs(want))


def test_gemm_kat_from_reference_doctest(ref):
    """odla_ops_test.cc:39-79: ones[4,16] x ones[16,8] = 16."""
    rb = ref.RefBuilder({})
    assert np.all(rb.gemm(np.ones((4, 16), np.float32), np.ones((16, 8), np.float32), None, False, False, 1.0, 0.0) == 16.0)


@pytest.mark.parametrize("i", range(2))
def test_softmax_against_reference_kernel_vectors(ref, i):
    rb = ref.RefBuilder({})
    y = rb.softmax(GOLD["softmax%d_x" % i], -1)
    assert np.max(np.abs(y - GOLD["softmax%d_y" % i])) <= 1e-6


def test_softmax_large_number_and_sum(ref):
    rb = ref.RefBuilder({})
    x = np.array([[0, 1, 2, 3], [10000, 10001, 10002, 10003]], np.float32)
    y = rb.softmax(x, -1)
    assert np.allclose(y[0], [0.032058604, 0.08714432, 0.23688284, 0.6439143], atol=1e-7)
    assert np.allclose(y[0], y[1]) and np.allclose(y.sum(axis=1), 1.0)
    ly = rb.softmax(x, -1, log=True)
    assert np.allclose(np.exp(ly), y, atol=1e-6)


# ------------------------------------------------------------ normalisation ----
def test_batchnorm_kat_from_reference_doctest(ref):
    """odla_ops_nn_test.cc:80-145."""
    rb = ref.RefBuilder({})
    x = np.array([-1, 0, 1, 2, 3, 4], np.float32).reshape(1, 2, 1, 3)
    y = rb.batchnorm(x, np.array([0, 3], np.float32), np.array([1, 1.5], np.float32), 1e-5,
                     np.array([1.0, 1.5], np.float32), np.array([0, 1], np.float32))
    assert np.max(np.abs(y.reshape(-1) - [-0.999995, 0, 0.999995, -0.224741, 1, 2.22474])) < 1e-5


def test_batchnorm_folding_formula(ref):
    """lib/transforms/inst_simplify.cc:1408-1415: y = x*m + (b - mean*m), m = s/sqrt(var+eps)."""
    r = rng(6)
    x = r.standard_normal((2, 3, 4, 4)).astype(np.float32)
    mean, var = r.standard_normal(3), r.random(3) + 0.5
    g, b = r.standard_normal(3), r.standard_normal(3)
    rb = ref.RefBuilder({})
    y = rb.batchnorm(x, mean, var, 1e-3, g, b)
    m = g / np.sqrt(var + 1e-3)
    want = x * m.reshape(1, 3, 1, 1) + (b - mean * m).reshape(1, 3, 1, 1)
    assert np.max(np.abs(y - want)) < 1e-5


def test_layernorm_invariants(ref):
    """lib/transforms/fusion.cc:296-313: biased variance; with gamma 1 / beta 0 each row
    has mean 0 and variance 1; gamma and beta act as an affine map afterwards."""
    r = rng(7)
    x = (r.standard_normal((5, 64)) * 3 + 2).astype(np.float32)
    rb = ref.RefBuilder({})
    y = rb.layernorm(x, 1, 1e-12)
    assert np.max(np.abs(y.mean(axis=1))) < 1e-6 and np.max(np.abs(y.var(axis=1) - 1)) < 1e-5
    g, b = r.standard_normal(64).astype(np.float32), r.standard_normal(64).astype(np.float32)
    assert np.max(np.abs(rb.layernorm(x, 1, 1e-12, g, b) - (y * g + b))) < 1e-5
    # translation invariance and scale invariance of the normalised value
    assert np.max(np.abs(rb.layernorm(x * 4 + 10, 1, 1e-12) - y)) < 1e-4


def test_gelu_erf_closed_forms(ref):
    """odla_dnnl.cc:1868-1876 against math.erf / math.tanh in float64."""
    rb = ref.RefBuilder({})
    x = np.linspace(-5, 5, 101).astype(np.float32)
    want = np.array([0.5 * v * (1 + math.erf(v / math.sqrt(2))) for v in x.astype(np.float64)])
    assert np.max(np.abs(rb.gelu(x) - want)) < 1e-6
    want_t = np.array([0.5 * v * (1 + math.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3))) for v in x.astype(np.float64)])
    assert np.max(np.abs(rb.gelu(x, True) - want_t)) < 1e-6
    assert np.max(np.abs(rb.erf(x) - np.array([math.erf(v) for v in x.astype(np.float64)]))) < 1e-6


# ------------------------------------------------------------- broadcast ----
def test_reference_alignment_examples(ref):
    """The three examples in the comment at odla_dnnl.h:303-306."""
    assert ref.align_like_reference((1, 5), (1, 4, 1)) == (1, 1, 5)
    assert ref.align_like_reference((64,), (1, 64, 128)) == (1, 64, 1)
    assert ref.align_like_reference((64,), (1, 64, 64)) == (1, 1, 64)
    with pytest.raises(ValueError):
        ref.align_like_reference((7, 31, 64), (2, 31, 64, 64))


# ---------------------------------------------------------- quantisation ----
def test_quantize_onnx_published_example(ref):
    rb = ref.RefBuilder({})
    x = np.array([0, 2, 3, 1000, -254, -1000], np.float32)
    q = rb.quantize(x, [2.0], [128])
    assert q.tolist() == [128, 129, 130, 255, 1, 0]
    assert rb.dequantize(q, [2.0], [128]).tolist() == [0, 2, 4, 254, -254, -256]


def test_quantize_round_half_even_exhaustive(ref):
    """Every half-integer in range rounds to the even neighbour."""
    rb = ref.RefBuilder({})
    k = np.arange(-300, 300)
    x = (k + 0.5).astype(np.float32)
    q = rb.quantize(x, [1.0], [0], signed=True).astype(np.int64)
    want = np.clip(np.where(k % 2 == 0, k, k + 1), -128, 127)
    assert np.array_equal(q, want)


def test_requant_formula_rounding_and_saturation(ref):
    """q = sat8(max(fma(float(acc), mul, zp), lo)): hand-worked, mul = 0.5 (exact products)."""
    acc = np.array([-1000, -3, -1, 0, 1, 3, 5, 1000, 2 ** 24 + 1], np.int32).reshape(1, 9, 1, 1)
    mul = np.full(9, 0.5, np.float32)
    # 0.5*acc + 10: -490, 8.5, 9.5, 10, 10.5, 11.5, 12.5, 510, 2^23 + 10 -> ties to even, saturate
    assert ref.requant_q8(acc, mul, zp=10, lo=0).reshape(-1).tolist() == [0, 8, 10, 10, 10, 12, 12, 255, 255]
    assert ref.requant_q8(acc, mul, zp=10, lo=10).reshape(-1).tolist() == [10, 10, 10, 10, 10, 12, 12, 255, 255]
    # the zero point is inside the rounding: with an odd one the ties fall the other way
    # 0.5*acc + 11: -489, 9.5, 10.5, 11, 11.5, 12.5, 13.5, 511, ...
    assert ref.requant_q8(acc, mul, zp=11, lo=0).reshape(-1).tolist() == [0, 10, 10, 11, 12, 12, 14, 255, 255]
    # with a residual: add = fma(r, r_mul, r_add); r_mul = 0.25, r_add = 5 - 20 * 0.25 = 0
    res = np.array([0, 20, 22, 21, 23, 255, 255, 0, 0], np.uint8).reshape(1, 9, 1, 1)
    # 0.5*acc:   -500  -1.5  -0.5  0     0.5   1.5    2.5    500  2^23
    # 0.25*r:    0     5     5.5   5.25  5.75  63.75  63.75  0    0
    # sum:       -500  3.5   5.0   5.25  6.25  65.25  66.25  500  2^23
    assert ref.requant_q8(acc, mul, 5, 0, res, 0.25, 0.0).reshape(-1).tolist() == [0, 4, 5, 5, 6, 65, 66, 255, 255]
    assert ref.requant_q8(acc, mul, 5, 5, res, 0.25, 0.0).reshape(-1).tolist() == [5, 5, 5, 5, 6, 65, 66, 255, 255]


def _round_to_f32(fr):
    """Nearest binary32 value (ties to even) of an exact rational, as a Fraction."""
    from fractions import Fraction
    if fr == 0:
        return Fraction(0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = 0
    while a >= 2 ** 24:
        a /= 2
        e += 1
    while a < 2 ** 23:
        a *= 2
        e -= 1
    n = round(a)          # Python rounds exact halves to the even integer
    return sign * Fraction(n) * Fraction(2) ** e


def test_requant_is_one_fused_multiply_add_against_exact_rationals(ref):
    """The requantisation rounds acc * mul + add ONCE to binary32 (a fused multiply-add),
    then to the nearest integer (ties to even), then saturates: checked against exact
    rational arithmetic, so that neither a separate multiply and add (two roundings)
    nor a double-precision detour would pass."""
    from fractions import Fraction
    r = rng(91)
    n = 4000
    acc = r.integers(-70000, 70000, n).astype(np.int32)
    acc[:8] = [1, 3, -3, 5, 2 ** 24 + 1, -(2 ** 24) - 3, 2 ** 31 - 1, -(2 ** 31)]
    mul = (r.random(n, dtype=np.float32) * np.float32(0.01)).astype(np.float32)
    mul[:4] = np.float32(0.5) + np.float32(2.0 ** -24)     # products just beside a tie
    # cases found by search in which rounding the product before the zero point is added
    # (two roundings) lands on the other side of a tie: one fused multiply-add gives 5, 5, 27, 17
    acc[8:12] = [-38736, -50321, -52629, -25444]
    mul[8:12] = [float.fromhex(h) for h in ("0x1.a7cfc8p-8", "0x1.44f044p-8", "0x1.1c89dap-8", "0x1.31dd26p-7")]
    zp = 255.0
    resq = r.integers(0, 256, n).astype(np.uint8)
    r_mul, r_add = np.float32(0.3713), np.float32(-11.625)
    got = ref.requant_q8(acc.reshape(1, n, 1, 1), mul, zp, 3).reshape(-1)
    got_r = ref.requant_q8(acc.reshape(1, n, 1, 1), mul, zp, 3, resq.reshape(1, n, 1, 1), r_mul, r_add).reshape(-1)

    def sat8(fr):
        fr = max(fr, Fraction(3))
        return int(min(max(round(fr), 0), 255))

    two_roundings_differ = 0
    for i in range(n):
        a = _round_to_f32(Fraction(int(acc[i])))                      # int32 -> float32
        m = Fraction(float(mul[i]))
        want = sat8(_round_to_f32(a * m + Fraction(zp)))
        assert int(got[i]) == want, (i, int(acc[i]), float(mul[i]))
        add = _round_to_f32(Fraction(int(resq[i])) * Fraction(float(r_mul)) + Fraction(float(r_add)))
        assert int(got_r[i]) == sat8(_round_to_f32(a * m + add)), i
        two_roundings_differ += sat8(_round_to_f32(_round_to_f32(a * m) + Fraction(zp))) != want
    assert got[8:12].tolist() == [5, 5, 27, 17]
    assert two_roundings_differ >= 4       # the sample does tell the two formulations apart


def test_qadd_hand_worked_levels(ref):
    """Residual add of two 8-bit tensors: dequantise, add, requantise.  Scales are
    powers of two, so every product below is exact and was worked by hand:
    a: s = 0.5, zp = 10; b: s = 0.25, zp = 20; out: s = 0.5, zp = 5."""
    a = np.array([12, 12, 13, 255, 0, 9, 8], np.uint8)
    b = np.array([22, 21, 21, 255, 0, 21, 21], np.uint8)
    # fa:        1.0   1.0   1.5  122.5  -5.0  -0.5  -1.0
    # fb:        0.5   0.25  0.25 58.75  -5.0  0.25  0.25
    # f / 0.5:   3.0   2.5   3.5  362.5  -20   -0.5  -1.5
    # rne:       3     2     4    362    -20   -0    -2     (ties go to the even neighbour)
    # + 5:       8     7     9    367    -15   5     3
    got = ref.qadd(a, (0.5, 10), b, (0.25, 20), (0.5, 5))
    assert got.dtype == np.uint8 and got.tolist() == [8, 7, 9, 255, 0, 5, 3]
    # a fused ReLU clamps at the zero point of the result instead of at 0
    assert ref.qadd(a, (0.5, 10), b, (0.25, 20), (0.5, 5), relu=True).tolist() == [8, 7, 9, 255, 5, 5, 5]


def test_resize_nearest_source_index_rule(ref):
    """src = floor(in * dst / out) per axis, as the reference's portable backend
    loops it (channels-last there, channels-first here)
    [ref: ODLA/platforms/odla_eigen.cc:619-631].  Hand-listed indices for ratios that
    are not integers, then the same loops in plain Python on random data."""
    rb = ref.RefBuilder({})
    x = np.arange(3, dtype=np.float32).reshape(1, 1, 1, 3)
    assert rb.resize_nearest(x, (1, 7)).reshape(-1).tolist() == [0, 0, 0, 1, 1, 2, 2]     # 3 -> 7
    x = np.arange(7, dtype=np.float32).reshape(1, 1, 7, 1)
    assert rb.resize_nearest(x, (3, 1)).reshape(-1).tolist() == [0, 2, 4]                 # 7 -> 3
    x = np.arange(5, dtype=np.float32).reshape(1, 1, 5, 1)
    assert rb.resize_nearest(x, (8, 1)).reshape(-1).tolist() == [0, 0, 1, 1, 2, 3, 3, 4]  # 5 -> 8
    x = np.arange(4, dtype=np.float32).reshape(1, 1, 2, 2)
    assert rb.resize_nearest(x, (4, 4))[0, 0].tolist() == [[0, 0, 1, 1], [0, 0, 1, 1], [2, 2, 3, 3], [2, 2, 3, 3]]

    r = rng(31)
    for (ih, iw), (oh, ow) in (((5, 7), (8, 3)), ((13, 13), (26, 26)), ((6, 4), (4, 9)), ((1, 3), (5, 5))):
        x = r.standard_normal((2, 3, ih, iw)).astype(np.float32)
        want = np.empty((2, 3, oh, ow), np.float32)
        for n in range(2):
            for h in range(oh):
                src_h = ih * h // oh
                for w in range(ow):
                    src_w = iw * w // ow
                    want[n, :, h, w] = x[n, :, src_h, src_w]
        assert np.array_equal(rb.resize_nearest(x, (oh, ow)), want)


def test_resize_linear_half_pixel_rule(ref):
    """ODLA_LINEAR is oneDNN's resampling_linear in the reference
    [ref: ODLA/platforms/dnnl/odla_dnnl.cc:1526-1551]; that library (1.x / 2.x) is
    not part of the reference tree, so the oracle restates its published rule
    (source coordinate (o + 0.5) * in / out - 0.5, two neighbours, edges clamped)
    and is pinned by what fixes that rule: hand-worked 2x weights, exactness on
    ramps in the interior, constancy, and two independent library routines that
    implement the same rule (torch bilinear without corner alignment; scipy's
    zoom in grid mode with edge replication)."""
    rb = ref.RefBuilder({})
    # 2 -> 4: sources at -0.25, 0.25, 0.75, 1.25 -> clamp, 3:1, 1:3, clamp
    x = np.array([10.0, 20.0], np.float32).reshape(1, 1, 1, 2)
    assert rb.resize_linear(x, (1, 4)).reshape(-1).tolist() == [10.0, 12.5, 17.5, 20.0]
    # 4 -> 2: sources at 0.5 and 2.5 -> plain means of neighbours
    x = np.array([1.0, 3.0, 5.0, 9.0], np.float32).reshape(1, 1, 4, 1)
    assert rb.resize_linear(x, (2, 1)).reshape(-1).tolist() == [2.0, 7.0]
    # 3 -> 5 (ratio 0.6): sources -0.2, 0.4, 1.0, 1.6, 2.2
    x = np.array([0.0, 10.0, 40.0], np.float32).reshape(1, 1, 1, 3)
    assert np.allclose(rb.resize_linear(x, (1, 5)).reshape(-1), [0.0, 4.0, 10.0, 28.0, 40.0], atol=1e-5)
    # a ramp is reproduced wherever both neighbours exist; a constant everywhere
    ramp = (3.0 * np.arange(9, dtype=np.float32) + 2.0).reshape(1, 1, 1, 9)
    got = rb.resize_linear(ramp, (1, 23)).reshape(-1)
    src = (np.arange(23) + 0.5) * 9 / 23 - 0.5
    inside = (src >= 0) & (src <= 8)
    assert np.allclose(got[inside], 3.0 * src[inside] + 2.0, atol=1e-4)
    assert np.array_equal(rb.resize_linear(np.full((2, 3, 5, 4), 7.5, np.float32), (9, 11)), np.full((2, 3, 9, 11), 7.5, np.float32))

    torch = pytest.importorskip("torch")
    from scipy import ndimage
    r = rng(32)
    for (ih, iw), (oh, ow) in (((5, 7), (8, 3)), ((13, 13), (26, 26)), ((6, 4), (4, 9)), ((1, 3), (5, 5)), ((7, 5), (7, 12))):
        x = r.standard_normal((2, 3, ih, iw)).astype(np.float32)
        got = rb.resize_linear(x, (oh, ow))
        want = torch.nn.functional.interpolate(torch.from_numpy(x), size=(oh, ow), mode="bilinear", align_corners=False).numpy()
        assert np.max(np.abs(got - want)) <= 1e-5
        zoomed = ndimage.zoom(x.astype(np.float64), (1, 1, oh / ih, ow / iw), order=1, mode="nearest", grid_mode=True)
        assert zoomed.shape == got.shape and np.max(np.abs(got - zoomed)) <= 1e-5


def test_cast_rounds_to_even_and_saturates(ref):
    """odla_Cast is a oneDNN reorder in the reference [ref: odla_dnnl_cast.cc:232-258]:
    float -> integer rounds to nearest even and saturates.  Hand-listed values."""
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 2.4999, 126.5, 127.5, 300.0, -128.5, -129.5, -1000.0, 254.5, 255.5],
                 np.float32)
    assert ref.cast_like_reference(x, np.int8).tolist() == \
        [0, 2, 2, 0, -2, -2, 2, 126, 127, 127, -128, -128, -128, 127, 127]
    assert ref.cast_like_reference(x, np.uint8).tolist() == \
        [0, 2, 2, 0, 0, 0, 2, 126, 128, 255, 0, 0, 0, 254, 255]
    assert ref.cast_like_reference(x, np.int32).tolist() == \
        [0, 2, 2, 0, -2, -2, 2, 126, 128, 300, -128, -130, -1000, 254, 256]
    big = np.array([3e9, -3e9, 2147483520.0, -2147483648.0, 16777217.0], np.float32)
    assert ref.cast_like_reference(big, np.int32).tolist() == [2147483520, -2147483648, 2147483520, -2147483648, 16777216]
    # integers: narrowing saturates, widening and int -> float are exact / round to nearest even
    i = np.array([-70000, -129, -128, -1, 0, 127, 128, 255, 256, 70000], np.int32)
    assert ref.cast_like_reference(i, np.int8).tolist() == [-128, -128, -128, -1, 0, 127, 127, 127, 127, 127]
    assert ref.cast_like_reference(i, np.uint8).tolist() == [0, 0, 0, 0, 0, 127, 128, 255, 255, 255]
    assert ref.cast_like_reference(np.array([16777217, 16777219], np.int32), np.float32).tolist() == [16777216.0, 16777220.0]
    assert ref.cast_like_reference(np.array([0.0, -0.0, 0.25, np.nan], np.float32), np.bool_).tolist() == [False, False, True, True]
    # float -> half precision: round to nearest even on the 10-bit (fp16) / 7-bit (bf16) mantissa
    h = ref.cast_like_reference(np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65520.0], np.float32), np.float16)
    assert h.astype(np.float32).tolist() == [1.0, 1.0 + 2.0 ** -9, np.inf]


def test_q8_accumulators_against_int64_brute_force(ref):
    r = rng(8)
    N, C, H, W, O, k = 2, 5, 6, 6, 4, 3
    xq = r.integers(0, 256, (N, C, H, W)).astype(np.uint8)
    wq = r.integers(-127, 128, (O, C, k, k)).astype(np.int8)
    b = r.integers(-1000, 1000, O).astype(np.int32)
    zp = 131
    acc = ref.conv2d_q8_acc(xq, zp, wq, b, (2, 2), (1, 1, 1, 1))
    want = brute_conv(xq.astype(np.float64) - zp, wq.astype(np.float64), b.astype(np.float64), (2, 2), (1, 1, 1, 1), (1, 1), 1)
    # padding contributes (zp - zp) = 0: brute_conv skips out-of-range taps, same thing
    assert np.array_equal(acc.astype(np.int64), want.astype(np.int64))


def test_weight_and_activation_schemes(ref, models):
    """utils/halo_pgq.py:283-297 and weights_quantizer.cc:126-176 of the reference:
    scale=(max-min)/255, zp=round(-min/scale) clamped to [0,255]; symmetric weights max|w|/127.
    The host-side table writer and the oracle agree."""
    s, z = ref.act_qparams(-1.0, 3.0)
    assert np.isclose(s, 4.0 / 255) and z == 64
    assert ref.act_qparams(0.5, 2.0)[1] == 0            # range widened to contain zero
    assert models.act_qparams(-1.0, 3.0) == (s, z)
    w = np.array([[0.5, -1.27], [0.0, 0.0]], np.float32)
    sw = ref.weight_qparams(w)
    assert np.isclose(sw[0], 0.01) and sw[1] == 1.0
    assert ref.quantize_weights(w, sw).tolist() == [[50, -127], [0, 0]]
    assert ref.quantize_bias(np.array([0.1, 0.0], np.float32), 0.02, sw).tolist() == [500, 0]


# -------------------------------------------------------------------- NMS ----
ONNX_BOXES = np.array([[[0, 0, 1, 1], [0, 0.1, 1, 1.1], [0, -0.1, 1, 0.9], [0, 10, 1, 11], [0, 10.1, 1, 11.1],
                        [0, 100, 1, 101]]], np.float32)
ONNX_SCORES = np.array([[[0.9, 0.75, 0.6, 0.95, 0.5, 0.3]]], np.float32)


def test_nms_onnx_published_examples(ref):
    sel = lambda o: [r[2] for r in o.tolist() if r[2] >= 0]
    assert sel(ref.nms(ONNX_BOXES, ONNX_SCORES, 3, 0.5, 0.0)) == [3, 0, 5]          # suppress_by_IOU
    assert sel(ref.nms(ONNX_BOXES, ONNX_SCORES, 3, 0.5, 0.4)) == [3, 0]             # ..._and_scores
    assert sel(ref.nms(ONNX_BOXES, ONNX_SCORES, 2, 0.5, 0.0)) == [3, 0]             # limit_output_size
    flipped = np.array([[[1, 1, 0, 0], [0, 0.1, 1, 1.1], [0, 0.9, 1, -0.1], [0, 10, 1, 11], [1, 10.1, 0, 11.1],
                         [1, 101, 0, 100]]], np.float32)
    assert sel(ref.nms(flipped, ONNX_SCORES, 3, 0.5, 0.0)) == [3, 0, 5]             # flipped_coordinates
    same = np.tile(np.array([0, 0, 1, 1], np.float32), (1, 10, 1))
    assert sel(ref.nms(same, np.full((1, 1, 10), 0.9, np.float32), 3, 0.5, 0.0)) == [0]   # identical_boxes
    two = np.concatenate([ONNX_BOXES, ONNX_BOXES])
    out = ref.nms(two, np.concatenate([ONNX_SCORES, ONNX_SCORES]), 2, 0.5, 0.0)
    assert out.tolist() == [[0, 0, 3], [0, 0, 0], [1, 0, 3], [1, 0, 0]]             # two_batches


def test_nms_against_brute_force(ref):
    """Sequential restatement of the reference selection loop (dnnl_utils_avx512.h:1020-1070)
    in float64-free plain Python on 48 boxes, plus the invariants of the result."""
    r = rng(9)
    B, C = 48, 3
    cy, cx = r.random(B) * 4, r.random(B) * 4
    boxes = np.stack([cy - 0.5, cx - 0.5, cy + 0.5, cx + 0.5], -1).astype(np.float32)[None]
    scores = r.random((1, C, B)).astype(np.float32)

    def iou(a, b):
        f = np.float32
        ai = f(f(a[2] - a[0]) * f(a[3] - a[1]))
        aj = f(f(b[2] - b[0]) * f(b[3] - b[1]))
        if ai <= 0 or aj <= 0:
            return f(0)
        ih = max(f(min(a[2], b[2]) - max(a[0], b[0])), f(0))
        iw = max(f(min(a[3], b[3]) - max(a[1], b[1])), f(0))
        inter = f(ih * iw)
        return f(inter / f(f(ai + aj) - inter))

    cand = []
    for b in range(B):
        c = int(np.argmax(scores[0, :, b]))
        if scores[0, c, b] > 0.3:
            cand.append((-float(scores[0, c, b]), b, c))
    cand.sort()
    kept = []
    for _, b, c in cand:
        if len(kept) >= 10:
            break
        if all(iou(boxes[0, b], boxes[0, kb]) < np.float32(0.45) for kb, _ in kept):
            kept.append((b, c))
    out = ref.nms(boxes, scores, 10, 0.45, 0.3)
    got = [(r_[2], r_[1]) for r_ in out.tolist() if r_[2] >= 0]
    assert got == kept
    for i in range(len(got)):
        for j in range(i):
            assert iou(boxes[0, got[i][0]], boxes[0, got[j][0]]) < 0.45


# -------------------------------------------------------- live reference ----
# ------------------------------------ more of the reference's own fp32 kernels ----
def test_batchnorm_against_reference_kernel_vectors(ref):
    rb = ref.RefBuilder({})
    y = rb.batchnorm(GOLD["bn_x"], GOLD["bn_mean"], GOLD["bn_var"], 1e-3, GOLD["bn_scale"], GOLD["bn_offset"])
    want = GOLD["bn_y"]
    assert np.max(np.abs(y - want)) <= 1e-5 * np.max(np.abs(want))


@pytest.mark.parametrize("i", range(3))
def test_batched_gemm_against_reference_kernel_vectors(ref, i):
    ta, tb = GOLD["bmm%d_attr" % i]
    rb = ref.RefBuilder({})
    y = rb.gemm(GOLD["bmm%d_a" % i], GOLD["bmm%d_b" % i], None, bool(ta), bool(tb), 1.0, 0.0)
    want = GOLD["bmm%d_y" % i]
    assert y.shape == want.shape
    assert np.max(np.abs(y - want)) <= 1e-5 * np.max(np.abs(want))


@pytest.mark.parametrize("i", range(4))
def test_reduce_mean_against_reference_kernel_vectors(ref, i):
    rb = ref.RefBuilder({})
    y = rb.reduce_mean(GOLD["reduce_x"], [int(a) for a in GOLD["reduce%d_axes" % i]], keep_dims=True)
    want = GOLD["reduce%d_y" % i]
    assert y.shape == want.shape
    assert np.max(np.abs(y - want)) <= 1e-6


@pytest.mark.parametrize("i", range(3))
def test_argmax_against_reference_kernel_vectors(ref, i):
    rb = ref.RefBuilder({})
    x = GOLD["reduce_x"]
    y = rb.argmax(x, int(GOLD["argmax%d_axis" % i][0]) % x.ndim, keep_dims=False, dtype=np.int64)
    assert np.array_equal(y, GOLD["argmax%d_y" % i])


def test_argmax_first_of_equal_values_like_the_reference_kernel(ref):
    # runtime/generic/reduction.cc of the reference tree keeps the first maximum
    # (strict comparison while walking the axis upwards)
    rb = ref.RefBuilder({})
    x = np.array([[1, 3, 3, 0], [2, 2, 2, 2]], np.float32)
    assert rb.argmax(x, 1, keep_dims=False).tolist() == [1, 0]
    assert rb.argmax(x, 1, keep_dims=False, last=True).tolist() == [2, 3]


def test_data_movement_against_reference_kernel_vectors(ref):
    rb = ref.RefBuilder({})
    x = GOLD["reduce_x"]
    st, sz = GOLD["slice_starts"], GOLD["slice_sizes"]
    assert np.array_equal(rb.slice(x, [int(v) for v in st], [int(a + b) for a, b in zip(st, sz)]), GOLD["slice_y"])
    idx = GOLD["gather_idx"]
    got = rb.gather(GOLD["gather_table"], idx, axis=0)
    assert got.shape == idx.shape + (GOLD["gather_table"].shape[1],)
    assert np.array_equal(got.reshape(idx.size, -1), GOLD["gather_y"])
    for i in range(3):
        assert np.array_equal(rb.transpose(x, [int(p) for p in GOLD["transpose%d_perm" % i]]), GOLD["transpose%d_y" % i])
    top, bottom, left, right = (int(v) for v in GOLD["pad_attr"])
    # the reference kernel pads H and W of a channels-last tensor
    assert np.array_equal(rb.pad(GOLD["pad_x"], [0, top, left, 0], [0, bottom, right, 0]), GOLD["pad_y"])


def test_erf_against_reference_kernel_vectors(ref):
    rb = ref.RefBuilder({})
    assert np.max(np.abs(rb.erf(GOLD["erf_x"]) - GOLD["erf_y"])) <= 2e-7


@pytest.mark.parametrize("name", ["add", "sub", "mul", "div"])
def test_broadcast_arithmetic_against_reference_kernel_vectors(ref, name):
    rb = ref.RefBuilder({})
    y = getattr(rb, name)(GOLD["bin_a"], GOLD["bin_b"])
    want = GOLD["bin_%s_y" % name]
    assert y.shape == want.shape == (2, 3, 5, 4)
    assert np.max(np.abs(y - want)) <= 1e-6 * np.max(np.abs(want))


def test_live_reference_kernels_if_built(ref):
    """When oracle/_ref/libsn_rt.so exists (built from the reference tree), one more
    conv shape is compared live; otherwise the committed vectors above stand in."""
    import ctypes
    path = os.path.join(entry.ROOT, "oracle", "_ref", "libsn_rt.so")
    if not os.path.exists(path):
        pytest.skip("oracle/_ref/libsn_rt.so not built on this machine")
    L = ctypes.CDLL(path)
    r = rng(10)
    x = r.standard_normal((1, 3, 10, 10)).astype(np.float32)
    w = r.standard_normal((4, 3, 3, 3)).astype(np.float32)
    y = np.zeros((1, 4, 5, 5), np.float32)
    f32p, i64 = ctypes.POINTER(ctypes.c_float), ctypes.c_int64
    L._sn_rt_conv2d_f32_nchw.argtypes = [f32p, f32p, f32p] + [i64] * 15
    L._sn_rt_conv2d_f32_nchw(y.ctypes.data_as(f32p), x.ctypes.data_as(f32p), w.ctypes.data_as(f32p),
                             1, 10, 10, 3, 5, 5, 4, 3, 3, 2, 2, 1, 1, 1, 1)
    got = ref.conv2d(x, w, None, (2, 2), (1, 1, 1, 1))
    assert np.max(np.abs(got - y)) <= 1e-5 * np.max(np.abs(y))
