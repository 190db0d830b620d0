"""Pins of the oracle's wider operator surface (no GPU needed): every numpy
restatement is checked against torch's CPU operator of the same name, or
against the defining formula evaluated another way (math library, brute-force
loops).  The reference's portable TopK is unimplemented, so its tie order is
this build's choice and only tie-free inputs are pinned.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F


def rng(seed):
    return np.random.default_rng(seed)


def _rb(ref):
    return ref.RefBuilder({})


def close(a, b, tol=2e-6):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.max(np.abs(a - b)) <= tol * max(1.0, float(np.max(np.abs(b))))


def test_activation_family_against_torch(ref):
    x = (rng(1).standard_normal((4, 33)) * 3).astype(np.float32)
    t = torch.tensor(x)
    b = _rb(ref)
    assert close(b.elu(x, 0.7), F.elu(t, 0.7).numpy())
    assert close(b.selu(x, 1.6732632, 1.0507010), F.selu(t).numpy())
    assert close(b.celu(x, 1.3), F.celu(t, 1.3).numpy())
    assert close(b.hard_sigmoid(x, 1.0 / 6, 0.5), F.hardsigmoid(t).numpy())
    assert close(b.softplus(x), F.softplus(t).numpy())
    assert close(b.softsign(x), F.softsign(t).numpy())
    assert np.array_equal(b.thresholded_relu(x, 0.8), F.threshold(t, 0.8, 0.0).numpy())
    assert close(b.shrink(x, 0.5, 0.5), F.softshrink(t, 0.5).numpy())      # bias == lambd: soft shrink
    assert np.array_equal(b.shrink(x, 0.0, 0.5), F.hardshrink(t, 0.5).numpy())  # bias == 0: hard shrink
    slope = rng(2).random(33).astype(np.float32)
    assert close(b.prelu(x, slope), np.where(x < 0, x * slope, x))
    assert close(b.prelu(x.reshape(1, 4, 33, 1), slope[:4].reshape(4, 1, 1)),
                 F.prelu(t.reshape(1, 4, 33, 1), torch.tensor(slope[:4])).numpy())


def test_trigonometry_against_math_library(ref):
    b = _rb(ref)
    x = np.linspace(-0.95, 0.95, 41, dtype=np.float32)
    for name, f in (("sin", math.sin), ("cos", math.cos), ("tan", math.tan), ("asin", math.asin), ("acos", math.acos),
                    ("atan", math.atan), ("sinh", math.sinh), ("cosh", math.cosh), ("asinh", math.asinh),
                    ("atanh", math.atanh)):
        want = np.array([f(float(v)) for v in x], np.float32)
        assert close(getattr(b, name)(x), want), name
    y = np.linspace(1.0, 9.0, 17, dtype=np.float32)
    assert close(b.acosh(y), np.array([math.acosh(float(v)) for v in y], np.float32))
    assert close(b.reciprocal(y), 1.0 / y)
    z = np.array([-1.5, -0.5, 0.0, 0.5, 1.5, 2.0], np.float32)
    assert b.ceil(z).tolist() == [-1, -0.0, 0, 1, 2, 2] and b.floor(z).tolist() == [-2, -1, 0, 0, 1, 2]
    assert b.sign(z).tolist() == [-1, -1, 0, 1, 1, 1]


def test_mod_matches_python_and_c_semantics(ref):
    b = _rb(ref)
    l = np.array([7, -7, 7, -7, 5, 0], np.int32)
    r = np.array([3, 3, -3, -3, 5, 4], np.int32)
    assert b.mod(l, r).tolist() == [int(a) % int(c) for a, c in zip(l, r)]              # sign of the divisor
    assert b.mod(l, r, fmod=True).tolist() == [int(math.fmod(a, c)) for a, c in zip(l, r)]  # sign of the dividend
    lf = np.array([7.5, -7.5, 7.5, -7.5], np.float32)
    rf = np.array([2.0, 2.0, -2.0, -2.0], np.float32)
    assert b.mod(lf, rf).tolist() == np.mod(lf, rf).tolist()
    assert b.mod(lf, rf, fmod=True).tolist() == np.fmod(lf, rf).tolist()


def test_reductions_against_torch(ref):
    x = (rng(3).random((3, 7, 5)) + 0.25).astype(np.float32)
    t = torch.tensor(x)
    b = _rb(ref)
    assert close(b.reduce_log_sum_exp(x, [1], False), torch.logsumexp(t, 1).numpy())
    assert close(b.reduce_log_sum_exp(x, [1, 2], True), torch.logsumexp(t, (1, 2), keepdim=True).numpy())
    assert close(b.reduce_l2(x, [2], True), torch.linalg.vector_norm(t, 2, 2, keepdim=True).numpy())
    assert close(b.reduce_l1(x, [2], False), torch.linalg.vector_norm(t, 1, 2).numpy())
    assert close(b.reduce_l2(x, [2], False, eps=0.5), np.sqrt((x.astype(np.float64) ** 2).sum(2) + 0.5))
    assert close(b.reduce_prod(x, [1], True), torch.prod(t, 1, keepdim=True).numpy())
    assert np.array_equal(b.reduce_min(x, [0], False), torch.amin(t, 0).numpy())
    assert close(b.reduce_sum_square(x, [1, 2], False), (t * t).sum((1, 2)).numpy())
    assert close(b.reduce_log_sum(x, [1], False), torch.log(t.sum(1)).numpy())


def test_arg_extreme_first_and_last_index(ref):
    b = _rb(ref)
    x = np.array([[1, 5, 5, 2], [3, 3, 0, 0]], np.float32)
    assert b.argmax(x, 1, False).tolist() == [1, 0]
    assert b.argmax(x, 1, False, last=True).tolist() == [2, 1]
    assert b.argmin(x, 1, True).tolist() == [[0], [2]]
    assert b.argmin(x, -1, True, last=True, dtype=np.int64).tolist() == [[0], [3]]
    y = rng(4).standard_normal((3, 9, 4)).astype(np.float32)
    assert np.array_equal(b.argmax(y, 1, False), torch.argmax(torch.tensor(y), 1).numpy())
    # the reference's loop, literally [odla_dnnl_statistics.cc:213-231]
    for last in (False, True):
        for is_max in (True, False):
            want = np.zeros((3, 4), np.int32)
            for i in range(3):
                for j in range(4):
                    val, idx = y[i, 0, j], 0
                    for k in range(1, 9):
                        cur = y[i, k, j]
                        if (is_max and cur > val) or (not is_max and cur < val) or (cur == val and last):
                            val, idx = cur, k
                    want[i, j] = idx
            got = (b.argmax if is_max else b.argmin)(y, 1, False, last=last)
            assert np.array_equal(got, want)


def test_topk_tie_free_against_torch(ref):
    b = _rb(ref)
    x = rng(5).permutation(2 * 11 * 3).reshape(2, 11, 3).astype(np.float32)
    for largest in (True, False):
        v, i = b.topk(x, 4, 1, largest)
        tv, ti = torch.topk(torch.tensor(x), 4, 1, largest=largest)
        assert np.array_equal(v, tv.numpy()) and np.array_equal(i, ti.numpy())


def test_lrn_instance_norm_deconv_against_torch(ref):
    b = _rb(ref)
    x = rng(6).standard_normal((2, 7, 5, 6)).astype(np.float32)
    t = torch.tensor(x)
    assert close(b.lrn(x, 5, 1e-2, 0.75, 1.5), F.local_response_norm(t, 5, 1e-2, 0.75, 1.5).numpy(), 1e-5)
    g, o = rng(7).random(7).astype(np.float32), rng(8).standard_normal(7).astype(np.float32)
    assert close(b.instance_norm(x, 1e-5, g, o), F.instance_norm(t, weight=torch.tensor(g), bias=torch.tensor(o), eps=1e-5).numpy(), 1e-5)
    assert close(b.instance_norm(x, 1e-3, None, None, 2.0, -1.0), F.instance_norm(t, eps=1e-3).numpy() * 2.0 - 1.0, 1e-5)
    for (cin, og, k, s, p, grp, op) in ((4, 3, 3, 2, 1, 1, 0), (4, 3, 3, 2, 1, 2, 1), (6, 2, 4, 2, 1, 3, 0), (3, 5, 2, 1, 0, 1, 0),
                                        (2, 2, 5, 3, 2, 1, 2)):
        xx = rng(9).standard_normal((2, cin, 5, 4)).astype(np.float32)
        w = rng(10).standard_normal((cin, og, k, k)).astype(np.float32)
        bias = rng(11).standard_normal(og * grp).astype(np.float32)
        want = F.conv_transpose2d(torch.tensor(xx), torch.tensor(w), torch.tensor(bias), stride=s, padding=p,
                                  output_padding=op, groups=grp).numpy()
        got = b.deconv(xx, w, bias, (s, s), (p, p, p, p), grp, want.shape[2:] if op else None)
        assert got.shape == want.shape and close(got, want, 1e-5), (cin, og, k, s, p, grp, op)


def test_data_movement_against_numpy(ref):
    b = _rb(ref)
    x = rng(12).standard_normal((2, 3, 4)).astype(np.float32)
    assert np.array_equal(b.pad(x, [1, 0, 2], [0, 2, 1]), F.pad(torch.tensor(x), (2, 1, 0, 2, 1, 0)).numpy())
    assert np.array_equal(b.tile(x, [2, 1, 3]), torch.tensor(x).repeat(2, 1, 3).numpy())
    assert np.array_equal(b.broadcast_to(x[:, :1], (2, 3, 4)), np.broadcast_to(x[:, :1], (2, 3, 4)))
    assert b.squeeze(x[:, :1], [1]).shape == (2, 4)
    assert np.array_equal(b.stack([x, x + 1], 1), torch.stack([torch.tensor(x), torch.tensor(x + 1)], 1).numpy())
    c = rng(13).random((2, 3, 4)) > 0.5
    assert np.array_equal(b.select(c, x, -x), torch.where(torch.tensor(c), torch.tensor(x), torch.tensor(-x)).numpy())
    assert np.array_equal(b.select(c[:, :, :1], x, -x[0]), np.where(c[:, :, :1], x, -x[0]))
    assert close(b.mean([x, x * 2, x * 3 + 1]), (x + x * 2 + x * 3 + 1) / 3)
