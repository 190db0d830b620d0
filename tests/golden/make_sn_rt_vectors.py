"""Writes tests/golden/sn_rt_vectors.npz: input/output vectors of the
reference's own dependency-free fp32 kernels (runtime/generic/**/*.cc of the
reference tree, compiled by oracle/Makefile to oracle/_ref/libsn_rt.so).

Run in a container that has the reference tree:
    make -C oracle && python tests/golden/make_sn_rt_vectors.py
The committed .npz holds data only (seeded random inputs and the outputs the
reference kernels produced for them).
"""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB = ctypes.CDLL(os.path.join(ROOT, "oracle", "_ref", "libsn_rt.so"))

f32p = ctypes.POINTER(ctypes.c_float)
i64 = ctypes.c_int64


def fp(a):
    return a.ctypes.data_as(f32p)


def conv_nchw(x, w, stride, pad):
    N, C, H, W = x.shape
    O, _, R, S = w.shape
    Ho = (H + 2 * pad - R) // stride + 1
    Wo = (W + 2 * pad - S) // stride + 1
    y = np.zeros((N, O, Ho, Wo), np.float32)
    LIB._sn_rt_conv2d_f32_nchw.argtypes = [f32p, f32p, f32p] + [i64] * 15
    LIB._sn_rt_conv2d_f32_nchw(fp(y), fp(x), fp(w), N, H, W, C, Ho, Wo, O, R, S, stride, stride, pad, pad, pad, pad)
    return y


def maxpool_nchw(x, k, stride, pad):
    N, C, H, W = x.shape
    Ho = (H + 2 * pad - k) // stride + 1
    Wo = (W + 2 * pad - k) // stride + 1
    y = np.zeros((N, C, Ho, Wo), np.float32)
    LIB._sn_rt_poolingmax_f32_nchw.argtypes = [f32p, f32p] + [i64] * 14
    LIB._sn_rt_poolingmax_f32_nchw(fp(y), fp(x), N, H, W, C, Ho, Wo, k, k, stride, stride, pad, pad, pad, pad)
    return y


def softmax_last(x):
    y = np.zeros_like(x)
    shape = (ctypes.c_int64 * x.ndim)(*x.shape)
    LIB._sn_rt_softmax_f32.argtypes = [f32p, f32p, ctypes.POINTER(ctypes.c_int64), ctypes.c_int32, ctypes.c_int32, i64]
    LIB._sn_rt_softmax_f32(fp(y), fp(x), shape, x.ndim - 1, x.ndim, x.size)
    return y


def gemm(a, b, c, ta, tb, alpha, beta):
    M = a.shape[1] if ta else a.shape[0]
    N = b.shape[0] if tb else b.shape[1]
    y = np.zeros((M, N), np.float32)
    LIB._sn_rt_gemm_f32.argtypes = [f32p, f32p, f32p, f32p] + [i64] * 5 + [ctypes.c_bool, ctypes.c_bool,
                                                                          ctypes.c_float, ctypes.c_float]
    LIB._sn_rt_gemm_f32(fp(y), fp(a), fp(b), fp(c), a.shape[0], a.shape[1], b.shape[0], b.shape[1], c.size,
                        ta, tb, alpha, beta)
    return y


i32p = ctypes.POINTER(ctypes.c_int32)
i64p = ctypes.POINTER(ctypes.c_int64)


def shape64(shape):
    return (ctypes.c_int64 * len(shape))(*shape)


def batchnorm_nchw(x, mean, var, offset, scale, eps):
    N, C, H, W = x.shape
    y = np.zeros_like(x)
    LIB._sn_rt_bn_f32_nchw.argtypes = [f32p] * 6 + [i64] * 4 + [ctypes.c_bool, ctypes.c_bool, ctypes.c_float, ctypes.c_float]
    LIB._sn_rt_bn_f32_nchw(fp(y), fp(x), fp(mean), fp(var), fp(offset), fp(scale), N, H, W, C, False, False, eps, 1.0)
    return y


def batch_matmul(a, b, ta, tb):
    batches = a.shape[0]
    M = a.shape[2] if ta else a.shape[1]
    N = b.shape[1] if tb else b.shape[2]
    y = np.zeros((batches, M, N), np.float32)
    LIB._sn_rt_batch_matmul_f32.argtypes = [f32p, f32p, f32p] + [i64] * 5 + [ctypes.c_bool, ctypes.c_bool]
    LIB._sn_rt_batch_matmul_f32(fp(y), fp(a), fp(b), batches, a.shape[1], a.shape[2], b.shape[1], b.shape[2], ta, tb)
    return y


def reduce_mean(x, axes):
    out_shape = [1 if i in axes else d for i, d in enumerate(x.shape)]
    y = np.zeros(out_shape, np.float32)
    ax = (ctypes.c_int32 * len(axes))(*axes)
    LIB._sn_rt_reduce_mean_f32.argtypes = [f32p, f32p, i64p, i32p, i64, ctypes.c_int32, ctypes.c_int32]
    LIB._sn_rt_reduce_mean_f32(fp(y), fp(x), shape64(x.shape), ax, x.size, x.ndim, len(axes))
    return y


def argmax(x, axis):
    out_shape = [d for i, d in enumerate(x.shape) if i != axis % x.ndim]
    y = np.zeros(out_shape, np.int64)
    ax = (ctypes.c_int32 * 1)(axis)
    LIB._sn_rt_argmax_f32.argtypes = [i64p, f32p, i64p, i32p, i64, ctypes.c_int32, ctypes.c_int32]
    LIB._sn_rt_argmax_f32(y.ctypes.data_as(i64p), fp(x), shape64(x.shape), ax, x.size, x.ndim, 1)
    return y


def slice_(x, starts, sizes):
    y = np.zeros(sizes, np.float32)
    st = (ctypes.c_int * len(starts))(*starts)
    sz = (ctypes.c_int * len(sizes))(*sizes)
    LIB._sn_rt_slice_f32.argtypes = [f32p, f32p, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int), i64p, ctypes.c_int]
    LIB._sn_rt_slice_f32(fp(y), fp(x), st, sz, shape64(x.shape), x.ndim)
    return y


def gather_rows(table, idx):
    y = np.zeros((idx.size, table.shape[1]), np.float32)
    ii = np.ascontiguousarray(idx, np.int32)
    LIB._sn_rt_gather_f32.argtypes = [f32p, f32p, ctypes.POINTER(ctypes.c_int), i64, i64]
    LIB._sn_rt_gather_f32(fp(y), fp(table), ii.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), table.shape[1], idx.size)
    return y


def transpose(x, perm):
    y = np.zeros([x.shape[p] for p in perm], np.float32)
    pm = (ctypes.c_int * len(perm))(*perm)
    LIB._sn_rt_transpose_f32.argtypes = [f32p, f32p, ctypes.POINTER(ctypes.c_int), i64p, ctypes.c_int]
    LIB._sn_rt_transpose_f32(fp(y), fp(x), pm, shape64(x.shape), x.ndim)
    return y


def erf(x):
    y = np.zeros_like(x)
    LIB._sn_rt_erf_f32.argtypes = [f32p, f32p, i64]
    LIB._sn_rt_erf_f32(fp(y), fp(x), x.size)
    return y


def binary(name, a, b):
    """add / sub / mul / div with the reference's broadcast (shapes of equal rank)."""
    out_shape = tuple(max(p, q) for p, q in zip(a.shape, b.shape))
    y = np.zeros(out_shape, np.float32)
    fn = getattr(LIB, "_sn_rt_%s_f32" % name)
    fn.argtypes = [f32p, f32p, f32p, i64, ctypes.c_bool, i64p, i64p, i64p, ctypes.c_int32]
    fn(fp(y), fp(a), fp(b), y.size, a.shape != b.shape, shape64(out_shape), shape64(a.shape), shape64(b.shape), len(out_shape))
    return y


def pad_hw_nhwc(x, top, bottom, left, right):
    N, H, W, C = x.shape
    y = np.full((N, H + top + bottom, W + left + right, C), np.nan, np.float32)
    pads = (ctypes.c_int32 * 8)(0, 0, top, bottom, left, right, 0, 0)
    LIB._sn_rt_pad_f32.argtypes = [f32p, f32p, ctypes.c_int, i64p, i32p]
    LIB._sn_rt_pad_f32(fp(y), fp(x), 4, shape64(x.shape), pads)
    return y


def more(rng, out):
    x = rng.standard_normal((2, 5, 4, 3)).astype(np.float32)
    mean, var = rng.standard_normal(5).astype(np.float32), (rng.random(5) + 0.5).astype(np.float32)
    offset, scale = rng.standard_normal(5).astype(np.float32), rng.standard_normal(5).astype(np.float32)
    out["bn_x"], out["bn_mean"], out["bn_var"], out["bn_offset"], out["bn_scale"] = x, mean, var, offset, scale
    out["bn_y"] = batchnorm_nchw(x, mean, var, offset, scale, 1e-3)
    for i, (ta, tb) in enumerate([(False, False), (False, True), (True, False)]):
        a = rng.standard_normal((3, 6, 4) if ta else (3, 4, 6)).astype(np.float32)
        b = rng.standard_normal((3, 5, 6) if tb else (3, 6, 5)).astype(np.float32)
        out["bmm%d_a" % i], out["bmm%d_b" % i] = a, b
        out["bmm%d_attr" % i] = np.array([ta, tb], np.int64)
        out["bmm%d_y" % i] = batch_matmul(a, b, ta, tb)
    x = rng.standard_normal((2, 3, 5, 4)).astype(np.float32)
    out["reduce_x"] = x
    for i, axes in enumerate([(1,), (3,), (2, 3), (0, 2)]):
        out["reduce%d_axes" % i] = np.array(axes, np.int64)
        out["reduce%d_y" % i] = reduce_mean(x, list(axes))
    for i, axis in enumerate([0, 2, -1]):
        out["argmax%d_axis" % i] = np.array([axis], np.int64)
        out["argmax%d_y" % i] = argmax(x, axis)
    out["slice_starts"], out["slice_sizes"] = np.array([1, 0, 2, 1], np.int64), np.array([1, 2, 3, 2], np.int64)
    out["slice_y"] = slice_(x, [1, 0, 2, 1], [1, 2, 3, 2])
    table = rng.standard_normal((9, 6)).astype(np.float32)
    idx = np.array([[3, 0, 8], [8, 8, 1]], np.int32)
    out["gather_table"], out["gather_idx"], out["gather_y"] = table, idx, gather_rows(table, idx)
    for i, perm in enumerate([(0, 2, 3, 1), (3, 1, 0, 2), (1, 0, 2, 3)]):
        out["transpose%d_perm" % i] = np.array(perm, np.int64)
        out["transpose%d_y" % i] = transpose(x, perm)
    e = (rng.standard_normal(64) * 2).astype(np.float32)
    out["erf_x"], out["erf_y"] = e, erf(e)
    a = rng.standard_normal((2, 3, 1, 4)).astype(np.float32)
    b = (rng.standard_normal((1, 3, 5, 1)) + 3).astype(np.float32)
    out["bin_a"], out["bin_b"] = a, b
    for name in ("add", "sub", "mul", "div"):
        out["bin_%s_y" % name] = binary(name, a, b)
    p = rng.standard_normal((2, 3, 4, 5)).astype(np.float32)     # NHWC
    out["pad_x"], out["pad_attr"] = p, np.array([1, 2, 0, 3], np.int64)
    out["pad_y"] = pad_hw_nhwc(p, 1, 2, 0, 3)


def main():
    rng = np.random.default_rng(20240)
    out = {}
    conv_cases = [(1, 3, 9, 9, 4, 1, 1, 0), (2, 4, 8, 8, 6, 3, 1, 1), (1, 3, 12, 12, 5, 3, 2, 1),
                  (1, 2, 14, 14, 3, 7, 2, 3), (2, 5, 6, 6, 7, 3, 1, 0)]
    for i, (N, C, H, W, O, k, s, p) in enumerate(conv_cases):
        x = rng.standard_normal((N, C, H, W)).astype(np.float32)
        w = rng.standard_normal((O, C, k, k)).astype(np.float32)
        out["conv%d_x" % i], out["conv%d_w" % i] = x, w
        out["conv%d_attr" % i] = np.array([s, p], np.int64)
        out["conv%d_y" % i] = conv_nchw(x, w, s, p)
    # the reference max pool treats padding as 0, so only unpadded cases (or
    # non-negative data) are comparable with the ODLA semantics
    pool_cases = [(1, 3, 8, 8, 2, 2, 0), (2, 2, 9, 9, 3, 2, 0), (1, 4, 7, 7, 3, 1, 0)]
    for i, (N, C, H, W, k, s, p) in enumerate(pool_cases):
        x = rng.standard_normal((N, C, H, W)).astype(np.float32)
        out["pool%d_x" % i] = x
        out["pool%d_attr" % i] = np.array([k, s, p], np.int64)
        out["pool%d_y" % i] = maxpool_nchw(x, k, s, p)
    for i, shape in enumerate([(4, 10), (3, 5, 17)]):
        x = (rng.standard_normal(shape) * 4).astype(np.float32)
        out["softmax%d_x" % i] = x
        out["softmax%d_y" % i] = softmax_last(x)
    gemm_cases = [(5, 7, 3, False, False, 1.0, 1.0), (4, 6, 8, False, True, 0.5, 2.0), (6, 5, 4, True, False, 1.0, 1.0)]
    for i, (M, K, N, ta, tb, alpha, beta) in enumerate(gemm_cases):
        a = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
        b = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
        c = rng.standard_normal((N,)).astype(np.float32)
        out["gemm%d_a" % i], out["gemm%d_b" % i], out["gemm%d_c" % i] = a, b, c
        out["gemm%d_attr" % i] = np.array([ta, tb, alpha, beta], np.float64)
        out["gemm%d_y" % i] = gemm(a, b, c, ta, tb, alpha, beta)
    more(np.random.default_rng(20241), out)
    np.savez(os.path.join(HERE, "sn_rt_vectors.npz"), **out)
    print("wrote %d arrays" % len(out))


if __name__ == "__main__":
    main()
