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
    np.savez(os.path.join(HERE, "sn_rt_vectors.npz"), **out)
    print("wrote %d arrays" % len(out))


if __name__ == "__main__":
    main()
