"""Tensors with more than 2^31 elements: element offsets beyond 32 bits in the
streaming kernels, the layout conversions and the convolution's output addressing.
Results are checked on slices taken from the start, the middle and the very end."""
import numpy as np
import pytest

from util import announce, run_hip

pytestmark = pytest.mark.gpu


def samples(n_img):
    return sorted({0, n_img // 2, n_img - 1})


def test_elementwise_and_1x1_convolution_beyond_2g_elements():
    N, C, H, W = 66, 8, 2048, 2048          # 2.2e9 elements per tensor
    assert N * C * H * W > 2 ** 31
    announce("large: %d x %d x %d x %d" % (N, C, H, W))
    r = np.random.default_rng(0)
    x = np.empty((N, C, H, W), np.float32)
    plane = r.standard_normal((C, H, W)).astype(np.float32)
    for n in range(N):                      # cheap to make, different per image
        np.multiply(plane, np.float32(1.0 + 0.01 * n), out=x[n])
    w = (r.standard_normal((C, C, 1, 1)) * 0.4).astype(np.float32)
    bias = r.standard_normal(C).astype(np.float32)

    def build(b):
        v = b.arg("x", (N, C, H, W))
        a = b.relu(v, name="r")                                  # row-major streaming kernel
        b.output(a, "r")
        y = b.conv(a, b.const("w", w), b.const("b", bias), (1, 1), (0, 0, 0, 0), name="y")   # NCHW -> NHWC -> conv
        z = b.add(y, a, name="z")                                # channels-last streaming kernel
        b.output(z, "z")                                         # NHWC -> NCHW on the way out

    got = run_hip(build, {"x": x}, fp16=True)
    for n in samples(N):
        xr = np.maximum(x[n].astype(np.float16).astype(np.float32), 0)
        assert np.array_equal(got["r"][n], xr), n
        want = np.tensordot(w[:, :, 0, 0], xr, axes=([1], [0])) + bias.reshape(C, 1, 1) + xr
        assert float(np.max(np.abs(got["z"][n] - want))) <= 2e-2 * max(1.0, float(np.max(np.abs(want)))), n
