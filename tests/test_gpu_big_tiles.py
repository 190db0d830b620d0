"""The large workgroup tiles of the implicit-GEMM kernel (256x256, 256x128 and
128x256 outputs per workgroup, both operands loaded straight into LDS) are not
picked by the default heuristics; ODLA_HIP_IGEMM_TILE selects one for every
launch whose shape fits it.  Each is held to the same parity bar as the default
kernels: the random convolution sweeps (fp16 / bf16 against the oracle within
the storage tolerance, int8 bit-exact), the int8 requantisation cases and a GEMM
with a fused transcendental activation.
"""
import numpy as np
import pytest

import test_gpu_conv_sweep as sweep
import test_gpu_int8 as q8
from util import announce, run_both

pytestmark = pytest.mark.gpu

TILES = ["big256x256", "big256x128", "big128x256"]


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("mode", ["fp16", "bf16"])
def test_float_convolution_sweep(tile, mode, monkeypatch):
    monkeypatch.setenv("ODLA_HIP_IGEMM_TILE", tile)
    sweep.test_random_convolutions(mode)


@pytest.mark.parametrize("tile", TILES)
def test_int8_convolution_sweep(tile, monkeypatch):
    monkeypatch.setenv("ODLA_HIP_IGEMM_TILE", tile)
    sweep.test_random_convolutions_int8()


@pytest.mark.parametrize("tile", TILES)
def test_int8_requantisation_cases(tile, monkeypatch, odla, ref):
    monkeypatch.setenv("ODLA_HIP_IGEMM_TILE", tile)
    for case in q8.Q8_CONV_CASES:
        q8.test_q8_conv_accumulators_and_requant(case, odla, ref)
    for dims in [(3, 128, 7, 7, 200), (4, 64, 21, 19, 256), (2, 128, 30, 30, 512)]:
        q8.test_q8_residual_fused_equals_unfused_equals_oracle(dims, 0, odla, ref, monkeypatch)


@pytest.mark.parametrize("tile", TILES)
def test_gemm_with_gelu_bf16(tile, monkeypatch, odla):
    """[600, 256] x [256, 520] + bias -> GELU: ragged in both tile directions.  The
    planner's debug log names the kernel it chose for the launch."""
    import ctypes
    monkeypatch.setenv("ODLA_HIP_IGEMM_TILE", tile)
    announce("big tile gemm %s" % tile)
    L = odla.load_library()
    seen = []
    CB = ctypes.CFUNCTYPE(None, ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p)
    cb = CB(lambda f, line, fn, lvl, msg: seen.append(msg.decode()))
    L.odla_SetLogger(ctypes.cast(cb, ctypes.c_void_p))
    L.odla_SetLogLevel(5)   # ODLA_LOG_LEVEL_DEBUG
    try:
        _gemm_with_gelu_bf16()
    finally:
        L.odla_SetLogLevel(2)
        L.odla_SetLogger(None)
    assert any(m.endswith("kernel " + tile[3:]) for m in seen), seen


def _gemm_with_gelu_bf16():
    r = np.random.default_rng(31)
    x = r.standard_normal((600, 256)).astype(np.float32)
    w = (r.standard_normal((256, 520)) * 0.06).astype(np.float32)
    bias = r.standard_normal((520,)).astype(np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        y = b.add(b.gemm(a, b.const("w", w), name="mm"), b.const("bias", bias), name="biased")
        b.output(b.gelu(y, False, name="act"), "y")

    got, want = run_both(build, {"x": x}, bf16=True)
    assert float(np.max(np.abs(got["y"] - want["y"]))) <= 6e-2 * max(1.0, float(np.max(np.abs(want["y"]))))
