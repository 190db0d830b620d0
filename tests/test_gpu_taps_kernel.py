"""Network stems: convolutions over three or four input channels in one or two
16-byte vectors per tap, or over their space-to-depth form.  The 8-bit 7x7
stride-2 stem (16 taps of one vector after space-to-depth) runs on the
short-tap streaming kernel - the planner's debug log must name it ("128x64t")
- with ragged pixel tiles, borders on every side, few and many output channels
and several pixel tiles per workgroup; the other stem shapes, in 8 and 16 bits,
are checked on whichever kernel serves them.

Tolerances: fp16 2e-2 / bf16 6e-2 of max(1, largest expected magnitude); int8
bit-exact against the oracle's integer accumulation and float requantisation.
"""
import ctypes

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, run_hip, run_ref
from test_gpu_conv_sweep import builder_for, tensors_for

pytestmark = pytest.mark.gpu


def case(N, C, H, W, O, k, s, pad, tail="none", bias=True):
    return dict(N=N, C=C, H=H, W=W, O=O, kh=k, kw=k, sh=s, sw=s, dh=1, dw=1, pad=list(pad), group=1, tail=tail, bias=bias)


FLOAT_CASES = [
    case(2, 3, 31, 29, 32, 3, 1, (1, 1, 1, 1), "leaky"),        # first layer of a detector: 3x3, 3 -> 32
    case(1, 3, 40, 40, 64, 3, 1, (1, 1, 1, 1), "relu"),
    case(3, 4, 17, 23, 72, 3, 1, (0, 2, 1, 0), "add_relu"),     # two channel tiles, uneven padding, residual
    case(2, 8, 19, 19, 128, 3, 2, (1, 1, 1, 1), "none", False),  # stride 2 without space-to-depth (8 channels)
    case(2, 3, 45, 37, 64, 7, 2, (3, 3, 3, 3), "relu"),         # 7x7 stride 2: 4x4 taps over 12 channels
    case(1, 3, 224, 224, 64, 7, 2, (3, 3, 3, 3), "relu"),       # the ResNet stem at full image size
    case(5, 1, 9, 11, 8, 3, 1, (1, 1, 1, 1), "clamp"),          # one input channel, eight results, tiny image
]


def run_logged(fn):
    odla = entry.load().odla
    L = odla.load_library()
    seen = []
    CB = ctypes.CFUNCTYPE(None, ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p)
    cb = CB(lambda f, line, fn_, lvl, msg: seen.append(msg.decode()))
    L.odla_SetLogger(ctypes.cast(cb, ctypes.c_void_p))
    L.odla_SetLogLevel(5)
    try:
        out = fn()
    finally:
        L.odla_SetLogLevel(2)
        L.odla_SetLogger(None)
    return out, seen


@pytest.mark.parametrize("mode", ["fp16", "bf16"])
@pytest.mark.parametrize("tiles", ["", "1", "3"])
def test_stem_shapes_float(mode, tiles, monkeypatch):
    if tiles:
        monkeypatch.setenv("ODLA_HIP_LEAN_TILES", tiles)
    kw = {"fp16": mode == "fp16", "bf16": mode == "bf16"}
    for i, c in enumerate(FLOAT_CASES):
        if tiles and c["H"] > 100:
            continue
        announce("stem %s tiles=%s #%d %s" % (mode, tiles or "auto", i, c))
        x, w, bias, res = tensors_for(c, 4100 + i)
        feeds = {"x": x}
        if "add" in c["tail"]:
            feeds["res"] = res
        build = builder_for(c, w, bias)
        got = run_hip(build, feeds, **kw)["out"]
        want = run_ref(build, feeds)["out"]
        tol = 2e-2 if mode == "fp16" else 6e-2
        assert float(np.max(np.abs(got - want))) <= tol * max(1.0, float(np.max(np.abs(want)))), (i, c)


INT8_CASES = [
    case(2, 3, 45, 37, 64, 7, 2, (3, 3, 3, 3), "relu"),      # 4x4 taps of 16 bytes
    case(1, 3, 224, 224, 64, 7, 2, (3, 3, 3, 3), "relu"),
    case(3, 4, 33, 20, 40, 7, 2, (3, 3, 3, 3), "none"),
    case(2, 3, 31, 29, 32, 3, 1, (1, 1, 1, 1), "relu"),      # 3x3 taps, nine units (the tenth is padding)
    case(2, 16, 18, 18, 128, 3, 1, (1, 1, 1, 1), "none"),
    case(4, 8, 15, 21, 72, 3, 2, (1, 1, 1, 1), "relu"),
    case(2, 3, 27, 27, 16, 5, 2, (2, 2, 2, 2), "relu"),      # 5x5 stride 2: 3x3 taps after space-to-depth
]


@pytest.mark.parametrize("tiles", ["", "2"])
def test_short_tap_kernel_int8(tiles, monkeypatch):
    if tiles:
        monkeypatch.setenv("ODLA_HIP_LEAN_TILES", tiles)
    odla = entry.load().odla
    models = entry.load().models
    ref = entry.load_oracle()
    for i, c in enumerate(INT8_CASES):
        if tiles and c["H"] > 100:
            continue
        announce("short taps int8 tiles=%s #%d %s" % (tiles or "auto", i, c))
        x, w, bias, _ = tensors_for(c, 4300 + i)
        x = (x * 1.5 + 0.3).astype(np.float32)
        x_rng = (float(x.min()), float(x.max()))
        y_rng = (-2.5, 4.0)
        x_qp, y_qp = ref.act_qparams(*x_rng), ref.act_qparams(*y_rng)
        relu = c["tail"] == "relu"
        entries = []
        for name, (mn, mx) in (("x", x_rng), ("t" if relu else "y", y_rng)):
            s, z = models.act_qparams(mn, mx)
            entries.append((name, s, z, mn, mx, None))
        wt = w.reshape(w.shape[0], -1)
        entries.append(("w", 1.0, 0, float(wt.min()), float(wt.max()),
                        list(zip(wt.min(axis=1).tolist(), wt.max(axis=1).tolist()))))
        table = odla.quant_table(entries)
        got, seen = run_logged(lambda: run_hip(builder_for(c, w, bias), {"x": x}, quant_table=table)["out"])
        if c["kh"] == 7:
            assert any(m.endswith("kernel 128x64t") for m in seen), (c, [m for m in seen if "kernel" in m])
        xq = ref.quantize_act(x, *x_qp)
        q_want, _ = ref.qconv(xq, x_qp, w, bias, y_qp, (c["sh"], c["sw"]), tuple(c["pad"]), relu=relu)
        want = ref.dequantize_act(q_want, *y_qp)
        assert np.array_equal(got, want), (i, c)
