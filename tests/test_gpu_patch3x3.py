"""3x3 / stride 1 / padding 1 convolutions on the kernel that keeps a tile's input patch
in LDS (the planner's debug log must name it: "patch3x3"): every block shape the launcher
picks (8, 13, 14, 16, 24, 28 columns), tiles that end past the image, images smaller than
a tile, one to three channel chunks, two and four channel slices per workgroup, bias /
activation / residual epilogues, in fp16, bf16 and int8.

Tolerances: fp16 2e-2 / bf16 6e-2 of max(1, largest expected magnitude) against the fp32
oracle; int8 bit-exact against the oracle's integer accumulation and float requantisation.
"""
import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, run_hip, run_ref
from test_gpu_conv_sweep import builder_for, tensors_for
from test_gpu_taps_kernel import run_logged

pytestmark = pytest.mark.gpu


def case(N, C, H, W, O, tail="none", bias=True):
    return dict(N=N, C=C, H=H, W=W, O=O, kh=3, kw=3, sh=1, sw=1, dh=1, dw=1, pad=[1, 1, 1, 1], group=1, tail=tail, bias=bias)


FLOAT_CASES = [
    case(2, 64, 56, 56, 64, "relu"),          # 8 columns x 4 rows per block, two channel slices
    case(2, 64, 28, 28, 128, "leaky_add"),    # 28 x 1, residual behind the activation
    case(3, 128, 14, 14, 256, "add_relu"),    # 14 x 2, second tile ends past the image, two chunks, two channel tiles
    case(2, 192, 13, 13, 128, "leaky"),       # 13 x 2, three chunks
    case(1, 64, 20, 24, 128, "none", False),  # 24 x 1, no bias
    case(2, 64, 9, 16, 64, "clamp"),          # 16 x 2, most of the second tile is past the image
    case(1, 128, 5, 4, 128, "relu"),          # an image smaller than one block
    case(1, 64, 40, 104, 64, "add"),          # wide image, 8 x 4 blocks
    case(1, 128, 16, 16, 384, "add_relu"),    # three channel tiles (of two wavefronts x two slices with ODLA_HIP_C3_SLICES=2)
    case(2, 64, 12, 28, 512, "leaky"),        # four channel tiles (two of four wavefronts x two slices)
    case(1, 64, 11, 26, 128, "add_relu"),     # 26 columns in one block of 32 that hangs over the right edge
    case(2, 128, 6, 30, 128, "leaky_add"),    # 30 of 32
]

INT8_CASES = [
    case(2, 64, 56, 56, 64, "relu"),          # 64-byte pixel rows: chunks of two K steps
    case(2, 128, 28, 28, 128, "relu"),
    case(3, 256, 14, 14, 256, "none"),
    case(2, 64, 13, 13, 128, "relu"),
    case(1, 128, 9, 16, 64, "none"),
    case(1, 64, 16, 16, 256, "relu"),         # 64-byte rows
    case(2, 256, 10, 28, 512, "relu"),
    case(1, 128, 11, 26, 128, "relu"),        # a block of 32 columns over a 26-column image
    case(2, 64, 7, 30, 128, "none"),
]


@pytest.mark.parametrize("mode", ["fp16", "bf16"])
@pytest.mark.parametrize("slices", ["", "2"])
def test_patch_kernel_float(mode, slices, monkeypatch):
    monkeypatch.setenv("ODLA_HIP_C3_MIN_FILL", "0")
    if slices:
        monkeypatch.setenv("ODLA_HIP_C3_SLICES", slices)   # two 32-channel slices per wavefront
    kw = {"fp16": mode == "fp16", "bf16": mode == "bf16"}
    for i, c in enumerate(FLOAT_CASES):
        announce("patch3x3 %s #%d %s" % (mode, i, c))
        x, w, bias, res = tensors_for(c, 5100 + i)
        feeds = {"x": x}
        if "add" in c["tail"]:
            feeds["res"] = res
        build = builder_for(c, w, bias if c["bias"] else None)
        got, seen = run_logged(lambda: run_hip(build, feeds, **kw)["out"])
        assert any(m.endswith("kernel patch3x3") for m in seen), (c, [m for m in seen if "kernel" in m])
        want = run_ref(build, feeds)["out"]
        tol = 2e-2 if mode == "fp16" else 6e-2
        assert float(np.max(np.abs(got - want))) <= tol * max(1.0, float(np.max(np.abs(want)))), (i, c)


@pytest.mark.parametrize("slices", ["", "2"])
def test_patch_kernel_int8(slices, monkeypatch):
    monkeypatch.setenv("ODLA_HIP_C3_MIN_FILL", "0")
    if slices:
        monkeypatch.setenv("ODLA_HIP_C3_SLICES", slices)
    odla = entry.load().odla
    models = entry.load().models
    ref = entry.load_oracle()
    for i, c in enumerate(INT8_CASES):
        announce("patch3x3 int8 #%d %s" % (i, c))
        x, w, bias, _ = tensors_for(c, 5300 + i)
        x = (x * 1.5 + 0.3).astype(np.float32)
        x_rng = (float(x.min()), float(x.max()))
        y_rng = (-6.0, 9.0)
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
        assert any(m.endswith("kernel patch3x3") for m in seen), (c, [m for m in seen if "kernel" in m])
        xq = ref.quantize_act(x, *x_qp)
        q_want, _ = ref.qconv(xq, x_qp, w, bias, y_qp, (1, 1), (1, 1, 1, 1), relu=relu)
        assert np.array_equal(got, ref.dequantize_act(q_want, *y_qp)), (i, c)


def test_patch_kernel_int8_residual(monkeypatch):
    """Conv 3x3 -> Add(residual) -> ReLU fused into the kernel's requantising epilogue."""
    monkeypatch.setenv("ODLA_HIP_C3_MIN_FILL", "0")
    odla = entry.load().odla
    models = entry.load().models
    ref = entry.load_oracle()
    r = np.random.default_rng(77)
    for N, C, H, W, O in [(2, 128, 14, 14, 128), (1, 64, 11, 28, 64)]:
        announce("patch3x3 int8 residual %s" % ((N, C, H, W, O),))
        x = r.standard_normal((N, C, H, W)).astype(np.float32)
        res = (r.standard_normal((N, O, H, W)) * 2).astype(np.float32)
        w = (r.standard_normal((O, C, 3, 3)) * 0.1).astype(np.float32)
        bias = r.standard_normal(O).astype(np.float32)
        ranges = {"x": (float(x.min()), float(x.max())), "res": (float(res.min()), float(res.max())),
                  "c": (-6.0, 6.0), "out": (0.0, 9.0)}
        qp = {k: ref.act_qparams(*v) for k, v in ranges.items()}
        entries = []
        for name, (mn, mx) in ranges.items():
            s, z = models.act_qparams(mn, mx)
            entries.append((name, s, z, mn, mx, None))
        wt = w.reshape(O, -1)
        entries.append(("w", 1.0, 0, float(wt.min()), float(wt.max()), list(zip(wt.min(axis=1).tolist(), wt.max(axis=1).tolist()))))

        def build(b):
            v = b.arg("x", x.shape)
            rr = b.arg("res", res.shape)
            c = b.conv(v, b.const("w", w), b.const("b", bias), (1, 1), (1, 1, 1, 1), name="c")
            b.output(b.relu(b.add(c, rr, name="add"), name="out"), "out")

        got, seen = run_logged(lambda: run_hip(build, {"x": x, "res": res}, quant_table=odla.quant_table(entries))["out"])
        assert any(m.endswith("kernel patch3x3") for m in seen), [m for m in seen if "kernel" in m]
        xq = ref.quantize_act(x, *qp["x"])
        rq = ref.quantize_act(res, *qp["res"])
        fq, _ = ref.qconv(xq, qp["x"], w, bias, qp["out"], (1, 1), (1, 1, 1, 1), relu=True, residual=(rq, qp["res"]))
        assert np.array_equal(got, ref.dequantize_act(fq, *qp["out"]))
