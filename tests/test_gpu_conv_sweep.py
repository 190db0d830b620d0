"""Seeded random sweep of convolution shapes and fused tails against the oracle:
every kernel variant (two-operand, weights-in-registers, streaming 1x1, space-to-depth
stems, grouped / depthwise) gets shapes nobody picked by hand - ragged tiles, uneven
paddings and strides, rectangular filters, dilation, bias or none, activation and
residual tails - in fp32, fp16 and bf16, and as int8 with bit-exact requantisation."""
import os
import sys

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, max_rel_err, run_hip, run_ref

pytestmark = pytest.mark.gpu

# ODLA_SWEEP_SEED=<n> shifts every seed below: other random cases, same code (default 0)
SEED0 = int(__import__("os").environ.get("ODLA_SWEEP_SEED", "0"))

sys.path.insert(0, os.path.join(entry.ROOT, "oracle"))

CH_IN = [1, 3, 4, 8, 16, 24, 32, 48, 64, 96, 128, 192, 256]
CH_OUT = [4, 8, 16, 40, 64, 72, 128, 136, 200, 256, 264]


def draw_case(r):
    C = int(r.choice(CH_IN))
    O = int(r.choice(CH_OUT))
    kh, kw = (int(r.choice([1, 1, 3, 3, 5])),) * 2
    if r.random() < 0.2:
        kw = int(r.choice([1, 2, 3, 4]))
    sh, sw = (int(r.choice([1, 1, 2])),) * 2
    if r.random() < 0.15:
        sw = 3 - sh if sh in (1, 2) else sh
    dh = dw = 1 if r.random() < 0.85 else 2
    pad = [int(r.integers(0, 3)) for _ in range(4)]          # top, left, bottom, right
    if r.random() < 0.6:
        pad = [kh // 2 * dh, kw // 2 * dw, kh // 2 * dh, kw // 2 * dw]
    group = 1
    if r.random() < 0.2:
        opts = [g for g in (2, 4, C) if g >= 2 and C % g == 0 and O % g == 0]
        if opts:
            group = int(r.choice(opts))
    N = int(r.integers(1, 5))
    H = int(r.integers(max(5, (kh - 1) * dh + 1), 21))
    W = int(r.integers(max(5, (kw - 1) * dw + 1), 21))
    tail = str(r.choice(["none", "relu", "leaky", "clamp", "add", "add_relu", "leaky_add"]))
    bias = bool(r.random() < 0.7)
    return dict(N=N, C=C, H=H, W=W, O=O, kh=kh, kw=kw, sh=sh, sw=sw, dh=dh, dw=dw, pad=pad, group=group,
                tail=tail, bias=bias)


def out_hw(c):
    ho = (c["H"] + c["pad"][0] + c["pad"][2] - ((c["kh"] - 1) * c["dh"] + 1)) // c["sh"] + 1
    wo = (c["W"] + c["pad"][1] + c["pad"][3] - ((c["kw"] - 1) * c["dw"] + 1)) // c["sw"] + 1
    return ho, wo


def tensors_for(c, seed):
    r = np.random.default_rng(seed)
    cg = c["C"] // c["group"]
    w = (r.standard_normal((c["O"], cg, c["kh"], c["kw"])) * np.sqrt(2.0 / (cg * c["kh"] * c["kw"]))).astype(np.float32)
    b = r.standard_normal(c["O"]).astype(np.float32) if c["bias"] else None
    x = r.standard_normal((c["N"], c["C"], c["H"], c["W"])).astype(np.float32)
    ho, wo = out_hw(c)
    res = r.standard_normal((c["N"], c["O"], ho, wo)).astype(np.float32)
    return x, w, b, res


def builder_for(c, w, bias, with_res_arg=True):
    ho, wo = out_hw(c)

    def build(b):
        v = b.arg("x", (c["N"], c["C"], c["H"], c["W"]))
        y = b.conv(v, b.const("w", w), b.const("b", bias) if bias is not None else None, (c["sh"], c["sw"]),
                   tuple(c["pad"]), (c["dh"], c["dw"]), c["group"], name="y")
        t = c["tail"]
        if t in ("relu",):
            y = b.relu(y, name="t")
        elif t == "leaky":
            y = b.leaky_relu(y, 0.1, name="t")
        elif t == "clamp":
            y = b.clamp(y, -0.5, 0.75, name="t")
        elif t in ("add", "add_relu"):
            y = b.add(y, b.arg("res", (c["N"], c["O"], ho, wo)), name="s")
            if t == "add_relu":
                y = b.relu(y, name="t")
        elif t == "leaky_add":
            y = b.add(b.leaky_relu(y, 0.1, name="l"), b.arg("res", (c["N"], c["O"], ho, wo)), name="t")
        b.output(y, "out")
    return build


def cases(seed, count):
    r = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        c = draw_case(r)
        ho, wo = out_hw(c)
        if ho >= 1 and wo >= 1:
            out.append(c)
    return out


@pytest.mark.parametrize("mode", ["fp32", "fp16", "bf16"])
def test_random_convolutions(mode):
    kw = {"fp16": mode == "fp16", "bf16": mode == "bf16"}
    for i, c in enumerate(cases(SEED0 + 2024, 60)):
        announce("sweep %s #%d %s" % (mode, i, c))
        x, w, bias, res = tensors_for(c, 500 + i)
        feeds = {"x": x}
        if "add" in c["tail"]:
            feeds["res"] = res
        build = builder_for(c, w, bias)
        got = run_hip(build, feeds, **kw)["out"]
        want = run_ref(build, feeds)["out"]
        assert got.shape == want.shape
        if mode == "fp32":
            assert max_rel_err(got, want) <= 1e-4, (i, c)
        else:
            tol = 2e-2 if mode == "fp16" else 6e-2
            assert float(np.max(np.abs(got - want))) <= tol * max(1.0, float(np.max(np.abs(want)))), (i, c)


def test_random_convolutions_int8():
    """Quant-table plan: conv (+ReLU) requantised to 8 bits, bit-exact against the oracle's
    integer accumulation and float requantisation."""
    odla = entry.load().odla
    models = entry.load().models
    ref = entry.load_oracle()
    done, wanted = 0, 30
    for i, c in enumerate(cases(SEED0 + 777, 1000)):
        if done == wanted:
            break
        if c["group"] != 1 or c["dh"] != 1 or c["dw"] != 1:
            continue        # the 8-bit plan covers dense, undilated convolutions; the rest stays in float
        if c["pad"][0] != c["pad"][2] or c["pad"][1] != c["pad"][3] or c["kh"] != c["kw"] or c["sh"] != c["sw"]:
            continue        # (the oracle's qconv takes one stride and symmetric paddings)
        c = dict(c, tail="relu" if c["tail"] in ("relu", "add_relu") else "none", bias=True)
        announce("sweep int8 #%d %s" % (i, c))
        x, w, bias, _ = tensors_for(c, 900 + i)
        x = (x * 1.5 + 0.3).astype(np.float32)
        x_rng = (float(x.min()), float(x.max()))
        y_rng = (-2.5, 4.0)
        x_qp, y_qp = ref.act_qparams(*x_rng), ref.act_qparams(*y_rng)
        relu = c["tail"] == "relu"
        out_name = "t" if relu else "y"
        entries = []
        for name, (mn, mx) in (("x", x_rng), (out_name, y_rng)):
            s, z = models.act_qparams(mn, mx)
            entries.append((name, s, z, mn, mx, None))
        wt = w.reshape(w.shape[0], -1)
        entries.append(("w", 1.0, 0, float(wt.min()), float(wt.max()),
                        list(zip(wt.min(axis=1).tolist(), wt.max(axis=1).tolist()))))
        table = odla.quant_table(entries)
        got = run_hip(builder_for(c, w, bias), {"x": x}, quant_table=table)["out"]
        xq = ref.quantize_act(x, *x_qp)
        q_want, _ = ref.qconv(xq, x_qp, w, bias, y_qp, (c["sh"], c["sw"]), tuple(c["pad"]), relu=relu)
        want = ref.dequantize_act(q_want, *y_qp)
        assert np.array_equal(got, want), (i, c)
        done += 1
    announce("sweep int8: %d eligible shapes ran (seed %d)" % (done, SEED0 + 777))
    assert done == wanted   # shapes are drawn until that many eligible ones have run
