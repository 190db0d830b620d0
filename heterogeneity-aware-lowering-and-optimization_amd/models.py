"""Graph descriptions of the benchmark configurations, written once against the
builder vocabulary shared by ``HipBuilder`` (GPU, through the ODLA C ABI) and
the CPU oracle's ``RefBuilder``.

Every ``build_*`` function takes a builder and a dict of weights (numpy) and
emits the same ODLA call sequence HALO-generated code would emit for the model:
``odla_CreateArgument`` / ``odla_CreateConstant`` / ``odla_<Op>`` /
``odla_SetValueAsOutput``.  Weights are synthetic (seeded), shaped like the
real architectures.
"""
import numpy as np


# ---------------------------------------------------------------------------
# C0: softmax regression of the reference's mnist_simple graph
#     (Gemm + Add + Softmax; docs/mnist_sample.md:22-56 of the reference tree)
# ---------------------------------------------------------------------------
def mnist_weights(seed=42):
    rng = np.random.default_rng(seed)
    return {"V": (rng.standard_normal((784, 10)) * 0.05).astype(np.float32),
            "V1": np.zeros((1, 10), np.float32)}


def mnist_input(batch=64, seed=1234):
    rng = np.random.default_rng(seed)
    return {"x": rng.random((batch, 784), dtype=np.float32)}


def build_mnist(b, w, batch=64):
    x = b.arg("x", (batch, 784))
    V = b.const("V", w["V"])
    V1 = b.const("V1", w["V1"])
    mm = b.gemm(x, V, None, False, False, 1.0, 0.0, name="MatMul")
    add = b.add(mm, V1, name="add")
    y = b.softmax(add, -1, name="y")
    b.output(y, "y")


# ---------------------------------------------------------------------------
# C1 / C2: ResNet-50 v1.5 (stride 2 on the 3x3 of each down-sampling bottleneck),
# BatchNorm folded into the convolutions (gamma 1, beta 0, mean 0, var 1).
# ---------------------------------------------------------------------------
RESNET50_STAGES = [(64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)]
BN_EPS = 1e-5


def resnet50_conv_specs(stages=RESNET50_STAGES, stem=64):
    """[(name, cout, cin, k, stride, pad)] in execution order."""
    specs = [("stem", stem, 3, 7, 2, 3)]
    cin = stem
    for si, (mid, blocks, stride) in enumerate(stages):
        cout = mid * 4
        for bi in range(blocks):
            s = stride if bi == 0 else 1
            p = "l%db%d" % (si + 1, bi)
            if bi == 0:
                specs.append((p + "ds", cout, cin, 1, s, 0))
            specs.append((p + "c1", mid, cin, 1, 1, 0))
            specs.append((p + "c2", mid, mid, 3, s, 1))
            specs.append((p + "c3", cout, mid, 1, 1, 0))
            cin = cout
    return specs


def resnet50_weights(seed=42, num_classes=1000, stages=RESNET50_STAGES, stem=64):
    """He-normal conv weights with the identity BatchNorm folded in."""
    rng = np.random.default_rng(seed)
    w = {}
    fold = np.float32(1.0 / np.sqrt(np.float32(1.0) + np.float32(BN_EPS)))
    for name, cout, cin, k, _, _ in resnet50_conv_specs(stages, stem):
        std = np.sqrt(2.0 / (cin * k * k))
        w[name + ".w"] = (rng.standard_normal((cout, cin, k, k)).astype(np.float32) * np.float32(std) * fold)
        w[name + ".b"] = np.zeros(cout, np.float32)
    feat = stages[-1][0] * 4
    w["fc.w"] = (rng.standard_normal((feat, num_classes)) * np.sqrt(1.0 / feat)).astype(np.float32)
    w["fc.b"] = np.zeros(num_classes, np.float32)
    return w


def resnet50_input(batch, hw=224, seed=1234):
    rng = np.random.default_rng(seed)
    return {"input": rng.standard_normal((batch, 3, hw, hw), dtype=np.float32)}


def build_resnet50(b, w, batch, hw=224, stages=RESNET50_STAGES, stem=64, num_classes=1000,
                   with_softmax=True, taps=None):
    """`taps`: optional list that receives (name, value) of every named
    activation in execution order (used for calibration / per-layer parity)."""
    def tap(name, v):
        if taps is not None:
            taps.append((name, v))
        return v

    def conv(x, name, k, stride, pad, relu):
        y = b.conv(x, b.const(name + ".w", w[name + ".w"]), b.const(name + ".b", w[name + ".b"]),
                   (stride, stride), (pad, pad, pad, pad), name=name)
        tap(name, y)
        if relu:
            y = tap(name + ".relu", b.relu(y, name=name + ".relu"))
        return y

    x = tap("input", b.arg("input", (batch, 3, hw, hw)))
    x = conv(x, "stem", 7, 2, 3, True)
    x = tap("pool1", b.maxpool(x, (3, 3), (2, 2), (1, 1, 1, 1), name="pool1"))
    for si, (mid, blocks, stride) in enumerate(stages):
        for bi in range(blocks):
            s = stride if bi == 0 else 1
            p = "l%db%d" % (si + 1, bi)
            identity = conv(x, p + "ds", 1, s, 0, False) if bi == 0 else x
            y = conv(x, p + "c1", 1, 1, 0, True)
            y = conv(y, p + "c2", 3, s, 1, True)
            y = conv(y, p + "c3", 1, 1, 0, False)
            y = tap(p + "add", b.add(y, identity, name=p + "add"))
            x = tap(p + "out", b.relu(y, name=p + "out"))
    x = tap("gap", b.reduce_mean(x, (2, 3), True, name="gap"))
    feat = stages[-1][0] * 4
    x = b.reshape(x, (batch, feat), name="flat")
    logits = tap("logits", b.gemm(x, b.const("fc.w", w["fc.w"]), b.const("fc.b", w["fc.b"]), False, False, 1.0, 1.0,
                                  name="logits"))
    b.output(logits, "logits")
    if with_softmax:
        b.output(b.softmax(logits, -1, name="prob"), "prob")


RESNET50_GFLOP_PER_IMAGE = 2 * (4087136256 + 2048000) / 1e9   # conv + FC multiply-adds, x2


def resnet50_conv_elements(batch, hw=224, stages=RESNET50_STAGES, stem=64, cin_stored=8):
    """Algorithmic element traffic of the convolution launches of one step:
    {name: (flops, activation elements read + written, weight elements, input elements)}.
    Each launch reads its input once, its residual once (c3 launches: the
    block's shortcut is fused into them) and writes its output once; the stem
    reads the library's channels-last copy of the image, which stores
    `cin_stored` channels per source pixel.  (The input elements alone are what a
    launch saves when the layer before it computes it from its own tiles.)"""
    out = {}
    h = (hw + 2 * 3 - 7) // 2 + 1
    out["stem"] = (2.0 * batch * h * h * stem * 3 * 49, batch * (hw * hw * cin_stored + h * h * stem), stem * 3 * 49,
                   batch * hw * hw * cin_stored)
    h = (h + 2 - 3) // 2 + 1
    cin = stem
    for si, (mid, blocks, stride) in enumerate(stages):
        cout = mid * 4
        for bi in range(blocks):
            s = stride if bi == 0 else 1
            p = "l%db%d" % (si + 1, bi)
            ho = (h - 1) // s + 1
            if bi == 0:
                out[p + "ds"] = (2.0 * batch * ho * ho * cout * cin, batch * (h * h * cin + ho * ho * cout), cout * cin,
                                 batch * h * h * cin)
            out[p + "c1"] = (2.0 * batch * h * h * mid * cin, batch * (h * h * cin + h * h * mid), mid * cin, batch * h * h * cin)
            out[p + "c2"] = (2.0 * batch * ho * ho * mid * mid * 9, batch * (h * h * mid + ho * ho * mid), mid * mid * 9,
                             batch * h * h * mid)
            out[p + "c3"] = (2.0 * batch * ho * ho * cout * mid, batch * (ho * ho * mid + 2 * ho * ho * cout), cout * mid,
                             batch * ho * ho * mid)
            cin, h = cout, ho
    return out


# ---------------------------------------------------------------------------
# C2: post-training quantisation of the same network.
#
# The graph stays FLOAT32-typed; an odla_value_quant_info table keyed by value
# id carries the ranges (this is the channel the reference defines for it:
# ODLA_QUANT_TABLE / ODLA_QUANT_TABLE_SIZE / ODLA_USE_DATA_TYPE, written by
# utils/halo_pgq.py:283-332 of the reference tree).
#   activations  asymmetric u8 per tensor: scale = (max-min)/255,
#                zp = clip(rne(-min/scale), 0, 255), range widened to contain 0
#   weights      symmetric s8 per output channel: scale = max|w_c| / 127,
#                expressed through the per-channel min/max records
# Values without a table entry stay floating point, which is how the fp32
# classifier head is expressed.
# ---------------------------------------------------------------------------
def act_qparams(mn, mx):
    mn = np.float32(min(float(mn), 0.0))
    mx = np.float32(max(float(mx), 0.0))
    scale = np.float32((mx - mn) / np.float32(255.0))
    if not scale > 0:
        scale = np.float32(1.0)
    zp = int(np.clip(np.rint(np.float32(-mn) / scale), 0, 255))
    return scale, zp


def resnet50_quantized_values(stages=RESNET50_STAGES):
    """Names of the activations that live as 8-bit levels in the int8 plan."""
    names = ["input", "stem.relu"]
    for si, (mid, blocks, stride) in enumerate(stages):
        for bi in range(blocks):
            p = "l%db%d" % (si + 1, bi)
            if bi == 0:
                names.append(p + "ds")
            names += [p + "c1.relu", p + "c2.relu", p + "c3", p + "out"]
    return names


def resnet50_quant_entries(w, ranges, stages=RESNET50_STAGES, stem=64):
    """ranges: name -> (min, max) of the calibrated activations.  Returns the
    entry list `odla.quant_table` turns into odla_value_quant_info records."""
    entries = []
    for name in resnet50_quantized_values(stages):
        mn, mx = ranges[name]
        scale, zp = act_qparams(mn, mx)
        entries.append((name, scale, zp, mn, mx, None))
    for name, cout, cin, k, _, _ in resnet50_conv_specs(stages, stem):
        wt = w[name + ".w"].reshape(cout, -1)
        ch = list(zip(wt.min(axis=1).tolist(), wt.max(axis=1).tolist()))
        entries.append((name + ".w", 1.0, 0, float(wt.min()), float(wt.max()), ch))
    return entries


def calibrate_ranges(run_taps, batches):
    """run_taps(feeds) -> {name: array}; min/max over all calibration batches."""
    ranges = {}
    for feeds in batches:
        for name, v in run_taps(feeds).items():
            mn, mx = float(np.min(v)), float(np.max(v))
            if name in ranges:
                ranges[name] = (min(ranges[name][0], mn), max(ranges[name][1], mx))
            else:
                ranges[name] = (mn, mx)
    return ranges
