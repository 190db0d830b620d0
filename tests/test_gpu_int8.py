"""int8 plan: bit-exact parity with the CPU oracle.

The graph handed to the library is FLOAT32-typed; a quant table
(ODLA_QUANT_TABLE / ODLA_QUANT_TABLE_SIZE / ODLA_USE_DATA_TYPE) selects the
int8 kernels.  Checked here:
  * raw int32 accumulators (+ int32 bias) of single convolutions,
  * requantised 8-bit outputs of Conv(+ReLU), of the fused Conv+Add+ReLU and of
    the unfused quantised Add,
  * every quantised activation and the fp32 logits of a small ResNet.
All integer comparisons are exact (np.array_equal).
"""
import os
import sys

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, run_hip

pytestmark = pytest.mark.gpu

sys.path.insert(0, os.path.join(entry.ROOT, "oracle"))


def rng(seed):
    return np.random.default_rng(seed)


def table_for(odla, acts, weights):
    """acts: name -> (min, max); weights: name -> array [O, ...]."""
    models = entry.load().models
    entries = []
    for name, (mn, mx) in acts.items():
        s, z = models.act_qparams(mn, mx)
        entries.append((name, s, z, mn, mx, None))
    for name, w in weights.items():
        wt = w.reshape(w.shape[0], -1)
        entries.append((name, 1.0, 0, float(wt.min()), float(wt.max()),
                        list(zip(wt.min(axis=1).tolist(), wt.max(axis=1).tolist()))))
    return odla.quant_table(entries)


Q8_CONV_CASES = [
    # N, C, H, W, O, k, stride, pad
    (2, 16, 10, 10, 32, 3, 1, 1),
    (2, 32, 9, 11, 48, 3, 2, 1),
    (3, 64, 7, 7, 64, 1, 1, 0),
    (2, 3, 20, 20, 16, 7, 2, 3),
    (1, 48, 6, 6, 200, 1, 2, 0),
    (1, 512, 7, 7, 64, 3, 1, 1),
    # weights-in-registers kernel (more than 64 output channels, input channels a
    # multiple of the 128-byte K stage): ragged tiles, stride, several K stages
    (2, 128, 9, 9, 160, 3, 1, 1),
    (1, 256, 7, 7, 128, 3, 2, 1),
    (3, 128, 6, 6, 200, 1, 1, 0),
    (1, 384, 5, 5, 72, 1, 1, 0),
    # few-channel stride-2 stems (space-to-depth lowering), odd sizes
    (2, 3, 15, 17, 8, 3, 2, 1),
    (1, 2, 11, 9, 6, 5, 2, 2),
]


@pytest.mark.parametrize("case", Q8_CONV_CASES)
def test_q8_conv_accumulators_and_requant(case, odla, ref):
    N, C, H, W, O, k, s, p = case
    announce("q8 conv %s" % (case,))
    r = rng(100 + O)
    x = (r.standard_normal((N, C, H, W)) * 1.5 + 0.3).astype(np.float32)
    w = (r.standard_normal((O, C, k, k)) * np.sqrt(2.0 / (C * k * k))).astype(np.float32)
    bias = (r.standard_normal(O) * 0.2).astype(np.float32)
    x_rng = (float(x.min()), float(x.max()))
    x_qp = ref.act_qparams(*x_rng)
    y_rng = (-2.5, 4.0)
    y_qp = ref.act_qparams(*y_rng)

    def build_acc(b):
        v = b.arg("x", x.shape)
        b.output(b.conv(v, b.const("w", w), b.const("b", bias), (s, s), (p, p, p, p), name="y"), "y")

    def build_q(b):
        v = b.arg("x", x.shape)
        y = b.conv(v, b.const("w", w), b.const("b", bias), (s, s), (p, p, p, p), name="y")
        b.output(b.relu(y, name="yr"), "yr")

    # oracle
    xq = ref.quantize_act(x, *x_qp)
    q_want, acc_want = ref.qconv(xq, x_qp, w, bias, y_qp, (s, s), (p, p, p, p), relu=True)

    # 1. raw accumulators: the result value has no table entry
    t = table_for(odla, {"x": x_rng}, {"w": w})
    got = run_hip(build_acc, {"x": x}, quant_table=t, raw_acc=True)["y"]
    acc_got = got.view(np.int32)
    assert acc_got.shape == acc_want.shape
    assert np.array_equal(acc_got, acc_want)

    # 2. requantised output (ReLU fused as a clamp at the zero point), read back dequantised
    t = table_for(odla, {"x": x_rng, "yr": y_rng}, {"w": w})
    got = run_hip(build_q, {"x": x}, quant_table=t)["yr"]
    want = ref.dequantize_act(q_want, *y_qp)
    assert np.array_equal(got, want)
    q_got = np.rint(got / y_qp[0]).astype(np.int64) + y_qp[1]
    assert np.array_equal(q_got, q_want.astype(np.int64))


@pytest.mark.parametrize("case", [c for c in Q8_CONV_CASES if c[4] > 64 and c[1] % 128 == 0])
def test_q8_conv_two_channel_slices_per_wavefront(case, odla, ref, monkeypatch):
    """Weights-in-registers kernel with two 32-channel slices per wavefront, 8-bit operands."""
    monkeypatch.setenv("ODLA_HIP_WREG_SLICES", "2")
    test_q8_conv_accumulators_and_requant(case, odla, ref)


@pytest.mark.parametrize("dims", [(2, 32, 8, 8, 64), (4, 64, 21, 19, 256), (2, 128, 30, 30, 512)])
def test_q8_two_half_batches_side_by_side(dims, odla, ref, monkeypatch):
    """The 8-bit residual block executed as two half-batch copies on two streams: bit-equal to
    the oracle like the whole batch (every image's arithmetic is its own)."""
    monkeypatch.setenv("ODLA_HIP_BATCH_SPLIT", "2")
    test_q8_residual_fused_equals_unfused_equals_oracle(dims, 0, odla, ref, monkeypatch)


@pytest.mark.parametrize("case", [c for c in Q8_CONV_CASES if c[1] % 128 == 0])
def test_q8_conv_two_k_groups_per_workgroup(case, odla, ref, monkeypatch):
    """Weights-in-registers kernel with two K groups per workgroup, 8-bit operands: the int32
    partial sums of the second group join the first's (which carry the bias) through LDS."""
    monkeypatch.setenv("ODLA_HIP_WREG_KSPLIT", "2")
    test_q8_conv_accumulators_and_requant(case, odla, ref)


@pytest.mark.parametrize("tiles_per_wg", [0, 3, -1])
@pytest.mark.parametrize("dims", [(2, 32, 8, 8, 64), (3, 128, 7, 7, 200), (4, 64, 21, 19, 256), (2, 128, 30, 30, 512),
                                  (3, 256, 9, 9, 136), (2, 64, 17, 9, 128), (1, 128, 40, 40, 384)])
def test_q8_residual_fused_equals_unfused_equals_oracle(dims, tiles_per_wg, odla, ref, monkeypatch):
    """Conv -> Add(residual) -> ReLU: fused into the conv epilogue, and as separate
    quantised kernels (the conv result is also a graph output, which blocks fusion).
    64 / 128 input channels take the streaming 1x1 kernel (whole groups of 128 output
    channels in its row-epilogue form, otherwise - and with tiles_per_wg = -1 - in its
    lane-exchange form), 256 the weights-in-registers kernel."""
    announce("q8 residual %s tiles/wg %d" % (dims, tiles_per_wg))
    if tiles_per_wg > 0:
        monkeypatch.setenv("ODLA_HIP_LEAN_TILES", str(tiles_per_wg))
    if tiles_per_wg < 0:   # the streaming kernel's lane-exchange epilogue instead of its row epilogue
        monkeypatch.setenv("ODLA_HIP_STREAM_ROWS", "0")
    r = rng(7)
    N, C, H, W, O = dims
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    res = (r.standard_normal((N, O, H, W)) * 2).astype(np.float32)
    w = (r.standard_normal((O, C, 1, 1)) * 0.3).astype(np.float32)
    bias = r.standard_normal(O).astype(np.float32)
    ranges = {"x": (float(x.min()), float(x.max())), "res": (float(res.min()), float(res.max())),
              "c": (-6.0, 6.0), "out": (0.0, 9.0)}
    qp = {k: ref.act_qparams(*v) for k, v in ranges.items()}

    def build(b, tap_conv):
        v = b.arg("x", x.shape)
        rr = b.arg("res", res.shape)
        c = b.conv(v, b.const("w", w), b.const("b", bias), name="c")
        if tap_conv:
            b.output(c, "c")
        b.output(b.relu(b.add(c, rr, name="add"), name="out"), "out")

    t = table_for(odla, ranges, {"w": w})
    fused = run_hip(lambda b: build(b, False), {"x": x, "res": res}, quant_table=t)
    t = table_for(odla, ranges, {"w": w})
    unfused = run_hip(lambda b: build(b, True), {"x": x, "res": res}, quant_table=t)

    xq = ref.quantize_act(x, *qp["x"])
    rq = ref.quantize_act(res, *qp["res"])
    # separate kernels: the convolution is requantised to its own entry, then dequantise / add / requantise
    cq, _ = ref.qconv(xq, qp["x"], w, bias, qp["c"], (1, 1), (0, 0, 0, 0), relu=False)
    oq = ref.qadd(cq, qp["c"], rq, qp["res"], qp["out"], relu=True)
    assert np.array_equal(unfused["c"], ref.dequantize_act(cq, *qp["c"]))
    assert np.array_equal(unfused["out"], ref.dequantize_act(oq, *qp["out"]))
    # fused: ONE requantisation behind convolution + residual + ReLU
    fq, _ = ref.qconv(xq, qp["x"], w, bias, qp["out"], (1, 1), (0, 0, 0, 0), relu=True, residual=(rq, qp["res"]))
    assert np.array_equal(fused["out"], ref.dequantize_act(fq, *qp["out"]))
    # where the intermediate tensor does not saturate, the two differ by its rounding only: half
    # a level of 'c' (12 / 255 wide) on either side, seen in levels of 'out' (9 / 255 wide)
    inside = (cq > 0) & (cq < 255)
    assert np.max(np.abs(fq.astype(np.int32) - oq.astype(np.int32))[inside]) <= 2


@pytest.mark.parametrize("dims", [(2, 9, 9, 64), (3, 21, 19, 64), (1, 40, 40, 128), (5, 7, 7, 128), (2, 16, 16, 96),
                                  (2, 9, 9, 128, 128, 512), (3, 21, 19, 128, 128, 512), (1, 28, 28, 128, 128, 512)])
@pytest.mark.parametrize("relu2", [True, False])
def test_q8_expanding_layer_carries_the_next_reducing_layer(dims, relu2, odla, ref, monkeypatch):
    """64 -> 256 (+ residual + ReLU) followed by a plain 1x1 layer 256 -> 64 / 128 over its result:
    the first launch computes both (the second layer from the first's tiles in LDS).  Both results
    are bit-equal to the oracle, and to the two layers launched one after the other
    (ODLA_HIP_STREAM_FUSE=0); 96 output channels, and the pair 128 -> 512 -> 128, are not carried and
    take the ordinary road.
    Pixel counts that end inside a wavefront's 32-pixel tile and inside a workgroup's group."""
    announce("q8 carried layer %s relu2=%s" % (dims, relu2))
    monkeypatch.delenv("ODLA_HIP_STREAM_FUSE", raising=False)
    N, H, W, O2 = dims[:4]
    C1, O1 = dims[4:] if len(dims) > 4 else (64, 256)
    r = rng(31)
    x = r.standard_normal((N, C1, H, W)).astype(np.float32)
    res = (r.standard_normal((N, O1, H, W)) * 2).astype(np.float32)
    w1 = (r.standard_normal((O1, C1, 1, 1)) * 0.3).astype(np.float32)
    b1 = r.standard_normal(O1).astype(np.float32)
    w2 = (r.standard_normal((O2, O1, 1, 1)) * 0.1).astype(np.float32)
    b2 = r.standard_normal(O2).astype(np.float32)
    ranges = {"x": (float(x.min()), float(x.max())), "res": (float(res.min()), float(res.max())),
              "c": (-6.0, 6.0), "out": (0.0, 9.0), "y2": ((0.0, 7.0) if relu2 else (-7.0, 7.0))}
    # ('c' needs its entry for the residual Add to be fused behind the convolution; the fused
    #  chain then requantises once, to the entry of 'out')
    qp = {k: ref.act_qparams(*v) for k, v in ranges.items()}

    def build(b):
        v = b.arg("x", x.shape)
        rr = b.arg("res", res.shape)
        c = b.conv(v, b.const("w1", w1), b.const("b1", b1), name="c")
        out = b.relu(b.add(c, rr, name="add"), name="out")
        b.output(out, "out")
        y2 = b.conv(out, b.const("w2", w2), b.const("b2", b2), name="y2pre" if relu2 else "y2")
        if relu2:
            y2 = b.relu(y2, name="y2")
        b.output(y2, "y2")

    def run():
        return run_hip(build, {"x": x, "res": res}, quant_table=table_for(odla, ranges, {"w1": w1, "w2": w2}))

    carried = run()
    monkeypatch.setenv("ODLA_HIP_STREAM_FUSE", "0")
    apart = run()

    xq = ref.quantize_act(x, *qp["x"])
    rq = ref.quantize_act(res, *qp["res"])
    oq, _ = ref.qconv(xq, qp["x"], w1, b1, qp["out"], (1, 1), (0, 0, 0, 0), relu=True, residual=(rq, qp["res"]))
    yq, _ = ref.qconv(oq, qp["out"], w2, b2, qp["y2"], (1, 1), (0, 0, 0, 0), relu=relu2)
    for got in (carried, apart):
        assert np.array_equal(got["out"], ref.dequantize_act(oq, *qp["out"]))
        assert np.array_equal(got["y2"], ref.dequantize_act(yq, *qp["y2"]))


def test_q8_carried_layer_in_two_half_batches(odla, ref, monkeypatch):
    """The pair above executed as two half-batch copies of the plan on two streams (each copy's
    first launch carries the second layer): both results bit-equal to the oracle."""
    monkeypatch.setenv("ODLA_HIP_BATCH_SPLIT", "2")
    test_q8_expanding_layer_carries_the_next_reducing_layer((4, 21, 19, 64), True, odla, ref, monkeypatch)
    test_q8_expanding_layer_carries_the_next_reducing_layer((6, 9, 9, 128), False, odla, ref, monkeypatch)


SMALL_STAGES = [(16, 2, 1), (32, 2, 2)]


def test_small_resnet_int8_bit_exact(odla, models, ref):
    """Whole int8 network: every 8-bit activation that ends a fused chain and the fp32 head."""
    announce("small resnet int8")
    import resnet_q8_ref
    batch, hw, stem, classes = 4, 64, 16, 50
    w = models.resnet50_weights(seed=11, num_classes=classes, stages=SMALL_STAGES, stem=stem)
    for k in w:  # non-zero biases exercise the int32 bias path
        if k.endswith(".b") and k != "fc.b":
            w[k] = (rng(len(k)).standard_normal(w[k].shape) * 0.1).astype(np.float32)

    # calibration: min/max of the fp32 oracle over 4 seeded batches
    def taps_of(feeds):
        rb = ref.RefBuilder(feeds)
        taps = []
        models.build_resnet50(rb, w, batch, hw, SMALL_STAGES, stem, classes, taps=taps)
        return dict(taps)

    ranges = models.calibrate_ranges(taps_of, [models.resnet50_input(batch, hw, seed=1000 + i) for i in range(4)])
    entries = models.resnet50_quant_entries(w, ranges, SMALL_STAGES, stem)
    qp = {e[0]: (e[1], e[2]) for e in entries if e[5] is None}
    feeds = models.resnet50_input(batch, hw, seed=1234)

    record = {}
    want = resnet_q8_ref.run(w, feeds, qp, SMALL_STAGES, stem, batch, hw, record)

    # chain-end activations can be tapped without changing the plan
    tap_names = [n for n in models.resnet50_quantized_values(SMALL_STAGES) if not n.endswith("c3") and n != "input"]

    def build(b):
        taps = []
        models.build_resnet50(b, w, batch, hw, SMALL_STAGES, stem, classes, taps=taps)
        d = dict(taps)
        for n in tap_names:
            b.output(d[n], n)

    got = run_hip(build, feeds, quant_table=odla.quant_table(entries))
    for n in tap_names:
        assert np.array_equal(got[n], ref.dequantize_act(record[n], *qp[n])), n
    # fp32 head behind the 8-bit trunk: same integer input, fp32 Gemm
    assert np.max(np.abs(got["logits"] - want["logits"])) <= 1e-4 * max(1.0, float(np.max(np.abs(want["logits"]))))
    assert np.array_equal(np.argmax(got["logits"], 1), np.argmax(want["logits"], 1))
