"""Per-operator parity: libodla_hip.so (through the ODLA C ABI) against the CPU
oracle on identical seeded inputs, plus the reference-held known-answer
vectors replayed through the ABI exactly as the reference's doctest suite
calls it (ODLA/platforms/odla_popart/test/*.cc of the reference tree).

Tolerances: fp32 graphs 1e-4 of the largest expected magnitude; fp16 / bf16
storage 2e-2 absolute on O(1) data; integer results bit-exact.
"""
import numpy as np
import pytest

from util import announce, max_rel_err, run_both, run_hip

pytestmark = pytest.mark.gpu

F32_TOL = 1e-4


def rng(seed):
    return np.random.default_rng(seed)


# --------------------------------------------------------------------------
# Known-answer vectors held by the reference's own tests
# --------------------------------------------------------------------------
def test_kat_conv_runtime_kernel():
    """odla_ops_nn_test.cc:147-200: 5x5 ramp * ones 3x3, pad 1; the kernel is an argument."""
    announce("kat conv")

    def build(b):
        x = b.arg("input", (1, 1, 5, 5))
        k = b.arg("kernel", (1, 1, 3, 3))
        b.output(b.conv(x, k, None, (1, 1), (1, 1, 1, 1), name="Conv"), "Conv")

    feeds = {"input": np.arange(25, dtype=np.float32).reshape(1, 1, 5, 5),
             "kernel": np.ones((1, 1, 3, 3), np.float32)}
    got = run_hip(build, feeds)["Conv"].reshape(-1)
    expected = [12, 21, 27, 33, 24, 33, 54, 63, 72, 51, 63, 99, 108, 117, 81, 93, 144, 153, 162, 111, 72, 111,
                117, 123, 84]
    assert got.tolist() == [float(v) for v in expected]


def test_kat_pools():
    """odla_ops_nn_test.cc:38-78 (avg -> 6,7,10,11) and :523-560 (max -> 11,12,15,16)."""
    announce("kat pools")
    x = np.arange(1, 17, dtype=np.float32).reshape(1, 1, 4, 4)

    def build(b):
        v = b.arg("input", (1, 1, 4, 4))
        b.output(b.avgpool(v, (3, 3), (1, 1), (0, 0, 0, 0), name="avg"), "avg")
        b.output(b.maxpool(v, (3, 3), (1, 1), (0, 0, 0, 0), name="max"), "max")

    got = run_hip(build, {"input": x})
    assert np.allclose(got["avg"].reshape(-1), [6, 7, 10, 11], atol=1e-5)
    assert got["max"].reshape(-1).tolist() == [11, 12, 15, 16]


def test_kat_batchnorm_runtime_params():
    """odla_ops_nn_test.cc:80-145: statistics passed as arguments."""
    announce("kat batchnorm")

    def build(b):
        x = b.arg("input", (1, 2, 1, 3))
        sc = b.arg("scale", (2,))
        of = b.arg("offset", (2,))
        mean = b.arg("mean", (2,))
        var = b.arg("var", (2,))
        b.output(b.batchnorm(x, mean, var, 1e-5, sc, of, 1.0, 1.0, name="bn"), "bn")

    feeds = {"input": np.array([-1, 0, 1, 2, 3, 4], np.float32).reshape(1, 2, 1, 3),
             "scale": np.array([1.0, 1.5], np.float32), "offset": np.array([0, 1], np.float32),
             "mean": np.array([0, 3], np.float32), "var": np.array([1, 1.5], np.float32)}
    got = run_hip(build, feeds)["bn"].reshape(-1)
    expected = np.array([-0.999995, 0, 0.999995, -0.224741, 1, 2.22474])
    assert np.max(np.abs(got - expected)) < 1e-5


def test_kat_leakyrelu_relu_gemm():
    """odla_ops_nn_test.cc:393-422, odla_ops_test.cc:240-267 and :39-79."""
    announce("kat leakyrelu/relu/gemm")

    def build(b):
        x = b.arg("x", (1, 3))
        b.output(b.leaky_relu(x, 0.1, name="lr"), "lr")
        b.output(b.relu(x, name="r"), "r")
        a = b.arg("a", (4, 16))
        w = b.arg("w", (16, 8))
        b.output(b.gemm(a, w, None, False, False, 1.0, 0.0, name="g"), "g")

    feeds = {"x": np.array([[-1, 0, 1]], np.float32), "a": np.ones((4, 16), np.float32),
             "w": np.ones((16, 8), np.float32)}
    got = run_hip(build, feeds)
    assert np.allclose(got["lr"].reshape(-1), [-0.1, 0, 1], atol=1e-7)
    assert got["r"].reshape(-1).tolist() == [0, 0, 1]
    assert np.all(got["g"] == 16.0)


def test_kat_executor_scaffold():
    """tests/compile/test_cxx_gen.cc:46-48 of the reference: (input + w0) * w1 -> 6, 9, 12."""
    announce("kat executor scaffold")

    def build(b):
        x = b.arg("input", (3,))
        w0 = b.const("w0", np.array([1, 1, 1], np.float32))
        w1 = b.const("w1", np.array([3, 3, 3], np.float32))
        b.output(b.mul(b.add(x, w0, name="add"), w1, name="mul"), "mul")

    got = run_hip(build, {"input": np.array([1, 2, 3], np.float32)})["mul"]
    assert got.tolist() == [6, 9, 12]


# --------------------------------------------------------------------------
# Convolution
# --------------------------------------------------------------------------
CONV_CASES = [
    # N, C, H, W, O, k, stride, pad, group, dilation
    (2, 16, 14, 14, 32, 3, 1, 1, 1, 1),
    (2, 16, 15, 13, 24, 3, 2, 1, 1, 1),
    (3, 64, 9, 9, 64, 1, 1, 0, 1, 1),
    (2, 3, 32, 32, 16, 7, 2, 3, 1, 1),
    (1, 32, 12, 12, 130, 1, 2, 0, 1, 1),
    (2, 8, 10, 10, 8, 3, 1, 2, 1, 2),
    (2, 32, 8, 8, 64, 3, 1, 1, 2, 1),
    (1, 20, 7, 7, 255, 1, 1, 0, 1, 1),
    (1, 4, 5, 5, 4, 5, 1, 0, 1, 1),
    # shapes that take the weights-in-registers kernel (more than 64 output
    # channels, input channels a multiple of the K stage, at most 32 taps):
    # ragged pixel and channel tiles, stride, dilation, 1 and many K stages
    (2, 64, 14, 14, 160, 3, 1, 1, 1, 1),
    (1, 128, 9, 9, 128, 3, 2, 1, 1, 1),
    (2, 64, 10, 10, 96, 3, 1, 2, 1, 2),
    (3, 192, 7, 7, 256, 1, 1, 0, 1, 1),
    (1, 64, 6, 6, 72, 5, 1, 2, 1, 1),
    (1, 64, 8, 8, 80, 1, 1, 0, 1, 1),
    (1, 64, 9, 9, 96, 7, 1, 3, 1, 1),   # 49 taps: stays on the two-operand kernel
    (5, 64, 12, 12, 300, 1, 1, 0, 1, 1),
    # few input channels, stride 2: lowered through the space-to-depth form of
    # the input (odd image sizes, even and odd paddings, 1..4 channels)
    (2, 3, 15, 17, 8, 3, 2, 1, 1, 1),
    (1, 1, 9, 9, 4, 5, 2, 2, 1, 1),
    (2, 4, 12, 12, 16, 7, 2, 3, 1, 1),
    (1, 2, 11, 8, 6, 4, 2, 0, 1, 1),
    (1, 3, 10, 10, 8, 3, 2, 2, 1, 1),
]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("mode", ["fp32", "fp16", "bf16"])
def test_conv_parity(case, mode):
    N, C, H, W, O, k, s, p, g, d = case
    announce("conv %s %s" % (mode, case))
    r = rng(hash(case) % 1000)
    w = (r.standard_normal((O, C // g, k, k)) * np.sqrt(2.0 / (C // g * k * k))).astype(np.float32)
    bias = r.standard_normal(O).astype(np.float32)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)

    def build(b):
        v = b.arg("x", (N, C, H, W))
        y = b.conv(v, b.const("w", w), b.const("b", bias), (s, s), (p, p, p, p), (d, d), g, name="y")
        b.output(y, "y")

    kw = {"fp16": mode == "fp16", "bf16": mode == "bf16"}
    got, want = run_both(build, {"x": x}, **kw)
    assert got["y"].shape == want["y"].shape
    if mode == "fp32":
        assert max_rel_err(got["y"], want["y"]) <= F32_TOL
    else:
        tol = 2e-2 if mode == "fp16" else 6e-2
        assert np.max(np.abs(got["y"] - want["y"])) <= tol * max(1.0, float(np.max(np.abs(want["y"]))))


@pytest.mark.parametrize("case", [c for c in CONV_CASES if c[4] > 64 and c[1] % 64 == 0 and c[8] == 1])
@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_conv_two_channel_slices_per_wavefront(case, mode, monkeypatch):
    """The weights-in-registers kernel with two 32-channel slices per wavefront (256-channel
    tiles), which the library picks by itself only for long K loops on large grids."""
    monkeypatch.setenv("ODLA_HIP_WREG_SLICES", "2")
    test_conv_parity(case, mode)


K_GROUP_CASES = [
    # N, C, H, W, O, k, stride, pad, group, dilation: an even number of 128-byte K stages in
    # every mode, ragged pixel and channel tiles, a tap boundary inside the second group's half
    (2, 128, 13, 13, 256, 3, 1, 1, 1, 1),
    (1, 256, 13, 13, 200, 1, 1, 0, 1, 1),
    (2, 128, 9, 9, 160, 3, 2, 1, 1, 1),
    (1, 128, 7, 7, 130, 3, 1, 2, 1, 2),
    (3, 64, 6, 6, 136, 2, 1, 0, 1, 1),
]


@pytest.mark.parametrize("case", K_GROUP_CASES + [c for c in CONV_CASES if c[1] % 64 == 0 and c[8] == 1 and c[4] > 64])
@pytest.mark.parametrize("mode", ["fp32", "fp16", "bf16"])
def test_conv_two_k_groups_per_workgroup(case, mode, monkeypatch):
    """The weights-in-registers kernel with eight wavefronts in two K groups (each half of the
    K stages, summed through LDS), which the library picks by itself for launches with fewer
    workgroups than compute units; forced here wherever the stage count is even."""
    monkeypatch.setenv("ODLA_HIP_WREG_KSPLIT", "2")
    test_conv_parity(case, mode)


def test_small_launch_takes_two_k_groups_by_itself():
    """A 3x3 layer over a 13 x 13 map at batch 2 (6 workgroups, 36 K stages in fp16) is given
    the two-group form without being asked, with a fused residual and LeakyReLU."""
    from test_gpu_taps_kernel import run_logged
    N, C, H, W, O = 2, 256, 13, 13, 256
    r = rng(77)
    w = (r.standard_normal((O, C, 3, 3)) * np.sqrt(2.0 / (C * 9))).astype(np.float32)
    bias = r.standard_normal(O).astype(np.float32)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    res = r.standard_normal((N, O, H, W)).astype(np.float32)

    def build(b):
        v = b.arg("x", (N, C, H, W))
        sc = b.arg("res", (N, O, H, W))
        y = b.conv(v, b.const("w", w), b.const("b", bias), (1, 1), (1, 1, 1, 1), (1, 1), 1, name="y")
        y = b.leaky_relu(y, 0.1, name="act")
        b.output(b.add(y, sc, name="sum"), "sum")

    announce("conv two K groups by default")
    (got, want), seen = run_logged(lambda: run_both(build, {"x": x, "res": res}, fp16=True))
    assert any(m.endswith("kernel 128x128w2k") for m in seen), [m for m in seen if "kernel" in m]
    assert np.max(np.abs(got["sum"] - want["sum"])) <= 2e-2 * max(1.0, float(np.max(np.abs(want["sum"]))))


LEAN_CASES = [
    # 1x1 filters over 64 / 128 bytes of input channels per pixel (the streaming kernel):
    # N, C, H, W, O, stride, residual
    (3, 64, 23, 17, 256, 1, True),
    (2, 64, 20, 20, 200, 2, False),
    (4, 32, 19, 19, 130, 1, True),
    (1, 32, 40, 40, 64, 1, False),
]


@pytest.mark.parametrize("tiles_per_wg", [0, 3])
@pytest.mark.parametrize("case", LEAN_CASES)
@pytest.mark.parametrize("mode", ["fp16", "bf16"])
def test_conv_1x1_short_k(case, mode, tiles_per_wg, monkeypatch):
    N, C, H, W, O, s, with_res = case
    announce("conv 1x1 short K %s %s tiles/wg %d" % (mode, case, tiles_per_wg))
    if tiles_per_wg:
        monkeypatch.setenv("ODLA_HIP_LEAN_TILES", str(tiles_per_wg))
    r = rng(7 * O + C)
    w = (r.standard_normal((O, C, 1, 1)) * np.sqrt(2.0 / C)).astype(np.float32)
    bias = r.standard_normal(O).astype(np.float32)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    Ho, Wo = (H - 1) // s + 1, (W - 1) // s + 1
    res = r.standard_normal((N, O, Ho, Wo)).astype(np.float32)

    def build(b):
        v = b.relu(b.arg("x", (N, C, H, W)), name="xr")
        y = b.conv(v, b.const("w", w), b.const("b", bias), (s, s), (0, 0, 0, 0), name="y")
        if with_res:
            y = b.add(y, b.relu(b.arg("res", res.shape), name="rr"), name="sum")
        b.output(b.relu(y, name="out"), "out")

    feeds = {"x": x, "res": res} if with_res else {"x": x}
    got, want = run_both(build, feeds, fp16=(mode == "fp16"), bf16=(mode == "bf16"))
    tol = 2e-2 if mode == "fp16" else 6e-2
    assert np.max(np.abs(got["out"] - want["out"])) <= tol * max(1.0, float(np.max(np.abs(want["out"]))))


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
@pytest.mark.parametrize("dims", [(2, 16, 13, 13, 32, 3), (1, 64, 12, 12, 128, 1), (2, 128, 9, 9, 160, 3)])
def test_conv_activation_then_shortcut(dims, mode):
    """y = LeakyReLU(conv(x)) + shortcut: the residual joins behind the activation (the
    order of Darknet's shortcut layers); one launch, equal to the unfused oracle sequence."""
    announce("conv act then shortcut %s %s" % (dims, mode))
    N, C, H, W, O, k = dims
    r = rng(31 + O)
    w = (r.standard_normal((O, C, k, k)) * np.sqrt(2.0 / (C * k * k))).astype(np.float32)
    bias = r.standard_normal(O).astype(np.float32)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    sc = r.standard_normal((N, O, H, W)).astype(np.float32)

    def build(b):
        v = b.arg("x", x.shape)
        s = b.relu(b.arg("sc", sc.shape), name="scr")
        y = b.conv(v, b.const("w", w), b.const("b", bias), (1, 1), (k // 2,) * 4, name="y")
        b.output(b.add(b.leaky_relu(y, 0.1, name="act"), s, name="out"), "out")

    got, want = run_both(build, {"x": x, "sc": sc}, fp16=(mode == "fp16"))
    if mode == "fp32":
        assert max_rel_err(got["out"], want["out"]) <= F32_TOL
    else:
        assert np.max(np.abs(got["out"] - want["out"])) <= 2e-2 * max(1.0, float(np.max(np.abs(want["out"]))))


@pytest.mark.parametrize("mode", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("act", ["gelu", "gelu_tanh", "sigmoid", "tanh"])
def test_gemm_and_conv_with_fused_transcendental_activation(act, mode):
    """Feed-forward GEMM + GELU (and the gate activations) in one launch: both the
    weights-in-registers kernel (wide N) and the two-operand kernel (narrow N), and a conv."""
    announce("fused %s %s" % (act, mode))
    r = rng(41)
    A = r.standard_normal((200, 128)).astype(np.float32)
    Bw = (r.standard_normal((128, 192)) * 0.1).astype(np.float32)
    Bn = (r.standard_normal((128, 24)) * 0.1).astype(np.float32)
    bias_w, bias_n = r.standard_normal(192).astype(np.float32), r.standard_normal(24).astype(np.float32)
    x = r.standard_normal((2, 64, 10, 10)).astype(np.float32)
    w = (r.standard_normal((96, 64, 3, 3)) * 0.05).astype(np.float32)

    def apply(b, v, name):
        if act == "gelu":
            return b.gelu(v, False, name=name)
        if act == "gelu_tanh":
            return b.gelu(v, True, name=name)
        return getattr(b, act)(v, name=name)

    def build(b):
        a = b.arg("A", A.shape)
        b.output(apply(b, b.gemm(a, b.const("Bw", Bw), b.const("bw", bias_w), name="gw"), "yw"), "yw")
        b.output(apply(b, b.gemm(a, b.const("Bn", Bn), b.const("bn", bias_n), name="gn"), "yn"), "yn")
        b.output(apply(b, b.conv(b.arg("x", x.shape), b.const("w", w), None, (1, 1), (1, 1, 1, 1), name="c"), "yc"), "yc")

    got, want = run_both(build, {"A": A, "x": x}, fp16=(mode == "fp16"), bf16=(mode == "bf16"))
    for k in want:
        if mode == "fp32":
            assert max_rel_err(got[k], want[k]) <= F32_TOL, k
        else:
            tol = 2e-2 if mode == "fp16" else 6e-2
            assert np.max(np.abs(got[k] - want[k])) <= tol * max(1.0, float(np.max(np.abs(want[k])))), k


@pytest.mark.parametrize("mode", ["fp32", "bf16"])
def test_masked_softmax_fused(mode):
    """softmax(scores + mask) with the attention mask shapes [B,1,1,S] and [1,1,S,S], a
    full-shape term, and a mask that cannot be folded (broadcast along the row)."""
    announce("masked softmax %s" % mode)
    r = rng(37)
    B, H, S = 3, 4, 64
    scores = (r.standard_normal((B, H, S, S)) * 2).astype(np.float32)
    pad = np.where(r.random((B, 1, 1, S)) < 0.25, -10000.0, 0.0).astype(np.float32)
    causal = np.triu(np.full((S, S), -10000.0, np.float32), 1).reshape(1, 1, S, S)
    full = r.standard_normal((B, H, S, S)).astype(np.float32)
    col = r.standard_normal((B, H, S, 1)).astype(np.float32)

    def build(b):
        s = b.arg("scores", scores.shape)
        b.output(b.softmax(b.add(s, b.arg("pad", pad.shape), name="a0"), -1, name="p0"), "p0")
        b.output(b.softmax(b.add(b.const("causal", causal), s, name="a1"), -1, name="p1"), "p1")
        b.output(b.softmax(b.add(s, b.arg("full", full.shape), name="a2"), -1, name="p2"), "p2")
        b.output(b.softmax(b.add(s, b.arg("col", col.shape), name="a3"), -1, name="p3"), "p3")

    got, want = run_both(build, {"scores": scores, "pad": pad, "full": full, "col": col}, bf16=(mode == "bf16"))
    for k in want:
        tol = 1e-4 if mode == "fp32" else 3e-2
        assert np.max(np.abs(got[k] - want[k])) <= tol, k
        assert np.max(np.abs(got[k].sum(-1) - 1.0)) <= (1e-4 if mode == "fp32" else 2e-2), k


def test_conv_fused_chain_fp32():
    """Conv + per-channel Add + BatchNorm + residual Add + ReLU collapses into one
    launch and must equal the unfused oracle sequence."""
    announce("conv fused chain")
    r = rng(5)
    N, C, H, W, O = 2, 16, 12, 12, 32
    w = (r.standard_normal((O, C, 3, 3)) * 0.1).astype(np.float32)
    extra = r.standard_normal((1, O, 1, 1)).astype(np.float32)
    mean, var = r.standard_normal(O).astype(np.float32), (r.random(O) + 0.5).astype(np.float32)
    gam, bet = r.standard_normal(O).astype(np.float32), r.standard_normal(O).astype(np.float32)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    res = r.standard_normal((N, O, H, W)).astype(np.float32)

    def build(b):
        v = b.arg("x", (N, C, H, W))
        rr = b.arg("res", (N, O, H, W))
        rr2 = b.relu(rr, name="res_relu")   # a computed residual
        y = b.conv(v, b.const("w", w), None, (1, 1), (1, 1, 1, 1), name="c")
        y = b.add(y, b.const("extra", extra), name="a0")
        y = b.batchnorm(y, b.const("m", mean), b.const("v", var), 1e-5, b.const("g", gam), b.const("be", bet), name="bn")
        y = b.add(y, rr2, name="a1")
        y = b.relu(y, name="out")
        b.output(y, "out")

    got, want = run_both(build, {"x": x, "res": res})
    assert max_rel_err(got["out"], want["out"]) <= F32_TOL


@pytest.mark.parametrize("mode", ["fp32", "fp16", "bf16"])
def test_conv_residual_relu_wide(mode):
    """Bottleneck tail at a width that takes the weights-in-registers kernel:
    3x3 conv + bias + ReLU, then 1x1 conv + bias + shortcut Add + ReLU, each
    fused into one launch; 2 x 13 x 13 pixels (338 rows: ragged 128-row tiles)."""
    announce("conv residual relu wide %s" % mode)
    r = rng(77)
    N, C, H, W, O = 2, 64, 13, 13, 192
    w1 = (r.standard_normal((C, C, 3, 3)) * np.sqrt(2.0 / (C * 9))).astype(np.float32)
    b1 = (r.standard_normal(C) * 0.1).astype(np.float32)
    w2 = (r.standard_normal((O, C, 1, 1)) * np.sqrt(2.0 / C)).astype(np.float32)
    b2 = (r.standard_normal(O) * 0.1).astype(np.float32)
    wd = (r.standard_normal((O, C, 1, 1)) * np.sqrt(2.0 / C)).astype(np.float32)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)

    def build(b):
        v = b.arg("x", (N, C, H, W))
        sc = b.conv(v, b.const("wd", wd), None, (1, 1), (0, 0, 0, 0), name="ds")
        y = b.relu(b.conv(v, b.const("w1", w1), b.const("b1", b1), (1, 1), (1, 1, 1, 1), name="c2"), name="c2r")
        y = b.conv(y, b.const("w2", w2), b.const("b2", b2), (1, 1), (0, 0, 0, 0), name="c3")
        y = b.relu(b.add(y, sc, name="sum"), name="out")
        b.output(y, "out")

    kw = {"fp16": mode == "fp16", "bf16": mode == "bf16"}
    got, want = run_both(build, {"x": x}, **kw)
    if mode == "fp32":
        assert max_rel_err(got["out"], want["out"]) <= F32_TOL
    else:
        tol = 2e-2 if mode == "fp16" else 6e-2
        assert np.max(np.abs(got["out"] - want["out"])) <= tol * max(1.0, float(np.max(np.abs(want["out"]))))


# --------------------------------------------------------------------------
# Gemm
# --------------------------------------------------------------------------
GEMM_CASES = [
    # M, K, N, tA, tB, alpha, beta, bias kind, const B
    (64, 784, 10, False, False, 1.0, 0.0, None, True),
    (33, 40, 17, False, True, 0.5, 2.0, "row", True),
    (16, 24, 32, True, False, 1.0, 1.0, "scalar", True),
    (20, 36, 12, False, False, 1.0, 0.0, None, False),
    (20, 36, 12, False, True, 1.0, 0.0, None, False),
    (7, 10, 5, False, False, 1.0, 1.0, "row", True),
    # constant B with more than 64 columns and K a multiple of the K stage:
    # the weights-in-registers kernel (ragged row / column tiles, both layouts of B, transposed A)
    (200, 256, 192, False, False, 1.0, 1.0, "row", True),
    (130, 128, 96, False, True, 0.5, 1.0, "row", True),
    (70, 64, 300, True, False, 1.0, 0.0, None, True),
    # few output tiles, long K: split along K into partial sums (classifier heads)
    (64, 2048, 100, False, False, 1.0, 1.0, "row", True),
    (256, 2048, 1000, False, True, 0.5, 1.0, "row", True),
    (40, 1536, 130, False, False, 1.0, 0.0, None, True),
    # at most 16 columns, a long reduction, few rows: one wavefront per output row
    (64, 784, 10, False, False, 1.0, 1.0, "row", True),
    (1, 2048, 16, False, True, 1.0, 0.0, None, True),
    (37, 260, 3, False, False, 0.5, 1.0, "row", True),
    (1000, 256, 1, False, True, 1.0, 1.0, "scalar", True),
    (5, 1028, 7, False, False, 1.0, 1.0, "row", False),
]


@pytest.mark.parametrize("case", GEMM_CASES)
def test_gemm_parity(case):
    M, K, N, tA, tB, alpha, beta, bias, const_b = case
    announce("gemm %s" % (case,))
    r = rng(11)
    A = r.standard_normal((K, M) if tA else (M, K)).astype(np.float32)
    B = r.standard_normal((N, K) if tB else (K, N)).astype(np.float32)
    Cb = None
    if bias == "row":
        Cb = r.standard_normal((N,)).astype(np.float32)
    elif bias == "scalar":
        Cb = r.standard_normal((1,)).astype(np.float32)

    def build(b):
        a = b.arg("A", A.shape)
        bb = b.const("B", B) if const_b else b.arg("B", B.shape)
        c = b.const("C", Cb) if Cb is not None else None
        b.output(b.gemm(a, bb, c, tA, tB, alpha, beta, name="y"), "y")

    feeds = {"A": A}
    if not const_b:
        feeds["B"] = B
    got, want = run_both(build, feeds)
    assert max_rel_err(got["y"], want["y"]) <= F32_TOL


@pytest.mark.parametrize("log", [False, True])
@pytest.mark.parametrize("dims", [(64, 784, 10), (7, 300, 16), (33, 256, 1), (64, 784, 24)])
def test_gemm_bias_softmax_head(dims, log, monkeypatch):
    """Gemm + bias + (Log)Softmax over a handful of columns - the softmax-regression head: one
    launch where the product has at most 16 columns (the row kernel finishes with the Softmax),
    two otherwise (24 columns) or with ODLA_HIP_ROWDOT=0; all against the oracle."""
    M, K, N = dims
    announce("gemm + softmax head %s log=%s" % (dims, log))
    r = rng(111)
    A = r.standard_normal((M, K)).astype(np.float32)
    B = (r.standard_normal((K, N)) * 0.2).astype(np.float32)
    C = r.standard_normal((N,)).astype(np.float32)

    def build(b):
        y = b.gemm(b.arg("A", A.shape), b.const("B", B), b.const("C", C), name="logits")
        b.output(b.softmax(y, -1, log, name="prob"), "prob")

    got, want = run_both(build, {"A": A})
    assert max_rel_err(got["prob"], want["prob"]) <= F32_TOL
    monkeypatch.setenv("ODLA_HIP_ROWDOT", "0")
    apart = run_hip(build, {"A": A})
    assert max_rel_err(apart["prob"], want["prob"]) <= F32_TOL
    if not log:
        assert np.allclose(got["prob"].sum(-1), 1.0, atol=1e-5)


def test_batched_gemm_parity():
    announce("batched gemm")
    r = rng(12)
    q = r.standard_normal((2, 3, 16, 8)).astype(np.float32)
    k = r.standard_normal((2, 3, 16, 8)).astype(np.float32)
    v = r.standard_normal((2, 3, 16, 8)).astype(np.float32)
    wt = r.standard_normal((8, 12)).astype(np.float32)

    def build(b):
        qq, kk, vv = b.arg("q", q.shape), b.arg("k", k.shape), b.arg("v", v.shape)
        s = b.gemm(qq, kk, None, False, True, 0.125, 0.0, name="s")        # [2,3,16,16]
        p = b.softmax(s, -1, name="p")
        o = b.gemm(p, vv, None, False, False, 1.0, 0.0, name="o")           # [2,3,16,8]
        z = b.gemm(o, b.const("w", wt), None, False, False, 1.0, 0.0, name="z")  # rank-2 weights
        b.output(s, "s")
        b.output(o, "o")
        b.output(z, "z")

    got, want = run_both(build, {"q": q, "k": k, "v": v})
    for name in ("s", "o", "z"):
        assert max_rel_err(got[name], want[name]) <= F32_TOL, name


# --------------------------------------------------------------------------
# Element-wise, normalisation, reductions
# --------------------------------------------------------------------------
def test_binary_broadcast_parity():
    announce("binary broadcast")
    r = rng(21)
    x = r.standard_normal((2, 6, 5, 7)).astype(np.float32)
    y = r.standard_normal((2, 6, 5, 7)).astype(np.float32) + 3.0
    c1 = r.standard_normal((1, 6, 1, 1)).astype(np.float32)
    c2 = r.standard_normal((7,)).astype(np.float32)
    c3 = r.standard_normal((6, 1, 1)).astype(np.float32)
    c4 = r.standard_normal((1,)).astype(np.float32)

    def build(b):
        a, bb = b.arg("x", x.shape), b.arg("y", y.shape)
        b.output(b.add(a, bb, name="o_add"), "o_add")
        b.output(b.div(a, bb, name="o_div"), "o_div")
        b.output(b.mul(a, b.const("c1", c1), name="o_c1"), "o_c1")
        b.output(b.sub(b.const("c2", c2), a, name="o_c2"), "o_c2")
        b.output(b.max(a, b.const("c3", c3), name="o_c3"), "o_c3")
        b.output(b.min(a, b.const("c4", c4), name="o_c4"), "o_c4")

    got, want = run_both(build, {"x": x, "y": y})
    for k in want:
        assert max_rel_err(got[k], want[k]) <= 1e-6, k


def test_reference_alignment_quirk():
    """[64] against [1,64,128] aligns with dim 1 (odla_dnnl.h:301-343), not with the last dim."""
    announce("alignment quirk")
    r = rng(22)
    x = r.standard_normal((1, 64, 128)).astype(np.float32)
    c = r.standard_normal((64,)).astype(np.float32)

    def build(b):
        b.output(b.add(b.arg("x", x.shape), b.const("c", c), name="y"), "y")

    got, want = run_both(build, {"x": x})
    assert np.array_equal(want["y"], x + c.reshape(1, 64, 1))
    assert max_rel_err(got["y"], want["y"]) <= 1e-6


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_unary_parity(mode):
    announce("unary %s" % mode)
    r = rng(23)
    x = (r.standard_normal((3, 5, 37)) * 2).astype(np.float32)
    pos = (r.random((3, 5, 37)) + 0.1).astype(np.float32)

    def build(b):
        a, p = b.arg("x", x.shape), b.arg("pos", pos.shape)
        for name in ("relu", "sigmoid", "tanh", "exp", "erf", "abs", "neg"):
            b.output(getattr(b, name)(a, name=name), name)
        b.output(b.gelu(a, False, name="gelu"), "gelu")
        b.output(b.gelu(a, True, name="gelu_tanh"), "gelu_tanh")
        b.output(b.leaky_relu(a, 0.1, name="leaky"), "leaky")
        b.output(b.clamp(a, -0.5, 0.75, name="clamp"), "clamp")
        for name in ("sqrt", "rsqrt", "log"):
            b.output(getattr(b, name)(p, name=name), name)

    got, want = run_both(build, {"x": x, "pos": pos}, fp16=(mode == "fp16"))
    for k in want:
        if mode == "fp32":
            assert max_rel_err(got[k], want[k]) <= F32_TOL, k
        else:
            assert np.max(np.abs(got[k] - want[k])) <= 2e-2 * max(1.0, float(np.max(np.abs(want[k])))), k


def test_gelu_against_the_exact_function():
    """odla_Gelu (erf form) against x * Phi(x) in float64, standalone and in the epilogue of a Gemm:
    absolute error below 1e-6 everywhere and relative error below 1e-5 wherever the result is
    above 1e-6 in magnitude - the negative tail included, where the float formula
    0.5 x (1 + erff(x / sqrt 2)) cancels; 0, -0, large arguments and a NaN."""
    from scipy.special import erfc
    announce("gelu exact")
    r = rng(231)
    x = np.concatenate([np.linspace(-8.0, 8.0, 64 * 511), r.standard_normal(64 * 512) * 2.0,
                        [0.0, -0.0, 1e-20, -1e-20, 30.0, -30.0, -5.65, -5.66, -5.67, 5.66, 1e10, -1e10]])
    x = np.concatenate([x, np.zeros(64 * 1024 - x.size)]).astype(np.float32).reshape(1024, 64)
    eye = np.eye(64, dtype=np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        b.output(b.gelu(a, False, name="alone"), "alone")
        b.output(b.gelu(b.gemm(a, b.const("eye", eye), name="mm"), False, name="fused"), "fused")

    got = run_hip(build, {"x": x})
    xd = x.astype(np.float64)
    want = xd * 0.5 * erfc(-xd / np.sqrt(2.0))
    for k in ("alone", "fused"):
        g = got[k].astype(np.float64)
        err = np.abs(g - want)
        assert err.max() <= 1e-6, (k, err.max(), x.flat[err.argmax()])
        big = np.abs(want) > 1e-6
        rel = err[big] / np.abs(want[big])
        assert rel.max() <= 1e-5, (k, rel.max())

    nan = np.full((64, 64), np.nan, np.float32)
    got = run_hip(lambda b: b.output(b.gelu(b.arg("x", nan.shape), False, name="y"), "y"), {"x": nan})
    assert np.all(np.isnan(got["y"]))


def test_round_half_even():
    announce("round")
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 2.4999, 3.5], np.float32)

    def build(b):
        b.output(b.round(b.arg("x", x.shape), name="y"), "y")

    got = run_hip(build, {"x": x})["y"]
    assert got.tolist() == [0, 2, 2, -0, -2, 2, 4]


@pytest.mark.parametrize("shape,axis", [((64, 10), -1), ((256, 1000), 1), ((4, 12, 16, 16), 3), ((3, 7, 5), 1),
                                        ((2, 3000), 1)])
def test_softmax_parity(shape, axis):
    announce("softmax %s axis %d" % (shape, axis))
    x = (rng(31).standard_normal(shape) * 3).astype(np.float32)

    def build(b):
        a = b.arg("x", shape)
        b.output(b.softmax(a, axis, name="y"), "y")
        b.output(b.softmax(a, axis, log=True, name="ly"), "ly")

    got, want = run_both(build, {"x": x})
    assert max_rel_err(got["y"], want["y"]) <= F32_TOL
    assert np.max(np.abs(got["ly"] - want["ly"])) <= 1e-4
    ax = len(shape) - 1 if axis < 0 else axis
    assert np.allclose(got["y"].sum(axis=ax), 1.0, atol=1e-5)


def test_softmax_large_numbers():
    """ONNX softmax_large_number: inputs near 10000 must not overflow."""
    announce("softmax large")
    x = np.array([[0, 1, 2, 3], [10000, 10001, 10002, 10003]], np.float32)

    def build(b):
        b.output(b.softmax(b.arg("x", x.shape), -1, name="y"), "y")

    got = run_hip(build, {"x": x})["y"]
    expected = np.array([0.032058604, 0.08714432, 0.23688284, 0.6439143], np.float32)
    assert np.allclose(got[0], expected, atol=1e-6) and np.allclose(got[1], expected, atol=1e-6)


@pytest.mark.parametrize("mode", ["fp32", "bf16"])
def test_layernorm_parity(mode):
    announce("layernorm %s" % mode)
    r = rng(41)
    x = r.standard_normal((4, 9, 768)).astype(np.float32) * 2 + 0.5
    g = r.standard_normal(768).astype(np.float32)
    be = r.standard_normal(768).astype(np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        b.output(b.layernorm(a, 1, 1e-12, b.const("g", g), b.const("b", be), name="y"), "y")

    got, want = run_both(build, {"x": x}, bf16=(mode == "bf16"))
    if mode == "fp32":
        assert max_rel_err(got["y"], want["y"]) <= F32_TOL
    else:
        assert np.max(np.abs(got["y"] - want["y"])) <= 6e-2 * float(np.max(np.abs(want["y"])))


def test_batchnorm_standalone_parity():
    announce("batchnorm standalone")
    r = rng(42)
    x = r.standard_normal((2, 12, 6, 5)).astype(np.float32)
    mean, var = r.standard_normal(12).astype(np.float32), (r.random(12) + 0.5).astype(np.float32)
    g, be = r.standard_normal(12).astype(np.float32), r.standard_normal(12).astype(np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        a2 = b.neg(a, name="neg")  # keep the BN from folding into anything
        b.output(b.batchnorm(a2, b.const("m", mean), b.const("v", var), 1e-3, b.const("g", g), b.const("b", be), name="y"), "y")

    got, want = run_both(build, {"x": x})
    assert max_rel_err(got["y"], want["y"]) <= F32_TOL


POOL_CASES = [
    # N, C, H, W, k, s, pad(t,l,b,r), include_pad
    (2, 16, 12, 12, 3, 2, (1, 1, 1, 1), False),
    (1, 5, 9, 7, 2, 2, (0, 0, 0, 0), False),
    (2, 8, 7, 7, 7, 1, (0, 0, 0, 0), False),
    (1, 3, 8, 8, 3, 1, (1, 1, 1, 1), True),
    (1, 4, 6, 6, 3, 2, (0, 0, 1, 1), False),
]


@pytest.mark.parametrize("case", POOL_CASES)
def test_pool_parity(case):
    N, C, H, W, k, s, pad, incl = case
    announce("pool %s" % (case,))
    x = rng(51).standard_normal((N, C, H, W)).astype(np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        b.output(b.maxpool(a, (k, k), (s, s), pad, name="mx"), "mx")
        b.output(b.avgpool(a, (k, k), (s, s), pad, incl, name="av"), "av")

    got, want = run_both(build, {"x": x})
    assert np.array_equal(got["mx"], want["mx"])
    assert max_rel_err(got["av"], want["av"]) <= 1e-6


def test_reduce_parity():
    announce("reduce")
    x = rng(52).standard_normal((3, 10, 7, 7)).astype(np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        b.output(b.reduce_mean(a, (2, 3), True, name="gap"), "gap")
        b.output(b.reduce_mean(a, (3,), False, name="last"), "last")
        b.output(b.reduce_sum(a, (1,), True, name="mid"), "mid")
        b.output(b.reduce_max(a, (1, 2, 3), False, name="mx"), "mx")

    got, want = run_both(build, {"x": x})
    for k in want:
        assert got[k].shape == want[k].shape, k
        assert max_rel_err(got[k], want[k]) <= 1e-5, k


@pytest.mark.parametrize("mode", ["fp32", "fp16", "bf16"])
def test_resize_linear_parity(mode):
    """Bilinear odla_Resize (up, down, mixed, non-integer ratios, a single row) on a
    graph argument and on the channels-last result of a convolution."""
    announce("resize linear (%s)" % mode)
    r = rng(62)
    x = r.standard_normal((2, 6, 5, 7)).astype(np.float32)
    w = (r.standard_normal((8, 6, 1, 1)) * 0.3).astype(np.float32)
    row = r.standard_normal((1, 3, 1, 9)).astype(np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        b.output(b.resize_linear(a, (10, 14), name="up2"), "up2")
        b.output(b.resize_linear(a, (8, 3), name="mixed"), "mixed")
        b.output(b.resize_linear(a, (3, 4), name="down"), "down")
        c = b.conv(a, b.const("w", w), None, name="c")
        b.output(b.resize_linear(c, (9, 16), name="after_conv"), "after_conv")
        b.output(b.resize_linear(b.arg("row", row.shape), (4, 23), name="row_up"), "row_up")

    got, want = run_both(build, {"x": x, "row": row}, fp16=(mode == "fp16"), bf16=(mode == "bf16"))
    for k in want:
        assert got[k].shape == want[k].shape, k
        err = float(np.max(np.abs(got[k] - want[k])))
        if mode == "fp32":
            assert err <= F32_TOL * max(1.0, float(np.max(np.abs(want[k])))), k
        else:
            assert err <= (2e-2 if mode == "fp16" else 6e-2), k


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_reduce_few_columns_parity(mode):
    """Reductions with too few columns to give every thread one: the rows of the
    reduced axis are split over the workgroup (long and short axes, a ragged
    column count, rows of a plain matrix)."""
    announce("reduce, split rows (%s)" % mode)
    r = rng(53)
    x1 = r.standard_normal((2, 64, 40, 40)).astype(np.float32)
    x2 = r.standard_normal((4, 256, 7, 7)).astype(np.float32)
    x3 = r.standard_normal((2, 48, 6, 6)).astype(np.float32)
    x4 = r.standard_normal((3, 40000)).astype(np.float32)

    def build(b):
        for name, x in (("a", x1), ("b", x2), ("c", x3)):
            a = b.arg(name, x.shape)
            cl = b.maxpool(a, (1, 1), (1, 1), (0, 0, 0, 0), name=name + "_cl")   # channels-last on the device
            b.output(b.reduce_mean(cl, (2, 3), True, name=name + "_mean"), name + "_mean")
            b.output(b.reduce_max(cl, (2, 3), False, name=name + "_max"), name + "_max")
            b.output(b.reduce_sum(a, (2, 3), False, name=name + "_sum"), name + "_sum")
        d = b.arg("d", x4.shape)
        b.output(b.reduce_max(d, (1,), False, name="d_max"), "d_max")
        b.output(b.reduce_mean(d, (1,), True, name="d_mean"), "d_mean")

    got, want = run_both(build, {"a": x1, "b": x2, "c": x3, "d": x4}, fp16=(mode == "fp16"))
    for k in want:
        assert got[k].shape == want[k].shape, k
        if mode == "fp32":
            assert np.max(np.abs(got[k] - want[k])) <= 1e-5 * max(1.0, float(np.max(np.abs(want[k])))), k
        else:   # inputs and results rounded to fp16, sums kept in fp32
            assert np.max(np.abs(got[k] - want[k])) <= 2e-3 * max(1.0, float(np.max(np.abs(want[k])))), k


# --------------------------------------------------------------------------
# Data movement
# --------------------------------------------------------------------------
def test_movement_parity():
    announce("movement")
    r = rng(61)
    x = r.standard_normal((2, 6, 4, 5)).astype(np.float32)
    y = r.standard_normal((2, 3, 4, 5)).astype(np.float32)
    table = r.standard_normal((50, 16)).astype(np.float32)
    idx = r.integers(0, 50, size=(3, 7)).astype(np.int32)
    idx64 = r.integers(0, 50, size=(5,)).astype(np.int64)

    def build(b):
        a, c = b.arg("x", x.shape), b.arg("y", y.shape)
        b.output(b.concat([a, c], 1, name="cat1"), "cat1")
        b.output(b.concat([a, a], 3, name="cat3"), "cat3")
        b.output(b.transpose(a, (0, 2, 3, 1), name="nhwc"), "nhwc")
        b.output(b.transpose(a, (1, 0, 3, 2), name="t2"), "t2")
        b.output(b.reshape(a, (2, 6, 20), name="rs"), "rs")
        b.output(b.slice(a, (0, 1, 0, 2), (2, 5, 4, 5), (1, 2, 1, 1), name="sl"), "sl")
        b.output(b.resize_nearest(a, (8, 10), name="up2"), "up2")
        b.output(b.resize_nearest(a, (6, 7), name="upx"), "upx")
        t = b.const("table", table)
        b.output(b.gather(t, b.arg("idx", idx.shape, np.int32), 0, name="emb"), "emb")
        b.output(b.gather(t, b.arg("idx64", idx64.shape, np.int64), 0, name="emb64"), "emb64")

    got, want = run_both(build, {"x": x, "y": y, "idx": idx, "idx64": idx64})
    for k in want:
        assert got[k].shape == want[k].shape, k
        assert np.array_equal(got[k], want[k]), k


@pytest.mark.parametrize("shape,perm,dtype", [
    ((3, 3, 85, 13, 13), (0, 1, 3, 4, 2), np.float32),     # detection head: runs of both sides, ragged tiles
    ((2, 70, 130), (0, 2, 1), np.float32),                 # batched 2-D transpose, several tiles each way
    ((2, 70, 130), (0, 2, 1), np.int64),                   # 8-byte elements
    ((5, 16, 3, 40), (3, 1, 2, 0), np.float32),            # outer dims on both sides of the tile plane
    ((4, 33, 2, 17), (1, 0, 3, 2), np.float32),            # innermost extent too small for tiles
    ((2, 3, 4, 5, 2, 3), (5, 3, 1, 4, 0, 2), np.float32),  # rank 6, nothing merges
    ((1, 64, 1, 48), (3, 2, 1, 0), np.int32),              # extents of 1 drop out
    ((6, 40, 24), (1, 0, 2), np.float32),                  # innermost dim stays: plain runs
])
def test_transpose_paths_parity(shape, perm, dtype):
    """Every route of the strided copy behind odla_Transpose: dims that merge or drop,
    64 x 64 tiles through LDS when the two sides run along different dims, and the
    element-wise walk otherwise.  Bit-exact (data movement)."""
    announce("transpose %s %s %s" % (shape, perm, np.dtype(dtype).name))
    r = rng(65)
    if np.issubdtype(dtype, np.integer):
        x = r.integers(-1000, 1000, size=shape).astype(dtype)
    else:
        x = r.standard_normal(shape).astype(dtype)

    def build(b):
        a = b.arg("x", x.shape, dtype)
        b.output(b.transpose(a, perm, name="t"), "t")

    got, want = run_both(build, {"x": x})
    assert got["t"].shape == want["t"].shape
    assert np.array_equal(got["t"], want["t"])
    assert np.array_equal(got["t"], np.transpose(x, perm))


@pytest.mark.parametrize("shape,perm", [
    ((4, 100, 72), (0, 2, 1)),        # source rows keep 16-byte alignment, destination rows do not
    ((3, 64, 80), (0, 2, 1)),         # both sides aligned: eight elements per request each way
    ((2, 48, 37), (0, 2, 1)),         # only the destination aligned
    ((2, 50, 37), (0, 2, 1)),         # neither: single elements
    ((2, 200, 136), (0, 2, 1)),       # several tiles each way, the last ones partly filled
    ((2, 3, 85, 13, 16), (0, 1, 3, 4, 2)),   # detection head
    ((2, 16, 3, 72), (3, 1, 2, 0)),   # outer dims on both sides of the tile plane
])
def test_transpose_fp16_storage_tiles(shape, perm):
    """2-byte elements through the tiled route (fp16 storage of an fp32 graph), with and
    without 16-byte requests on either side."""
    announce("transpose fp16 tiles %s %s" % (shape, perm))
    x = rng(66).standard_normal(shape).astype(np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        b.output(b.transpose(a, perm, name="t"), "t")

    got = run_hip(build, {"x": x}, fp16=True)
    assert np.array_equal(got["t"], np.transpose(x.astype(np.float16).astype(np.float32), perm))


def test_nhwc_chain_then_concat_resize():
    """Conv -> LeakyReLU -> nearest 2x -> channel concat stays channels-last on the device."""
    announce("nhwc chain")
    r = rng(62)
    x = r.standard_normal((2, 8, 6, 6)).astype(np.float32)
    skip = r.standard_normal((2, 16, 12, 12)).astype(np.float32)
    w1 = (r.standard_normal((8, 8, 3, 3)) * 0.2).astype(np.float32)
    w2 = (r.standard_normal((16, 16, 1, 1)) * 0.2).astype(np.float32)
    w3 = (r.standard_normal((255, 24, 1, 1)) * 0.2).astype(np.float32)

    def build(b):
        a = b.arg("x", x.shape)
        s = b.arg("skip", skip.shape)
        y = b.leaky_relu(b.conv(a, b.const("w1", w1), None, (1, 1), (1, 1, 1, 1), name="c1"), 0.1, name="l1")
        up = b.resize_nearest(y, (12, 12), name="up")
        s2 = b.leaky_relu(b.conv(s, b.const("w2", w2), None, name="c2"), 0.1, name="l2")
        cat = b.concat([up, s2], 1, name="cat")
        head = b.conv(cat, b.const("w3", w3), None, name="head")
        b.output(head, "head")
        b.output(b.sigmoid(head, name="sig"), "sig")

    got, want = run_both(build, {"x": x, "skip": skip})
    assert max_rel_err(got["head"], want["head"]) <= F32_TOL
    assert max_rel_err(got["sig"], want["sig"]) <= F32_TOL


# --------------------------------------------------------------------------
# Quantize / Dequantize
# --------------------------------------------------------------------------
def test_quantize_onnx_example():
    """ONNX QuantizeLinear example (passes on the reference CPU backend):
    rounding at 1.5 -> 2 and saturation at both ends."""
    announce("quantize onnx example")
    x = np.array([0, 2, 3, 1000, -254, -1000], np.float32)

    def build(b):
        q = b.quantize(b.arg("x", x.shape), [2.0], [128], name="q")
        b.output(q, "q")
        b.output(b.dequantize(q, [2.0], [128], name="dq"), "dq")

    got = run_hip(build, {"x": x})
    assert got["q"].tolist() == [128, 129, 130, 255, 1, 0]
    assert got["dq"].tolist() == [0, 2, 4, 254, -254, -256]


def test_quantize_parity_per_axis_and_ties():
    announce("quantize per axis")
    r = rng(71)
    x = (r.standard_normal((2, 4, 9)) * 40).astype(np.float32)
    # exact ties: k + 0.5 multiples of the scale
    x[0, 0, :] = (np.arange(9, dtype=np.float32) - 4 + 0.5) * 0.25
    sc = np.array([0.25, 0.5, 1.0, 2.0], np.float32)
    zp = np.array([0, 10, 128, 200], np.uint8)

    def build(b):
        a = b.arg("x", x.shape)
        q = b.quantize(a, sc, zp, axis=1, name="q")
        b.output(q, "q")
        b.output(b.dequantize(q, sc, zp, axis=1, name="dq"), "dq")
        b.output(b.quantize(a, [0.5], None, signed=True, name="qs"), "qs")

    got, want = run_both(build, {"x": x})
    assert np.array_equal(got["q"], want["q"])
    assert np.array_equal(got["dq"], want["dq"])
    assert np.array_equal(got["qs"], want["qs"])


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
@pytest.mark.parametrize("scale", [0.02, 0.037, 1.0 / 3.0, 2.0])
def test_quantize_per_tensor_large_with_near_ties(mode, scale):
    """Per-tensor parameters on a tensor large enough for the tiled path, whose rounding avoids
    the division where x * (1 / scale) is clearly away from a rounding boundary: values placed
    on and one float step beside every boundary k + 0.5 must give the oracle's levels (the
    oracle divides), as must values far outside the range, in unsigned, stored-signed and
    signed form."""
    announce("quantize per tensor, near ties, %s scale %g" % (mode, scale))
    r = rng(72)
    n = 3 * 8192 + 40          # three full tiles and a ragged rest
    x = (r.standard_normal(n) * 60 * scale).astype(np.float32)
    k = np.arange(-140, 140, dtype=np.float32)
    ties = ((k + 0.5) * np.float32(scale)).astype(np.float32)
    x[:280] = ties
    x[280:560] = np.nextafter(ties, np.float32(np.inf))
    x[560:840] = np.nextafter(ties, np.float32(-np.inf))
    x[840:850] = [1e30, -1e30, 3e4, -3e4, 0.0, -0.0, 1e-30, -1e-30, 255 * scale, 256 * scale]
    x[9000:9280] = ties * np.float32(1.0000001)
    if mode == "fp16":
        x = x.astype(np.float16).astype(np.float32)
    x = x.reshape(1, -1)

    def build(b):
        a = b.arg("x", x.shape)
        b.output(b.quantize(a, [scale], [117], name="qu"), "qu")
        b.output(b.quantize(a, [scale], None, signed=True, name="qs"), "qs")

    got, want = run_both(build, {"x": x}, fp16=mode == "fp16")
    assert np.array_equal(got["qu"], want["qu"])
    assert np.array_equal(got["qs"], want["qs"])


# --------------------------------------------------------------------------
# NMS
# --------------------------------------------------------------------------
def test_nms_onnx_examples():
    """Published ONNX NonMaxSuppression cases (single class): suppress by IoU ->
    [3, 0, 5]; identical boxes -> 1 box; flipped coordinates; score threshold."""
    announce("nms onnx examples")
    boxes = np.array([[[0, 0, 1, 1], [0, 0.1, 1, 1.1], [0, -0.1, 1, 0.9], [0, 10, 1, 11], [0, 10.1, 1, 11.1],
                       [0, 100, 1, 101]]], np.float32)
    flipped = np.array([[[1, 1, 0, 0], [0, 0.1, 1, 1.1], [0, 0.9, 1, -0.1], [0, 10, 1, 11], [1, 10.1, 0, 11.1],
                         [1, 101, 0, 100]]], np.float32)
    scores = np.array([[[0.9, 0.75, 0.6, 0.95, 0.5, 0.3]]], np.float32)
    same = np.tile(np.array([0, 0, 1, 1], np.float32), (1, 10, 1))
    same_scores = np.full((1, 1, 10), 0.9, np.float32)

    def build(b):
        bx, sc = b.arg("boxes", boxes.shape), b.arg("scores", scores.shape)
        fl = b.arg("flipped", flipped.shape)
        sm, ss = b.arg("same", same.shape), b.arg("same_scores", same_scores.shape)
        b.output(b.nms(bx, sc, 3, 0.5, 0.0, name="a"), "a")
        b.output(b.nms(fl, sc, 3, 0.5, 0.0, name="f"), "f")
        b.output(b.nms(bx, sc, 3, 0.5, 0.4, name="t"), "t")
        b.output(b.nms(bx, sc, 2, 0.5, 0.0, name="m2"), "m2")
        b.output(b.nms(sm, ss, 3, 0.5, 0.0, name="s"), "s")

    got = run_hip(build, {"boxes": boxes, "scores": scores, "flipped": flipped, "same": same,
                          "same_scores": same_scores})
    assert got["a"].tolist() == [[0, 0, 3], [0, 0, 0], [0, 0, 5]]
    assert got["f"].tolist() == [[0, 0, 3], [0, 0, 0], [0, 0, 5]]
    assert got["t"].tolist() == [[0, 0, 3], [0, 0, 0], [-1, -1, -1]]
    assert got["m2"].tolist() == [[0, 0, 3], [0, 0, 0]]
    assert got["s"].tolist() == [[0, 0, 0], [-1, -1, -1], [-1, -1, -1]]


# (the last case has more candidates than the kernel keeps in LDS: 40 000 boxes on a wide field)
# (the one before: more results allowed than the kernel lists in LDS before it writes them)
@pytest.mark.parametrize("N,B,C,max_out", [(2, 200, 5, 20), (3, 1500, 80, 100), (1, 64, 1, 64), (2, 2100, 3, 128),
                                           (1, 6000, 1, 2500), (2, 40000, 2, 300)])
def test_nms_parity_random(N, B, C, max_out):
    announce("nms random %s" % ((N, B, C, max_out),))
    r = rng(81 + B)
    span = 10 if B < 10000 else 120
    cy, cx = r.random((N, B)) * span, r.random((N, B)) * span
    h, w = r.random((N, B)) * 2 + 0.2, r.random((N, B)) * 2 + 0.2
    boxes = np.stack([cy - h / 2, cx - w / 2, cy + h / 2, cx + w / 2], axis=-1).astype(np.float32)
    scores = r.random((N, C, B)).astype(np.float32) ** 4
    scores[:, :, :5] = 0.77  # ties resolved by box index

    def build(b):
        b.output(b.nms(b.arg("boxes", boxes.shape), b.arg("scores", scores.shape), max_out, 0.45, 0.3, name="y"), "y")

    got, want = run_both(build, {"boxes": boxes, "scores": scores})
    assert np.array_equal(got["y"], want["y"])


@pytest.mark.parametrize("mode", ["fp32", "bf16"])
def test_sibling_gemms_share_one_launch(mode):
    """Several GEMMs of one left operand against constant matrices of one shape (attention
    projections) run as one batched launch; a sibling with another tail (ReLU), one whose
    result is a graph output, one with another shape and one with a scalar factor stay on
    their own - all must come out as if computed alone."""
    announce("sibling gemms %s" % mode)
    r = rng(77)
    B_, S_, H_ = 3, 40, 96
    x = r.standard_normal((B_, S_, H_)).astype(np.float32)
    ws = [(r.standard_normal((H_, H_)) * 0.1).astype(np.float32) for _ in range(6)]
    bs = [r.standard_normal((H_,)).astype(np.float32) for _ in range(6)]
    w_wide = (r.standard_normal((H_, 2 * H_)) * 0.1).astype(np.float32)

    def build(b):
        v = b.arg("x", x.shape)
        h = b.tanh(v, name="h")                          # the shared operand is a computed value
        q = b.add(b.gemm(h, b.const("w0", ws[0]), name="q0"), b.const("b0", bs[0]), name="q")
        k = b.add(b.gemm(h, b.const("w1", ws[1]), name="k0"), b.const("b1", bs[1]), name="k")
        vv = b.gemm(h, b.const("w2", ws[2]), name="v")   # no bias
        rl = b.relu(b.add(b.gemm(h, b.const("w3", ws[3]), name="r0"), b.const("b3", bs[3]), name="r1"), name="rl")
        out_direct = b.gemm(h, b.const("w4", ws[4]), b.const("b4", bs[4].reshape(1, H_)), name="direct")
        wide = b.gemm(h, b.const("ww", w_wide), name="wide")
        half = b.gemm(h, b.const("w5", ws[5]), alpha=0.5, name="half")
        s = b.add(b.add(q, k, name="qk"), b.add(vv, rl, name="vr"), name="s")
        b.output(b.add(s, half, name="total"), "total")
        b.output(out_direct, "direct")
        b.output(wide, "wide")
        # head split of one projection, as attention does
        b.output(b.transpose(b.reshape(k, (B_, S_, 4, H_ // 4), name="kr"), (0, 2, 1, 3), name="kt"), "kt")

    kw = {"bf16": mode == "bf16"}
    got, want = run_both(build, {"x": x}, **kw)
    for name in want:
        if mode == "fp32":
            assert max_rel_err(got[name], want[name]) <= F32_TOL, name
        else:
            assert np.max(np.abs(got[name] - want[name])) <= 6e-2 * max(1.0, float(np.max(np.abs(want[name])))), name
