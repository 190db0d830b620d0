"""End-to-end parity of whole graphs through the ODLA C ABI against the CPU
oracle: the mnist softmax regression (config 0) and ResNet-50-shaped networks
(reduced depth/width so the CPU oracle finishes in seconds; the full-size
network is covered by test_gpu_resnet50_full.py).
"""
import numpy as np
import pytest

from util import run_ref_emulated, announce, max_rel_err, run_hip, run_ref

pytestmark = pytest.mark.gpu

SMALL_STAGES = [(16, 2, 1), (32, 2, 2), (64, 1, 2)]


def test_mnist_softmax_regression_fp32(models):
    """Config 0: Gemm + Add + Softmax, N=64, fp32; max rel err 1e-4 on probabilities."""
    announce("mnist fp32")
    w = models.mnist_weights()
    feeds = models.mnist_input(64)
    build = lambda b: models.build_mnist(b, w, 64)
    got = run_hip(build, feeds, repeats=3)["y"]
    want = run_ref(build, feeds)["y"]
    rel = np.max(np.abs(got - want) / np.abs(want))
    assert rel <= 1e-4, rel
    assert np.array_equal(np.argmax(got, 1), np.argmax(want, 1))


def test_mnist_with_the_reference_weights(pkg, models):
    """Config 0 with the trained weights of the reference's mnist_simple.pb (tests/golden holds a
    copy of that data file), read by the GraphDef constant extractor."""
    announce("mnist fp32, trained weights")
    import os
    import __graft_entry__ as entry
    consts = pkg.weights.read_graphdef_constants(open(os.path.join(entry.ROOT, "tests", "golden", "mnist_simple.pb"), "rb").read())
    w = {"V": consts["Variable"], "V1": consts["Variable_1"].reshape(1, 10)}
    feeds = models.mnist_input(64, seed=77)
    build = lambda b: models.build_mnist(b, w, 64)
    got = run_hip(build, feeds)["y"]
    want = run_ref(build, feeds)["y"]
    assert np.max(np.abs(got - want)) <= 1e-4 * float(np.max(want))
    assert np.array_equal(np.argmax(got, 1), np.argmax(want, 1))
    assert np.max(np.abs(got.sum(axis=1) - 1.0)) <= 1e-5


def test_small_resnet_fp32(models):
    announce("small resnet fp32")
    w = models.resnet50_weights(seed=3, num_classes=100, stages=SMALL_STAGES, stem=16)
    feeds = models.resnet50_input(4, 64, seed=4)
    build = lambda b: models.build_resnet50(b, w, 4, 64, SMALL_STAGES, 16, 100)
    got = run_hip(build, feeds)
    want = run_ref(build, feeds)
    assert max_rel_err(got["logits"], want["logits"]) <= 1e-4
    assert max_rel_err(got["prob"], want["prob"]) <= 1e-4
    assert np.array_equal(np.argmax(got["logits"], 1), np.argmax(want["logits"], 1))


@pytest.mark.parametrize("mode", ["fp16", "bf16"])
def test_small_resnet_reduced_precision(models, mode):
    """fp16 / bf16 storage with fp32 accumulation: 2e-2 abs on logits (fp16), top-1 equal."""
    announce("small resnet %s" % mode)
    w = models.resnet50_weights(seed=3, num_classes=100, stages=SMALL_STAGES, stem=16)
    feeds = models.resnet50_input(4, 64, seed=4)
    build = lambda b: models.build_resnet50(b, w, 4, 64, SMALL_STAGES, 16, 100)
    got = run_hip(build, feeds, fp16=(mode == "fp16"), bf16=(mode == "bf16"))
    want = run_ref(build, feeds)
    # fp16: 2e-2 absolute; bf16 (8 significant bits) the same bound relative to the logit magnitude
    tol = 2e-2 if mode == "fp16" else 2e-2 * max(1.0, float(np.max(np.abs(want["logits"]))))
    assert np.max(np.abs(got["logits"] - want["logits"])) <= tol
    if mode == "fp16":
        assert np.array_equal(np.argmax(got["logits"], 1), np.argmax(want["logits"], 1))


def test_small_resnet_bf16_accuracy_mode(models):
    """BF16_ACCURACY_MODE: values stay fp32, only Conv / Gemm operands are bf16.  Against the oracle
    that rounds exactly those operands the logits agree to a small fraction of what the operand
    rounding itself costs; against fp32 they are several times closer than with bf16 storage."""
    announce("small resnet bf16, accuracy mode")
    w = models.resnet50_weights(seed=3, num_classes=100, stages=SMALL_STAGES, stem=16)
    feeds = models.resnet50_input(4, 64, seed=4)
    build = lambda b: models.build_resnet50(b, w, 4, 64, SMALL_STAGES, 16, 100)
    got = run_hip(build, feeds, bf16="accuracy")["logits"]
    perf = run_hip(build, feeds, bf16="performance")["logits"]
    want = run_ref(build, feeds)["logits"]
    emu = run_ref_emulated(build, feeds, "operands", "bf16")["logits"]
    floor = float(np.max(np.abs(emu - want)))
    e_acc, e_perf, d = (float(np.max(np.abs(a - b))) for a, b in ((got, want), (perf, want), (got, emu)))
    announce("small resnet bf16: operands floor %.3e, accuracy mode vs fp32 %.3e, vs emulated %.3e; performance mode vs fp32 %.3e"
             % (floor, e_acc, d, e_perf))
    assert e_acc <= 1.5 * floor and d <= floor
    assert np.array_equal(np.argmax(got, 1), np.argmax(emu, 1))


def test_graph_replay_equals_eager(models):
    """hipGraph replay (several times, with eager executions in between) gives the
    same bytes as the un-captured launch sequence."""
    announce("graph replay")
    w = models.resnet50_weights(seed=5, num_classes=10, stages=[(8, 1, 1), (16, 1, 2)], stem=8)
    build = lambda b: models.build_resnet50(b, w, 2, 32, [(8, 1, 1), (16, 1, 2)], 8, 10)
    f1 = models.resnet50_input(2, 32, seed=6)
    f2 = models.resnet50_input(2, 32, seed=7)
    eager1 = run_hip(build, f1, use_graph=False)
    eager2 = run_hip(build, f2, use_graph=False)
    import __graft_entry__ as entry
    pkg = entry.load()
    hb = pkg.odla.HipBuilder()
    build(hb)
    s = hb.session(True)
    for f, e in ((f1, eager1), (f2, eager2), (f1, eager1), (f2, eager2)):
        out = s.run(f)
        assert np.array_equal(out["logits"], e["logits"])
        assert np.array_equal(out["prob"], e["prob"])
    s.close()
    hb.destroy()


def test_device_resident_io(models, odla):
    """Binding device pointers (odla_AllocateDeviceMemory) gives the same result as host buffers."""
    announce("device io")
    w = models.mnist_weights()
    feeds = models.mnist_input(64)
    hb = odla.HipBuilder()
    models.build_mnist(hb, w, 64)
    s = hb.session()
    host = s.run(feeds)["y"].copy()
    s.bind_device_io(feeds)
    s.execute()
    s.execute()
    dev = s.fetch_device_outputs()["y"]
    s.close()
    hb.destroy()
    assert np.array_equal(host, dev)


def test_two_contexts_and_error_paths(models, odla):
    """Two contexts over one computation; unknown ids and unbound arguments are
    reported as status codes, not crashes."""
    announce("contexts and errors")
    import ctypes
    w = models.mnist_weights()
    feeds = models.mnist_input(64)
    hb = odla.HipBuilder()
    models.build_mnist(hb, w, 64)
    s1, s2 = hb.session(), hb.session()
    a = s1.run(feeds)["y"]
    b = s2.run(feeds)["y"]
    assert np.array_equal(a, b)
    L = hb.L
    buf = np.zeros((64, 784), np.float32)
    st = L.odla_BindToArgumentById(b"nope", buf.ctypes.data_as(ctypes.c_void_p), s1.ctx)
    assert st == odla.ODLA_INVALID_PARAM
    s3 = hb.session()
    st = L.odla_ExecuteComputation(hb.comp, s3.ctx, odla.ODLA_COMPUTE_INFERENCE, None)
    assert st == odla.ODLA_INVALID_PARAM  # argument not bound
    # a compiled computation with contexts takes no further operators: they could not run
    L.odla_SetLogLevel(0)
    with pytest.raises(odla.OdlaError):
        hb.relu(hb.outs["y"][0], name="late")
    L.odla_SetLogLevel(2)
    assert np.array_equal(s1.run(feeds)["y"], a)
    for s in (s1, s2, s3):
        s.close()
    hb.destroy()
