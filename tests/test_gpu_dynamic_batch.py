"""Dynamic batch through the C ABI: a computation recorded once with
ODLA_DYNAMIC_BATCH / ODLA_MAX_BATCH_SIZE and a batch extent of -1 runs at every
batch up to the largest one (ODLA_RUN_BATCH_SIZE, odla_SetRuntimeShape) and must
give what the oracle gives for a graph built at that batch.
[ref: ODLA/platforms/tensorrt/odla_tensorrt.cc:138-179,251-296;
 lib/target/generic_cpp/generic_cxx_codegen.cc:624-637,848-852 - the calls the
 generated code makes]"""
import ctypes

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, max_rel_err, run_ref

pytestmark = pytest.mark.gpu


def cnn_weights(seed):
    r = np.random.default_rng(seed)
    return {"w1": (r.standard_normal((32, 3, 3, 3)) * 0.2).astype(np.float32),
            "b1": r.standard_normal(32).astype(np.float32) * 0.1,
            "w2": (r.standard_normal((32, 32, 3, 3)) * 0.06).astype(np.float32),
            "w3": (r.standard_normal((96, 32, 1, 1)) * 0.15).astype(np.float32),
            "b3": r.standard_normal(96).astype(np.float32) * 0.1,
            "wf": (r.standard_normal((96, 10)) * 0.2).astype(np.float32),
            "bf": r.standard_normal((1, 10)).astype(np.float32)}


def build_cnn(w, batch):
    """batch: -1 for the dynamic recording, the actual batch for the oracle."""
    def build(b):
        x = b.arg("x", (batch, 3, 20, 20))
        c1 = b.relu(b.conv(x, b.const("w1", w["w1"]), b.const("b1", w["b1"]), (1, 1), (1, 1, 1, 1), name="c1"), name="r1")
        p1 = b.maxpool(c1, (2, 2), (2, 2), (0, 0, 0, 0), name="p1")
        c2 = b.conv(p1, b.const("w2", w["w2"]), None, (1, 1), (1, 1, 1, 1), name="c2")
        s = b.relu(b.add(c2, p1, name="sum"), name="r2")                         # residual
        c3 = b.relu(b.conv(s, b.const("w3", w["w3"]), b.const("b3", w["b3"]), (1, 1), (0, 0, 0, 0), name="c3"), name="r3")
        g = b.reduce_mean(c3, (2, 3), True, name="gap")
        f = b.reshape(g, (-1, 96), name="flat")
        y = b.softmax(b.gemm(f, b.const("wf", w["wf"]), b.const("bf", w["bf"]), name="fc"), -1, name="prob")
        b.output(c3, "c3")
        b.output(y, "prob")
    return build


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_cnn_runs_at_every_batch_up_to_the_largest(mode):
    odla = entry.load().odla
    w = cnn_weights(3)
    MAXB = 12
    hb = odla.HipBuilder(fp16=(mode == "fp16"), max_batch=MAXB)
    try:
        build_cnn(w, -1)(hb)
        s = hb.session(True)
        try:
            r = np.random.default_rng(4)
            # back and forth between batches: every batch keeps its own plan, arena and graph
            for bs in (MAXB, 1, 5, MAXB, 3, 1, 5):
                announce("dynamic batch cnn %s batch %d" % (mode, bs))
                x = r.standard_normal((bs, 3, 20, 20)).astype(np.float32)
                s.set_batch(bs)
                assert s.runtime_shape(hb.outs["c3"][0]) == (bs, 96, 10, 10)
                got = s.run({"x": x})
                want = run_ref(build_cnn(w, bs), {"x": x})
                assert got["prob"].shape == (bs, 10) and got["c3"].shape == (bs, 96, 10, 10)
                tol = 1e-4 if mode == "fp32" else 2e-2
                assert max_rel_err(got["c3"], want["c3"]) <= tol, bs
                assert np.max(np.abs(got["prob"] - want["prob"])) <= (1e-5 if mode == "fp32" else 2e-2), bs
        finally:
            s.close()
    finally:
        hb.destroy()


def attention_weights(seed, H, V, S):
    r = np.random.default_rng(seed)
    g = lambda *sh: (r.standard_normal(sh) * 0.08).astype(np.float32)
    return {"emb": g(V, H), "pos": g(S, H), "wq": g(H, H), "wk": g(H, H), "wv": g(H, H), "wo": g(H, H),
            "bq": g(1, H), "bk": g(1, H), "bv": g(1, H), "bo": g(1, H),
            "g": (1 + g(H)).astype(np.float32), "be": g(H)}


def build_attention(w, batch, S, H, heads):
    """Embedding gather, one self-attention block with a mask, layer norm: the
    reshapes, the head transpose and the batched products of a BERT encoder."""
    dh = H // heads

    def build(b):
        ids = b.arg("ids", (batch, S), np.int32)
        mask = b.arg("mask", (batch, S), np.float32)
        e = b.gather(b.const("emb", w["emb"]), ids, 0, name="tok")             # [B,S,H]
        e = b.add(e, b.const("pos", w["pos"]), name="emb_sum")
        x2 = b.reshape(e, (-1, H), name="x2")                                   # [B*S,H]
        def heads_of(t, nm):
            return b.transpose(b.reshape(t, (-1, S, heads, dh), name=nm + "_r"), (0, 2, 1, 3), name=nm + "_t")
        q = heads_of(b.gemm(x2, b.const("wq", w["wq"]), b.const("bq", w["bq"]), name="q"), "q")
        k = heads_of(b.gemm(x2, b.const("wk", w["wk"]), b.const("bk", w["bk"]), name="k"), "k")
        v = heads_of(b.gemm(x2, b.const("wv", w["wv"]), b.const("bv", w["bv"]), name="v"), "v")
        sc = b.gemm(q, k, None, False, True, 1.0 / np.sqrt(dh), 0.0, name="scores")      # [B,h,S,S]
        m = b.reshape(mask, (-1, 1, 1, S), name="mask4")
        neg = b.mul(b.sub(m, b.const("one", np.ones(1, np.float32)), name="m1"), b.const("big", np.full(1, 10000.0, np.float32)), name="bias")
        pr = b.softmax(b.add(sc, neg, name="masked"), -1, name="probs")
        ctxv = b.gemm(pr, v, name="ctx")                                          # [B,h,S,dh]
        ctx2 = b.reshape(b.transpose(ctxv, (0, 2, 1, 3), name="ctx_t"), (-1, H), name="ctx2")
        o = b.add(b.gemm(ctx2, b.const("wo", w["wo"]), b.const("bo", w["bo"]), name="o"), x2, name="res")
        y = b.layernorm(b.reshape(o, (-1, S, H), name="o3"), 1, 1e-5, b.const("g", w["g"]), b.const("be", w["be"]), name="ln")
        b.output(y, "ln")
    return build


@pytest.mark.parametrize("mode", ["fp32", "bf16"])
def test_attention_block_with_gather_reshape_and_head_transposes(mode):
    odla = entry.load().odla
    S, H, heads, V, MAXB = 16, 64, 4, 50, 6
    w = attention_weights(7, H, V, S)
    hb = odla.HipBuilder(bf16=(mode == "bf16"), max_batch=MAXB)
    try:
        build_attention(w, -1, S, H, heads)(hb)
        s = hb.session(True)
        try:
            r = np.random.default_rng(8)
            for bs in (2, MAXB, 1, 4, 2):
                announce("dynamic batch attention %s batch %d" % (mode, bs))
                ids = r.integers(0, V, (bs, S)).astype(np.int32)
                mask = (r.random((bs, S)) > 0.2).astype(np.float32)
                mask[:, 0] = 1
                s.set_batch(bs)
                got = s.run({"ids": ids, "mask": mask})["ln"]
                want = run_ref(build_attention(w, bs, S, H, heads), {"ids": ids, "mask": mask})["ln"]
                assert got.shape == (bs, S, H)
                assert np.max(np.abs(got - want)) <= (2e-4 if mode == "fp32" else 6e-2), bs
        finally:
            s.close()
    finally:
        hb.destroy()


def test_set_runtime_shape_and_limits():
    odla = entry.load().odla
    L = odla.load_library()
    w = cnn_weights(5)
    hb = odla.HipBuilder(max_batch=4)
    try:
        build_cnn(w, -1)(hb)
        s = hb.session(True)
        try:
            xh = hb.args["x"][0]
            announce("dynamic batch: odla_SetRuntimeShape")
            assert L.odla_SetRuntimeShape(s.ctx, xh, odla.make_shape((3, 3, 20, 20))) == 0
            assert s.runtime_shape(xh) == (3, 3, 20, 20)
            t = odla.ValueType()
            assert L.odla_GetRuntimeValueType(s.ctx, hb.outs["prob"][0], ctypes.byref(t)) == 0
            assert (t.shape.size, t.shape.dims[0], t.shape.dims[1]) == (2, 3, 10)
            x = np.random.default_rng(6).standard_normal((3, 3, 20, 20)).astype(np.float32)
            got = s.run({"x": x})
            want = run_ref(build_cnn(w, 3), {"x": x})
            assert np.max(np.abs(got["prob"] - want["prob"])) <= 1e-5
            # refused: another extent than the batch, a batch beyond the largest, a value that is no argument
            assert L.odla_SetRuntimeShape(s.ctx, xh, odla.make_shape((3, 3, 24, 24))) != 0
            assert L.odla_SetRuntimeShape(s.ctx, xh, odla.make_shape((5, 3, 20, 20))) != 0
            assert L.odla_SetRuntimeShape(s.ctx, hb.outs["prob"][0], odla.make_shape((3, 10))) != 0
            with pytest.raises(odla.OdlaError):
                s.set_batch(0)
            with pytest.raises(odla.OdlaError):
                s.set_batch(5)
            # the refused calls changed nothing
            assert s.runtime_shape(xh) == (3, 3, 20, 20)
            got2 = s.run({"x": x})
            assert np.array_equal(got2["prob"], got["prob"])
        finally:
            s.close()
    finally:
        hb.destroy()
    # a computation recorded without the items has no run-time batch, and -1 is refused at record time
    hb = odla.HipBuilder()
    try:
        with pytest.raises(odla.OdlaError):
            hb.arg("x", (-1, 3, 8, 8))
        build_cnn(w, 2)(hb)
        s = hb.session(True)
        try:
            with pytest.raises(odla.OdlaError):
                s.set_batch(1)
        finally:
            s.close()
    finally:
        hb.destroy()


def test_graphs_that_move_the_batch_are_refused_but_run_at_the_recorded_batch():
    odla = entry.load().odla
    r = np.random.default_rng(9)
    wt = (r.standard_normal((8, 6)) * 0.3).astype(np.float32)

    def build(batch):
        def f(b):
            x = b.arg("x", (batch, 5, 8))
            t = b.transpose(x, (1, 0, 2), name="t")                 # the batch leaves the leading extent
            y = b.gemm(b.reshape(t, (-1, 8), name="r"), b.const("w", wt), name="y")
            b.output(y, "y")
        return f

    def build_reduce(batch):
        def f(b):
            x = b.arg("x", (batch, 5, 8))
            b.output(b.reduce_sum(x, (0,), True, name="s"), "s")
        return f

    for bld, key in ((build, "y"), (build_reduce, "s")):
        hb = odla.HipBuilder(max_batch=4)
        try:
            bld(-1)(hb)
            s = hb.session(True)
            try:
                announce("dynamic batch: refused graph, output %s" % key)
                with pytest.raises(odla.OdlaError):
                    s.set_batch(2)
                x = r.standard_normal((4, 5, 8)).astype(np.float32)
                got = s.run({"x": x})
                want = run_ref(bld(4), {"x": x})
                assert max_rel_err(got[key], want[key]) <= 1e-4
            finally:
                s.close()
        finally:
            hb.destroy()


def test_axis_operators_with_a_dynamic_batch():
    """Hardmax, CumSum and GatherElements along a non-batch axis follow the batch; along the
    batch (or with indices that do not depend on it) the batch cannot be changed."""
    odla = entry.load().odla
    r = np.random.default_rng(19)
    MAXB = 6

    def build(batch):
        def f(b):
            x = b.arg("x", (batch, 7, 9))
            idx = b.arg("idx", (batch, 4, 9), np.int32)
            b.output(b.hardmax(x, 2, name="hm"), "hm")
            b.output(b.cumsum(x, 1, exclusive=True, name="cs"), "cs")
            b.output(b.gather_elements(x, idx, 1, name="ge"), "ge")
        return f

    hb = odla.HipBuilder(max_batch=MAXB)
    try:
        build(-1)(hb)
        s = hb.session(True)
        try:
            for bs in (MAXB, 2, 5):
                announce("dynamic batch axis operators, batch %d" % bs)
                feeds = {"x": np.round(r.standard_normal((bs, 7, 9)) * 3).astype(np.float32),
                         "idx": r.integers(-7, 7, (bs, 4, 9)).astype(np.int32)}
                s.set_batch(bs)
                got = s.run(feeds)
                want = run_ref(build(bs), feeds)
                for k in want:
                    assert got[k].shape == want[k].shape and np.array_equal(got[k], want[k]), (k, bs)
        finally:
            s.close()
    finally:
        hb.destroy()

    def along_batch(b):
        b.output(b.cumsum(b.arg("x", (-1, 7, 9)), 0, name="cs"), "cs")

    def constant_indices(b):
        x = b.arg("x", (-1, 7, 9))
        b.output(b.gather_elements(x, b.const("i", np.zeros((MAXB, 2, 9), np.int32)), 1, name="ge"), "ge")

    for bld in (along_batch, constant_indices):
        hb = odla.HipBuilder(max_batch=MAXB)
        try:
            bld(hb)
            s = hb.session(True)
            try:
                with pytest.raises(odla.OdlaError):
                    s.set_batch(3)
            finally:
                s.close()
        finally:
            hb.destroy()


def test_int8_plan_at_a_smaller_batch_is_bit_exact():
    """The quantisation table names values, so the same table drives the plan of every batch."""
    pkg = entry.load()
    odla, models = pkg.odla, pkg.models
    r = np.random.default_rng(11)
    w1 = (r.standard_normal((64, 16, 3, 3)) * 0.1).astype(np.float32)
    b1 = (r.standard_normal(64) * 0.1).astype(np.float32)

    def build(batch):
        def f(b):
            x = b.arg("x", (batch, 16, 14, 14))
            xr = b.relu(x, name="xr")
            y = b.relu(b.conv(xr, b.const("w1", w1), b.const("b1", b1), (1, 1), (1, 1, 1, 1), name="c1"), name="r1")
            b.output(y, "r1")
        return f

    MAXB = 6
    entries = []
    for name, (lo, hi) in {"x": (0.0, 4.5), "xr": (0.0, 4.5), "r1": (0.0, 3.0)}.items():
        scale, zp = models.act_qparams(lo, hi)
        entries.append((name, scale, zp, lo, hi, None))
    wt = w1.reshape(w1.shape[0], -1)
    entries.append(("w1", 1.0, 0, float(wt.min()), float(wt.max()),
                    list(zip(wt.min(axis=1).tolist(), wt.max(axis=1).tolist()))))
    table = odla.quant_table(entries)
    hb = odla.HipBuilder(quant_table=table, max_batch=MAXB)
    try:
        build(-1)(hb)
        s = hb.session(True)
        try:
            base = np.abs(r.standard_normal((MAXB, 16, 14, 14))).astype(np.float32)
            announce("dynamic batch int8: batch %d" % MAXB)
            full = s.run({"x": base})["r1"]
            for bs in (1, 4):
                announce("dynamic batch int8: batch %d" % bs)
                s.set_batch(bs)
                got = s.run({"x": base[:bs]})["r1"]
                # integer arithmetic per image: the first rows of the full batch, bit for bit
                assert np.array_equal(got, full[:bs]), bs
        finally:
            s.close()
    finally:
        hb.destroy()


def test_stored_executable_keeps_the_dynamic_batch(tmp_path):
    """Store the recording, destroy it, load it as an executable: the loaded
    computation still runs at a smaller batch."""
    odla = entry.load().odla
    L = odla.load_library()
    w = cnn_weights(13)
    loc, keep = odla.path_location(str(tmp_path / "dyn.odla"))
    hb = odla.HipBuilder(max_batch=5)
    try:
        build_cnn(w, -1)(hb)
        exe0 = ctypes.c_void_p()
        assert L.odla_CompileComputation(hb.comp, None, ctypes.byref(exe0)) == 0
        assert L.odla_StoreExecutable(loc, exe0) == 0
    finally:
        hb.destroy()
    exe = ctypes.c_void_p()
    assert L.odla_LoadExecutable(loc, None, ctypes.byref(exe)) == 0
    ctx = ctypes.c_void_p()
    assert L.odla_CreateContext(ctypes.byref(ctx)) == 0
    try:
        for bs in (2, 5):
            announce("dynamic batch: stored executable at batch %d" % bs)
            n = ctypes.c_int(bs)
            assert L.odla_SetContextItem(ctx, odla.ODLA_RUN_BATCH_SIZE, ctypes.byref(n)) == 0
            x = np.random.default_rng(14 + bs).standard_normal((bs, 3, 20, 20)).astype(np.float32)
            prob = np.empty((bs, 10), np.float32)
            c3 = np.empty((bs, 96, 10, 10), np.float32)
            assert L.odla_BindToArgumentById(b"x", x.ctypes.data_as(ctypes.c_void_p), ctx) == 0
            assert L.odla_BindToOutputById(b"prob", prob.ctypes.data_as(ctypes.c_void_p), ctx) == 0
            assert L.odla_BindToOutputById(b"r3", c3.ctypes.data_as(ctypes.c_void_p), ctx) == 0
            assert L.odla_LaunchExecutable(exe, ctx) == 0
            want = run_ref(build_cnn(w, bs), {"x": x})
            assert np.max(np.abs(prob - want["prob"])) <= 1e-5
            assert max_rel_err(c3, want["c3"]) <= 1e-4
    finally:
        L.odla_DestroyContext(ctx)
        assert L.odla_DestroyExecutable(exe) == 0


SMALL_STAGES = [(16, 2, 1), (32, 2, 2), (64, 1, 2)]


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_resnet_builder_recorded_with_a_dynamic_batch(mode):
    """The package's ResNet-50 builder (stem with its space-to-depth copy, bottleneck
    blocks with projection shortcuts, pooling, classifier) recorded once at batch -1."""
    pkg = entry.load()
    odla, models = pkg.odla, pkg.models
    w = models.resnet50_weights(seed=3, num_classes=100, stages=SMALL_STAGES, stem=16)
    MAXB = 6
    hb = odla.HipBuilder(fp16=(mode == "fp16"), max_batch=MAXB)
    try:
        models.build_resnet50(hb, w, -1, 64, SMALL_STAGES, 16, 100)
        s = hb.session(True)
        try:
            for bs in (1, MAXB, 4, 1):
                announce("dynamic batch resnet builder %s batch %d" % (mode, bs))
                feeds = models.resnet50_input(bs, 64, seed=40 + bs)
                s.set_batch(bs)
                got = s.run(feeds)
                want = run_ref(lambda b: models.build_resnet50(b, w, bs, 64, SMALL_STAGES, 16, 100), feeds)
                assert got["logits"].shape == (bs, 100)
                scale = max(1.0, float(np.max(np.abs(want["logits"]))))
                tol = 1e-4 if mode == "fp32" else 2e-2
                assert np.max(np.abs(got["logits"] - want["logits"])) <= tol * scale, bs
                if mode == "fp16":
                    assert np.array_equal(np.argmax(got["logits"], 1), np.argmax(want["logits"], 1))
        finally:
            s.close()
    finally:
        hb.destroy()


def test_bert_builder_recorded_with_a_dynamic_batch():
    pkg = entry.load()
    odla, mb = pkg.odla, pkg.models_bert
    cfg = dict(layers=2, hidden=96, heads=3, ffn=192, vocab=120, max_pos=64)
    w = mb.bert_weights(cfg, seed=31)
    MAXB, seq = 5, 33
    for mode in ("fp32", "bf16"):
        hb = odla.HipBuilder(bf16=(mode == "bf16"), max_batch=MAXB)
        try:
            mb.build_bert(hb, w, -1, seq, cfg)
            s = hb.session(True)
            try:
                for bs in (2, MAXB, 1):
                    announce("dynamic batch bert builder %s batch %d" % (mode, bs))
                    feeds = mb.bert_input(bs, seq, cfg, seed=50 + bs)
                    feeds["attention_mask"][0, 0, 0, seq - 9:] = 0.0
                    s.set_batch(bs)
                    got = s.run(feeds)["hidden"]
                    want = run_ref(lambda b: mb.build_bert(b, w, bs, seq, cfg), feeds)["hidden"]
                    assert got.shape == want.shape
                    if mode == "fp32":
                        assert max_rel_err(got, want) <= 2e-4, bs
                    else:
                        assert np.max(np.abs(got - want)) <= 3e-2 * max(1.0, float(np.max(np.abs(want)))), bs
            finally:
                s.close()
        finally:
            hb.destroy()


def test_many_batch_sizes_keep_device_memory_bounded():
    """A server that sweeps the batch must not pile up one planned copy of the weights
    per batch: a context keeps at most four batches planned (ODLA_HIP_MAX_BATCH_VARIANTS),
    the one used longest ago goes first, and a batch that was dropped runs again -
    rebuilt - with the same result.  The weights here are 16 MiB; 31 copies would be
    about 500 MiB."""
    odla = entry.load().odla
    r = np.random.default_rng(21)
    wf = (r.standard_normal((2048, 2048)) * 0.02).astype(np.float32)
    MAXB = 32

    def graph(batch):
        def build(b):
            x = b.arg("x", (batch, 2048))
            b.output(b.relu(b.gemm(x, b.const("wf", wf), name="fc"), name="y"), "y")
        return build

    hb = odla.HipBuilder(max_batch=MAXB)
    try:
        graph(-1)(hb)
        s = hb.session(True)
        try:
            x = r.standard_normal((MAXB, 2048)).astype(np.float32)
            want = run_ref(graph(MAXB), {"x": x})["y"]
            first = {}
            used = []
            for sweep in range(2):
                for bs in range(1, MAXB + 1):
                    if bs % 8 == 1:
                        announce("batch sweep %d: batch %d" % (sweep, bs))
                    s.set_batch(bs)
                    got = s.run({"x": x[:bs]})["y"]
                    assert max_rel_err(got, want[:bs]) <= 1e-4, bs
                    if sweep == 0:
                        first[bs] = got
                    else:
                        assert np.array_equal(got, first[bs]), bs      # the rebuilt plan computes the same
                    used.append(odla.used_device_memory())
            growth = max(used) - used[4]    # from the point where the four slots are taken
            announce("device memory over 64 batch changes: %.1f MiB at the start, largest %.1f MiB"
                     % (used[4] / 2 ** 20, max(used) / 2 ** 20))
            assert growth <= 64 * 2 ** 20, growth
        finally:
            s.close()
    finally:
        hb.destroy()


def test_batches_below_the_smallest_are_refused():
    """ODLA_MIN_BATCH_SIZE bounds the run-time batch from below."""
    odla = entry.load().odla
    w = cnn_weights(9)
    hb = odla.HipBuilder(max_batch=8, min_batch=4)
    try:
        build_cnn(w, -1)(hb)
        s = hb.session(True)
        try:
            announce("dynamic batch: below ODLA_MIN_BATCH_SIZE")
            for bs in (1, 3):
                with pytest.raises(odla.OdlaError):
                    s.set_batch(bs)
            s.set_batch(4)
            x = np.random.default_rng(10).standard_normal((4, 3, 20, 20)).astype(np.float32)
            got = s.run({"x": x})
            want = run_ref(build_cnn(w, 4), {"x": x})
            assert np.max(np.abs(got["prob"] - want["prob"])) <= 1e-5
        finally:
            s.close()
    finally:
        hb.destroy()
