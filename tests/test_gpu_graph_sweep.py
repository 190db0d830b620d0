"""Random operator chains against the oracle: convolutions with per-channel constant
arithmetic, activations, BatchNorm, shortcuts, pooling, concat, resize and channel
slices in random order, with random intermediate values marked as outputs (which
forbids folding them away).  This is aimed at the planner - epilogue fusion, layout
choices, aliasing and the arena - rather than at any one kernel."""
import numpy as np
import pytest

from util import announce, max_rel_err, run_hip, run_hip_stored, run_ref, run_ref_emulated

pytestmark = pytest.mark.gpu

# ODLA_SWEEP_SEED=<n> shifts every seed below: other random cases, same code (default 0)
SEED0 = int(__import__("os").environ.get("ODLA_SWEEP_SEED", "0"))


class Chain:
    """A recorded random program: a list of steps replayed on any builder."""

    def __init__(self, seed):
        r = np.random.default_rng(seed)
        self.in_shape = (int(r.integers(1, 4)), int(r.choice([3, 8, 16, 32])), int(r.integers(8, 17)), int(r.integers(8, 17)))
        self.steps = []
        shapes = [self.in_shape]          # shape of value k
        n_steps = int(r.integers(4, 13))
        for _ in range(n_steps):
            src = int(r.integers(max(0, len(shapes) - 3), len(shapes)))
            N, C, H, W = shapes[src]
            kind = str(r.choice(["conv", "conv", "conv", "chan_arith", "chan_arith", "act", "bn", "shortcut", "pool",
                                 "concat", "resize", "slice"]))
            if kind == "conv":
                k = int(r.choice([1, 1, 3, 3, 5]))
                s = int(r.choice([1, 1, 1, 2]))
                p = k // 2 if r.random() < 0.8 else 0
                O = int(r.choice([8, 16, 24, 64, 72, 136]))
                if (H + 2 * p - k) // s + 1 < 2 or (W + 2 * p - k) // s + 1 < 2:
                    continue
                w = (r.standard_normal((O, C, k, k)) * np.sqrt(1.5 / (C * k * k))).astype(np.float32)
                b = r.standard_normal(O).astype(np.float32) * 0.3 if r.random() < 0.6 else None
                self.steps.append(("conv", src, w, b, s, p))
                shapes.append((N, O, (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1))
            elif kind == "chan_arith":
                op = str(r.choice(["add", "mul", "sub", "div"]))
                form = str(r.choice(["c11", "1c11", "scalar"]))
                shape = {"c11": (C, 1, 1), "1c11": (1, C, 1, 1), "scalar": (1,)}[form]
                k = r.standard_normal(shape).astype(np.float32)
                if op in ("mul", "div"):
                    k = (np.abs(k) * 0.5 + 0.5).astype(np.float32)
                self.steps.append(("chan_arith", src, op, k, bool(r.random() < 0.2)))
                shapes.append((N, C, H, W))
            elif kind == "act":
                self.steps.append(("act", src, str(r.choice(["relu", "leaky", "clamp", "sigmoid", "tanh", "gelu"]))))
                shapes.append((N, C, H, W))
            elif kind == "bn":
                self.steps.append(("bn", src, r.standard_normal(C).astype(np.float32) * 0.2,
                                   (r.random(C) + 0.5).astype(np.float32), (r.random(C) + 0.5).astype(np.float32),
                                   r.standard_normal(C).astype(np.float32) * 0.2))
                shapes.append((N, C, H, W))
            elif kind == "shortcut":
                same = [i for i, sh in enumerate(shapes) if sh == shapes[src] and i != src]
                if not same:
                    continue
                self.steps.append(("shortcut", src, int(r.choice(same)), bool(r.random() < 0.5)))
                shapes.append((N, C, H, W))
            elif kind == "pool":
                if H < 4 or W < 4:
                    continue
                mx = bool(r.random() < 0.5)
                k, s, p = (3, 2, 1) if r.random() < 0.5 else (2, 2, 0)
                self.steps.append(("pool", src, mx, k, s, p))
                shapes.append((N, C, (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1))
            elif kind == "concat":
                same = [i for i, sh in enumerate(shapes) if sh[0] == N and sh[2:] == (H, W) and i != src]
                if not same:
                    continue
                other = int(r.choice(same))
                self.steps.append(("concat", src, other))
                shapes.append((N, C + shapes[other][1], H, W))
            elif kind == "resize":
                if H * W > 400:
                    continue
                self.steps.append(("resize", src))
                shapes.append((N, C, 2 * H, 2 * W))
            else:
                if C < 4:
                    continue
                c0 = int(r.integers(0, C // 2))
                c1 = int(r.integers(c0 + 1, C + 1))
                self.steps.append(("slice", src, c0, c1))
                shapes.append((N, c1 - c0, H, W))
        self.shapes = shapes
        n_vals = len(shapes)
        marks = set(int(v) for v in r.choice(np.arange(1, n_vals), size=min(n_vals - 1, int(r.integers(1, 4))), replace=False)) if n_vals > 1 else set()
        marks.add(n_vals - 1)
        self.outputs = sorted(marks)
        self.x = r.standard_normal(self.in_shape).astype(np.float32)

    def build(self, b, probe=None, batch=None, rows=None):
        """batch: leading extent given to the argument (-1 records a dynamic batch);
        rows: the batch the slices span (the largest batch of a dynamic recording)."""
        vals = [b.arg("x", self.in_shape if batch is None else (batch,) + self.in_shape[1:])]
        rows = rows or (self.in_shape[0] if batch is None else batch)
        for i, st in enumerate(self.steps):
            name = "v%d" % (i + 1)
            kind, src = st[0], vals[st[1]]
            if kind == "conv":
                _, _, w, bias, s, p = st
                v = b.conv(src, b.const(name + ".w", w), b.const(name + ".b", bias) if bias is not None else None,
                           (s, s), (p, p, p, p), name=name)
            elif kind == "chan_arith":
                _, _, op, k, swap = st
                kc = b.const(name + ".k", k)
                v = getattr(b, op)(kc, src, name=name) if swap and op in ("add", "mul") else getattr(b, op)(src, kc, name=name)
            elif kind == "act":
                a = st[2]
                v = {"relu": lambda: b.relu(src, name=name), "leaky": lambda: b.leaky_relu(src, 0.1, name=name),
                     "clamp": lambda: b.clamp(src, -1.0, 1.5, name=name), "sigmoid": lambda: b.sigmoid(src, name=name),
                     "tanh": lambda: b.tanh(src, name=name), "gelu": lambda: b.gelu(src, name=name)}[a]()
            elif kind == "bn":
                _, _, mean, var, g, be = st
                v = b.batchnorm(src, b.const(name + ".m", mean), b.const(name + ".v", var), 1e-5,
                                b.const(name + ".g", g), b.const(name + ".be", be), name=name)
            elif kind == "shortcut":
                v = b.add(src, vals[st[2]], name=name + (".s" if st[3] else ""))
                if st[3]:
                    v = b.relu(v, name=name)
            elif kind == "pool":
                _, _, mx, k, s, p = st
                v = (b.maxpool if mx else b.avgpool)(src, (k, k), (s, s), (p, p, p, p), name=name)
            elif kind == "concat":
                v = b.concat([src, vals[st[2]]], 1, name=name)
            elif kind == "resize":
                sh = self.shapes[st[1]]
                v = b.resize_nearest(src, (2 * sh[2], 2 * sh[3]), name=name)
            else:
                sh = self.shapes[st[1]]
                v = b.slice(src, (0, st[2], 0, 0), (rows, st[3], sh[2], sh[3]), name=name)
            vals.append(v)
            if probe is not None:
                probe(len(vals) - 1, v)
        for k in self.outputs:
            b.output(vals[k], "v%d" % k)


def _mode_kwargs(mode):
    return {"fp32": {}, "fp16": {"fp16": True}, "bf16acc": {"bf16": "accuracy"}}[mode]


@pytest.mark.parametrize("mode", ["fp32", "fp16", "bf16acc"])
def test_random_chains(mode, tmp_path):
    """bf16acc: BF16_ACCURACY_MODE (values fp32, Conv operands bf16) against the oracle that
    rounds exactly those operands - what is left are roundings that fell the other way."""
    kw = _mode_kwargs(mode)
    for seed in range(200):
        ch = Chain(SEED0 + seed)
        if not ch.steps:
            continue
        announce("chain %s seed %d: %s -> outputs %s" % (mode, seed, [s[0] for s in ch.steps], ch.outputs))
        feeds = {"x": ch.x}
        want = run_ref_emulated(ch.build, feeds, "operands", "bf16") if mode == "bf16acc" else run_ref(ch.build, feeds)
        got = run_hip(ch.build, feeds, repeats=2, **kw)
        if seed % 4 == 0:
            # the same program stored to a file and loaded back computes the same bits
            again = run_hip_stored(ch.build, feeds, str(tmp_path / ("chain%d.odla" % seed)), **kw)
            for k in got:
                assert np.array_equal(again[k], got[k]), (seed, k, "stored")
        for k, w in want.items():
            assert got[k].shape == w.shape, (seed, k)
            if mode == "fp32":
                assert max_rel_err(got[k], w) <= 5e-4, (seed, k, [s[0] for s in ch.steps])
            else:
                scale = max(1.0, float(np.max(np.abs(w))))
                tol = 6e-2 if mode == "fp16" else 1e-2
                assert float(np.max(np.abs(got[k] - w))) <= tol * scale, (seed, k, [s[0] for s in ch.steps])


@pytest.mark.parametrize("mode", ["fp32", "fp16"])
def test_random_chains_recorded_with_a_dynamic_batch(mode):
    """The same programs recorded once with a batch of -1 and a largest batch above
    the chain's own, run at the chain's batch, at the largest one and at the chain's
    batch again: every batch is planned from a rescaled copy of the recording."""
    import __graft_entry__ as entry
    odla = entry.load().odla
    for seed in range(1, 200, 3):
        ch = Chain(SEED0 + seed)
        if not ch.steps:
            continue
        n = ch.in_shape[0]
        big = n + 1 + seed % 3
        announce("dynamic-batch chain %s seed %d: %s, batch %d of %d" % (mode, seed, [s[0] for s in ch.steps], n, big))
        r = np.random.default_rng(SEED0 + 9000 + seed)
        xs = {n: ch.x, big: r.standard_normal((big,) + ch.in_shape[1:]).astype(np.float32)}
        want = {k: run_ref(lambda b: ch.build(b, batch=k), {"x": x}) for k, x in xs.items()}
        hb = odla.HipBuilder(fp16=(mode == "fp16"), max_batch=big)
        try:
            ch.build(hb, batch=-1, rows=big)
            sess = hb.session(True)
            try:
                for k in (n, big, n):
                    sess.set_batch(k)
                    got = sess.run({"x": xs[k]})
                    for name, w in want[k].items():
                        assert got[name].shape == w.shape, (seed, k, name)
                        if mode == "fp32":
                            assert max_rel_err(got[name], w) <= 5e-4, (seed, k, name)
                        else:
                            scale = max(1.0, float(np.max(np.abs(w))))
                            assert float(np.max(np.abs(got[name] - w))) <= 6e-2 * scale, (seed, k, name)
            finally:
                sess.close()
        finally:
            hb.destroy()


def test_random_chains_in_interpret_mode():
    """The same programs recorded in interpret mode: the input is a value with data of
    its own, random values are read back with odla_GetValueData while the graph still
    grows (each read compiles what exists so far), and again, in another order, once it
    is complete."""
    import ctypes
    import __graft_entry__ as entry
    odla = entry.load().odla

    class Interp(odla.HipBuilder):
        def __init__(self, feeds):
            super().__init__()
            self.feeds, self.held = feeds, []

        def arg(self, name, shape, dtype=np.float32):
            a = np.ascontiguousarray(self.feeds[name], dtype=dtype)
            self.held.append(a)
            h = self._ret(self.L.odla_CreateValue(odla.make_type(dtype, shape), name.encode()), "odla_CreateValue")
            assert self.L.odla_SetValueData(h, a.ctypes.data_as(ctypes.c_void_p)) == 0
            return h

        def output(self, v, name):
            pass

        def read(self, v):
            shape, dt = self.shape_of(v)
            out = np.empty(shape, dt)
            assert self.L.odla_GetValueData(v, out.ctypes.data_as(ctypes.c_void_p), None) == 0
            return out

    r = np.random.default_rng(SEED0 + 5)
    for seed in range(0, 200, 5):
        ch = Chain(SEED0 + seed)
        if not ch.steps:
            continue
        announce("interpret chain seed %d: %s" % (seed, [s[0] for s in ch.steps]))
        feeds = {"x": ch.x}
        ref = run_ref(lambda b: ch.build(b, probe=lambda k, v: b.output(v, "p%d" % k)), feeds)
        ib = Interp(feeds)
        try:
            handles = {}

            def probe(k, v):
                handles[k] = v
                if r.random() < 0.4:
                    got = ib.read(v)
                    assert max_rel_err(got, ref["p%d" % k]) <= 5e-4, (seed, k, "while growing")

            ch.build(ib, probe=probe)
            for k in r.permutation(sorted(handles)):
                got = ib.read(handles[int(k)])
                assert max_rel_err(got, ref["p%d" % int(k)]) <= 5e-4, (seed, int(k), "complete")
        finally:
            ib.destroy()


def test_random_chains_under_the_calibration_profiler(tmp_path):
    """Profiler mode over random programs: the recorded range of every named value -
    whole tensor and per channel - equals the range of the oracle's value."""
    import __graft_entry__ as entry
    pkg = entry.load()
    cal, odla = pkg.calibration, pkg.odla
    for seed in range(2, 200, 9):
        ch = Chain(SEED0 + seed)
        if not ch.steps:
            continue
        announce("profiled chain seed %d: %s" % (seed, [s[0] for s in ch.steps]))
        feeds = {"x": ch.x}
        ref = run_ref(lambda b: ch.build(b, probe=lambda k, v: b.output(v, "p%d" % k)), feeds)
        prof_path = str(tmp_path / ("chain%d.prof" % seed))
        with cal.Profiler(prof_path, channel_axis=1) as p:
            hb = odla.HipBuilder()
            try:
                ch.build(hb)
                s = hb.session()
                try:
                    with p.run("only"):
                        s.run(feeds)
                finally:
                    s.close()
            finally:
                hb.destroy()
        rec = cal.load_profile(prof_path)["ProfilingResults"]["only"]
        n_checked = 0
        for k in range(1, len(ch.steps) + 1):
            name, want = "v%d" % k, ref["p%d" % k]
            if name not in rec:
                continue
            scale = max(float(np.max(np.abs(want))), 1e-6)
            assert abs(rec[name]["min_value"] - float(want.min())) <= 5e-4 * scale, (seed, name)
            assert abs(rec[name]["max_value"] - float(want.max())) <= 5e-4 * scale, (seed, name)
            assert rec[name]["shape"] == list(want.shape), (seed, name)
            if "channels_max" in rec[name] and rec[name].get("channels") == want.shape[1]:
                assert np.allclose(rec[name]["channels_max"], want.max(axis=(0, 2, 3)), rtol=0, atol=5e-4 * scale), (seed, name)
                assert np.allclose(rec[name]["channels_min"], want.min(axis=(0, 2, 3)), rtol=0, atol=5e-4 * scale), (seed, name)
            n_checked += 1
        assert n_checked == len(ch.steps), (seed, sorted(rec))
