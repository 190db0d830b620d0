"""Several threads, each with a context of its own over one computation, bind and
execute at the same time - the use the reference tests in
ODLA/platforms/odla_popart/test/odla_compute_test.cc:186-204 (contexts made, bound
and destroyed inside std::threads) and utils.cc:72-82 (execute inside threads).
ctypes drops the interpreter lock during a call, so the library calls overlap."""
import threading

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, run_ref

pytestmark = pytest.mark.gpu


def build_net(w):
    def build(b):
        x = b.arg("x", (4, 16, 12, 12))
        c1 = b.relu(b.conv(x, b.const("w1", w["w1"]), b.const("b1", w["b1"]), (1, 1), (1, 1, 1, 1), name="c1"), name="r1")
        c2 = b.conv(c1, b.const("w2", w["w2"]), None, (2, 2), (0, 0, 0, 0), name="c2")
        p = b.reduce_mean(c2, (2, 3), True, name="gap")
        f = b.reshape(p, (4, 160), name="flat")
        y = b.softmax(b.gemm(f, b.const("w3", w["w3"]), b.const("b3", w["b3"]), name="fc"), -1, name="prob")
        b.output(c2, "c2")
        b.output(y, "prob")
    return build


@pytest.mark.parametrize("use_graph", [True, False])
def test_contexts_of_one_computation_execute_from_threads(use_graph):
    announce("threads, graph=%s" % use_graph)
    odla = entry.load().odla
    r = np.random.default_rng(21)
    w = {"w1": (r.standard_normal((32, 16, 3, 3)) * 0.1).astype(np.float32),
         "b1": r.standard_normal(32).astype(np.float32),
         "w2": (r.standard_normal((160, 32, 2, 2)) * 0.1).astype(np.float32),
         "w3": (r.standard_normal((160, 10)) * 0.2).astype(np.float32),
         "b3": r.standard_normal((1, 10)).astype(np.float32)}
    build = build_net(w)
    n_threads, rounds = 6, 8
    inputs = [[r.standard_normal((4, 16, 12, 12)).astype(np.float32) for _ in range(rounds)] for _ in range(n_threads)]

    hb = odla.HipBuilder()
    try:
        build(hb)
        # one serial pass first: the expected results of every (thread, round) pair
        s0 = hb.session(use_graph)
        want = [[{k: v.copy() for k, v in s0.run({"x": x}).items()} for x in xs] for xs in inputs]
        s0.close()
        ref = run_ref(build, {"x": inputs[0][0]})
        assert np.allclose(want[0][0]["prob"], ref["prob"], rtol=1e-4, atol=1e-6)

        errors = []
        start = threading.Barrier(n_threads)

        def worker(t):
            try:
                s = hb.session(use_graph)       # odla_CreateContext inside the thread
                try:
                    start.wait()
                    for k in range(rounds):
                        got = s.run({"x": inputs[t][k]})
                        for name in ("c2", "prob"):
                            if not np.array_equal(got[name], want[t][k][name]):
                                errors.append((t, k, name))
                finally:
                    s.close()
            except Exception as e:  # noqa: BLE001 - reported through the list
                errors.append((t, repr(e)))

        threads = [threading.Thread(target=worker, args=(t,)) for t in range(n_threads)]
        for th in threads:
            th.start()
        for th in threads:
            th.join(120)
        assert not any(th.is_alive() for th in threads)
        assert errors == []
    finally:
        hb.destroy()
