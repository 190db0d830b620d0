"""Shared helpers of the parity tests: run one graph description on the GPU
library (through the ODLA C ABI) and on the CPU oracle with the same feeds."""
import sys

import numpy as np

import __graft_entry__ as entry


def run_hip(build_fn, feeds, use_graph=True, repeats=1, **builder_kwargs):
    pkg = entry.load()
    hb = pkg.odla.HipBuilder(**builder_kwargs)
    try:
        build_fn(hb)
        s = hb.session(use_graph)
        try:
            out = None
            for _ in range(repeats):
                out = s.run(feeds)
            return out
        finally:
            s.close()
    finally:
        hb.destroy()


def run_ref(build_fn, feeds):
    ref = entry.load_oracle()
    rb = ref.RefBuilder(feeds)
    build_fn(rb)
    return rb.outputs


def run_both(build_fn, feeds, **kw):
    return run_hip(build_fn, feeds, **kw), run_ref(build_fn, feeds)


def max_rel_err(got, want):
    """Largest |got-want| relative to the largest magnitude of the expected tensor."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    scale = max(float(np.max(np.abs(want))), 1e-30)
    return float(np.max(np.abs(got - want))) / scale


def announce(msg):
    """Name the case before touching the GPU so that a fault can be attributed."""
    print(msg, flush=True)
    sys.stdout.flush()
