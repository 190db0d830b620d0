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


def run_hip_stored(build_fn, feeds, path, **builder_kwargs):
    """Record, store the computation to `path`, destroy it, load the file as an
    executable and run that: name -> numpy array like run_hip."""
    import ctypes
    pkg = entry.load()
    odla = pkg.odla
    L = odla.load_library()
    hb = odla.HipBuilder(**builder_kwargs)
    try:
        build_fn(hb)
        outs = {name: (shape, dt) for name, (h, shape, dt) in hb.outs.items()}
        args = {name: (shape, dt) for name, (h, shape, dt) in hb.args.items()}
        loc, keep = odla.path_location(path)
        exe0 = ctypes.c_void_p()
        assert L.odla_CompileComputation(hb.comp, None, ctypes.byref(exe0)) == 0 and exe0.value
        assert L.odla_StoreExecutable(loc, exe0) == 0
    finally:
        hb.destroy()
    exe = ctypes.c_void_p()
    assert L.odla_LoadExecutable(loc, None, ctypes.byref(exe)) == 0
    ctx = ctypes.c_void_p()
    assert L.odla_CreateContext(ctypes.byref(ctx)) == 0
    try:
        held = []
        n = ctypes.c_uint32()
        assert L.odla_GetNumOfArgsFromExecutable(exe, ctypes.byref(n)) == 0 and n.value == len(args)
        for i in range(n.value):
            v = ctypes.c_void_p()
            assert L.odla_GetArgFromExecutableByIdx(exe, i, ctypes.byref(v)) == 0
            vid = ctypes.c_char_p()
            assert L.odla_GetValueId(v, ctypes.byref(vid)) == 0
            name = vid.value.decode()
            a = np.ascontiguousarray(feeds[name], dtype=args[name][1])
            held.append(a)
            assert L.odla_BindToArgument(v, a.ctypes.data_as(ctypes.c_void_p), ctx) == 0
        assert L.odla_GetNumOfOutputsFromExecutable(exe, ctypes.byref(n)) == 0 and n.value == len(outs)
        got = {}
        for i in range(n.value):
            v = ctypes.c_void_p()
            assert L.odla_GetOutputFromExecutableByIdx(exe, i, ctypes.byref(v)) == 0
            vid = ctypes.c_char_p()
            assert L.odla_GetValueId(v, ctypes.byref(vid)) == 0
            name = vid.value.decode()
            got[name] = np.empty(outs[name][0], outs[name][1])
            assert L.odla_BindToOutput(v, got[name].ctypes.data_as(ctypes.c_void_p), ctx) == 0
        assert L.odla_LaunchExecutable(exe, ctx) == 0
        return got
    finally:
        L.odla_DestroyContext(ctx)
        assert L.odla_DestroyExecutable(exe) == 0


def run_ref(build_fn, feeds):
    ref = entry.load_oracle()
    rb = ref.RefBuilder(feeds)
    build_fn(rb)
    return rb.outputs


def run_ref_emulated(build_fn, feeds, emulate, storage):
    """The oracle with values rounded to a 16-bit storage type: emulate = "operands"
    (Conv / Gemm operands only) or "stored" (every tensor a 16-bit plan stores)."""
    ref = entry.load_oracle()
    rb = ref.RefBuilder(feeds, emulate=emulate, storage=storage)
    build_fn(rb)
    return rb.outputs


def err_stats(got, want):
    """(max, 99.9th percentile, mean) of |got - want|."""
    d = np.abs(np.asarray(got, np.float64) - np.asarray(want, np.float64))
    return float(d.max()), float(np.quantile(d, 0.999)), float(d.mean())


def run_both(build_fn, feeds, **kw):
    return run_hip(build_fn, feeds, **kw), run_ref(build_fn, feeds)


REL_ERR_FLOOR = 0.05


def max_rel_err(got, want, floor=REL_ERR_FLOOR):
    """Largest element-wise relative error  |got - want| / max(|want|, floor * max|want|).
    Elements smaller than `floor` x the tensor's largest magnitude are measured against that
    magnitude instead of their own: they are sums that cancel, and a sum that cancels has no
    relative accuracy of its own in any summation order (its absolute error is that of its
    terms, which are of the tensor's scale)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    scale = max(float(np.max(np.abs(want))) if want.size else 0.0, 1e-30)
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), floor * scale))) if want.size else 0.0


def announce(msg):
    """Name the case before touching the GPU so that a fault can be attributed."""
    print(msg, flush=True)
    sys.stdout.flush()
