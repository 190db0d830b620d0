"""A stored computation, loaded as an executable, computes bit for bit what the
recorded one does (fp16 plan and int8 plan with its quantisation table), driven
through the executable entry points of the C ABI.
"""
import ctypes

import numpy as np
import pytest

from test_stored_computation_cpu import _record
from util import announce

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("with_table", [False, True])
def test_loaded_executable_equals_recorded_computation(odla, tmp_path, with_table):
    announce("stored executable, %s plan" % ("int8" if with_table else "fp16"))
    L = odla.load_library()
    x = np.random.default_rng(9).standard_normal((2, 3, 8, 8)).astype(np.float32)
    hb = _record(odla, with_table)
    path = str(tmp_path / "model.odla")
    loc, keep = odla.path_location(path)
    exe0 = ctypes.c_void_p()
    assert L.odla_CompileComputation(hb.comp, None, ctypes.byref(exe0)) == 0 and exe0.value
    assert L.odla_StoreExecutable(loc, exe0) == 0
    s = hb.session()
    want = s.run({"x": x})
    s.close()
    assert L.odla_DestroyExecutable(exe0) == 0   # a compiled executable belongs to its computation
    hb.destroy()

    exe = ctypes.c_void_p()
    assert L.odla_LoadExecutable(loc, None, ctypes.byref(exe)) == 0
    ctx = ctypes.c_void_p()
    assert L.odla_CreateContext(ctypes.byref(ctx)) == 0
    try:
        arg = ctypes.c_void_p()
        assert L.odla_GetArgFromExecutableByIdx(exe, 0, ctypes.byref(arg)) == 0
        assert L.odla_BindToArgument(arg, x.ctypes.data_as(ctypes.c_void_p), ctx) == 0
        n = ctypes.c_uint32()
        assert L.odla_GetNumOfOutputsFromExecutable(exe, ctypes.byref(n)) == 0 and n.value == len(want)
        got = {}
        for i in range(n.value):
            v = ctypes.c_void_p()
            assert L.odla_GetOutputFromExecutableByIdx(exe, i, ctypes.byref(v)) == 0
            vid = ctypes.c_char_p()
            assert L.odla_GetValueId(v, ctypes.byref(vid)) == 0
            name = vid.value.decode()
            got[name] = np.empty_like(want[name])
            assert L.odla_BindToOutput(v, got[name].ctypes.data_as(ctypes.c_void_p), ctx) == 0
        assert L.odla_LaunchExecutable(exe, ctx) == 0
        for k in want:
            assert np.array_equal(got[k], want[k]), k
    finally:
        L.odla_DestroyContext(ctx)
        assert L.odla_DestroyExecutable(exe) == 0
