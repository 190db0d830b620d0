"""Interpret mode through the C ABI: values with their own data
(odla_CreateValue / odla_SetValueData), operators recorded one by one, results
read back with odla_GetValueData(value, ptr, NULL) - the calling sequence of the
reference's interpreter build (ODLA/platforms/dnnl/odla_dnnl.cc:74-82,161-179,
225-230,276-295 of the reference tree) - against the CPU oracle.
"""
import ctypes

import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, max_rel_err

pytestmark = pytest.mark.gpu


def _vp(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def test_interpret_mode_grows_and_reevaluates(odla, ref):
    announce("interpret mode")
    L = odla.load_library()
    comp = ctypes.c_void_p()
    assert L.odla_CreateComputation(ctypes.byref(comp)) == 0
    try:
        r = np.random.default_rng(7)
        x = r.standard_normal((4, 8, 6, 6)).astype(np.float32)
        w = (r.standard_normal((16, 8, 3, 3)) * 0.2).astype(np.float32)
        vx = L.odla_CreateValue(odla.make_type(np.float32, x.shape), b"x")
        assert vx and L.odla_SetValueData(vx, _vp(x)) == 0
        vw = L.odla_CreateConstant(odla.make_type(np.float32, w.shape), _vp(w), b"w")
        one = (ctypes.c_uint32 * 2)(1, 1)
        y = L.odla_Conv(vx, odla.ODLA_CHANNELS_FIRST, 1, vw, odla.ODLA_OIS, one, one, one, one, None,
                        odla.undefined_shape(), b"y")
        assert y
        got = np.empty((4, 16, 6, 6), np.float32)
        assert L.odla_GetValueData(y, _vp(got), None) == 0
        want = ref.conv2d(x, w, None, (1, 1), (1, 1, 1, 1))
        assert max_rel_err(got, want) <= 1e-4

        # the graph grows: a later value is asked for, the earlier one stays available
        z = L.odla_Relu(y, b"z")
        s = L.odla_Sigmoid(z, b"s")
        got_s = np.empty_like(got)
        assert L.odla_GetValueDataById(b"s", _vp(got_s)) == 0
        want_s = 1.0 / (1.0 + np.exp(-np.maximum(want.astype(np.float64), 0)))
        assert max_rel_err(got_s, want_s) <= 1e-4
        got_y = np.empty_like(got)
        assert L.odla_GetValueData(y, _vp(got_y), None) == 0
        assert np.array_equal(got_y, got)

        # new data behind a new pointer: no recompilation needed, results follow the data
        x2 = r.standard_normal(x.shape).astype(np.float32)
        assert L.odla_SetValueDataById(b"x", _vp(x2)) == 0
        assert L.odla_GetValueData(s, _vp(got_s), None) == 0
        want2 = ref.conv2d(x2, w, None, (1, 1), (1, 1, 1, 1))
        assert max_rel_err(got_s, 1.0 / (1.0 + np.exp(-np.maximum(want2.astype(np.float64), 0)))) <= 1e-4
        assert L.odla_ReleaseValue(z) == 0

        # a value without data cannot be evaluated
        v2 = L.odla_CreateValue(odla.make_type(np.float32, (3,)), b"nodata")
        t = L.odla_Relu(v2, b"t")
        out = np.empty(3, np.float32)
        assert L.odla_GetValueData(t, _vp(out), None) != 0
        # data can only be attached to values made by odla_CreateValue
        arg = L.odla_CreateArgument(odla.make_type(np.float32, (3,)), b"arg")
        assert L.odla_SetValueData(arg, _vp(out)) != 0
    finally:
        L.odla_DestroyComputation(comp)
