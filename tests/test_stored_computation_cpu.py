"""Stored computations (no GPU needed: nothing is compiled): a recorded graph is
written, read back, and written again - the two files must be identical, and
the loaded computation must describe the same arguments, outputs and values.
"""
import ctypes

import numpy as np
import pytest


def _record(odla, with_table=False):
    r = np.random.default_rng(5)
    w = (r.standard_normal((8, 3, 3, 3)) * 0.2).astype(np.float32)
    bias = r.standard_normal(8).astype(np.float32)
    fc = (r.standard_normal((8, 5)) * 0.3).astype(np.float32)
    idx = np.array([2, 0, 1], np.int32)
    table = None
    if with_table:
        table = odla.quant_table([("x", 0.02, 128, -2.5, 2.5, None), ("y", 0.05, 0, 0.0, 12.0, None),
                                  ("w", 1.0, 0, float(w.min()), float(w.max()),
                                   list(zip(w.reshape(8, -1).min(1).tolist(), w.reshape(8, -1).max(1).tolist())))])
    hb = odla.HipBuilder(fp16=not with_table, quant_table=table)
    x = hb.arg("x", (2, 3, 8, 8))
    y = hb.relu(hb.conv(x, hb.const("w", w), hb.const("b", bias), (1, 1), (1, 1, 1, 1), name="c"), name="y")
    g = hb.reshape(hb.reduce_mean(y, (2, 3), True, name="gap"), (2, 8), name="flat")
    logits = hb.gemm(g, hb.const("fc", fc), None, name="logits")
    hb.output(hb.softmax(logits, -1, name="prob"), "prob")
    hb.output(hb.gather(hb.transpose(logits, (1, 0), name="lt"), hb.const("idx", idx), 0, name="picked"), "picked")
    v, i = hb.topk(logits, 2, 1, names=("tv", "ti"))
    hb.output(i, "ti")
    return hb


@pytest.mark.parametrize("with_table", [False, True])
def test_store_load_store_is_identical(odla, tmp_path, with_table):
    L = odla.load_library()
    hb = _record(odla, with_table)
    p1, p2 = str(tmp_path / "a.odla"), str(tmp_path / "b.odla")
    loc1, k1 = odla.path_location(p1)
    assert L.odla_StoreComputation(loc1, hb.comp) == 0
    blob = open(p1, "rb").read()
    assert blob[:8] == b"ODLAHIP2" and len(blob) > 8 * 3 * 3 * 3 * 4

    comp2 = ctypes.c_void_p()
    assert L.odla_LoadComputation(loc1, ctypes.byref(comp2)) == 0
    try:
        loc2, k2 = odla.path_location(p2)
        assert L.odla_StoreComputation(loc2, comp2) == 0
        assert open(p2, "rb").read() == blob
        n = ctypes.c_uint32()
        assert L.odla_GetNumOfArgsFromComputation(comp2, ctypes.byref(n)) == 0 and n.value == 1
        assert L.odla_GetNumOfOutputsFromComputation(comp2, ctypes.byref(n)) == 0 and n.value == 3
        v = ctypes.c_void_p()
        assert L.odla_GetOutputFromComputationByIdx(comp2, 2, ctypes.byref(v)) == 0
        t = odla.ValueType()
        assert L.odla_GetValueType(v, ctypes.byref(t)) == 0
        assert t.element_type == odla.ODLA_INT32 and [t.shape.dims[i] for i in range(t.shape.size)] == [2, 2]
        vid = ctypes.c_char_p()
        assert L.odla_GetValueId(v, ctypes.byref(vid)) == 0 and vid.value == b"ti"
        # the loaded computation is the current one: look-ups by id work
        assert L.odla_FindValueById(b"prob", ctypes.byref(v)) == 0 and v.value
    finally:
        L.odla_DestroyComputation(comp2)
        hb.destroy()


def test_load_from_memory_and_reject_garbage(odla, tmp_path):
    L = odla.load_library()
    hb = _record(odla)
    p = str(tmp_path / "a.odla")
    loc, keep = odla.path_location(p)
    assert L.odla_StoreComputation(loc, hb.comp) == 0
    hb.destroy()
    blob = open(p, "rb").read()
    exe = ctypes.c_void_p()
    mloc, mk = odla.memory_location(blob)
    assert L.odla_LoadExecutable(mloc, None, ctypes.byref(exe)) == 0 and exe.value
    n = ctypes.c_uint32()
    assert L.odla_GetNumOfArgsFromExecutable(exe, ctypes.byref(n)) == 0 and n.value == 1
    assert L.odla_GetNumOfOutputsFromExecutable(exe, ctypes.byref(n)) == 0 and n.value == 3
    assert L.odla_DestroyExecutable(exe) == 0
    for bad in (b"", b"ODLAHIP1", blob[:len(blob) // 2], b"X" + blob[1:], blob[:40] + b"\xff" * 64 + blob[104:]):
        comp = ctypes.c_void_p()
        bloc, bk = odla.memory_location(bad) if bad else (odla.ResourceLocation(odla.ODLA_LOCATION_MEMORY, None, 0), None)
        assert L.odla_LoadComputation(bloc, ctypes.byref(comp)) != 0 and not comp.value
    missing, mk2 = odla.path_location(str(tmp_path / "nope.odla"))
    comp = ctypes.c_void_p()
    assert L.odla_LoadComputation(missing, ctypes.byref(comp)) != 0
    uri = odla.ResourceLocation(odla.ODLA_LOCATION_URI, ctypes.cast(keep, ctypes.c_void_p), 0)
    assert L.odla_LoadComputation(uri, ctypes.byref(comp)) != 0
