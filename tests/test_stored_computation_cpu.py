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
    # operators along an axis (recorded, not marked as outputs: the counts above stay)
    hm = hb.hardmax(logits, -1, name="hm")
    cs = hb.cumsum(hm, 1, exclusive=True, name="cs")
    ge = hb.gather_elements(cs, hb.const("gi", np.array([[0, 4, 1], [2, 3, 3]], np.int64)), 1, name="ge")
    hb.compress(ge, hb.const("cc", np.array([1, 0, 1], np.bool_)), 1, (2, 3), name="cp")
    return hb


@pytest.mark.parametrize("with_table", [False, True])
def test_store_load_store_is_identical(odla, tmp_path, with_table):
    L = odla.load_library()
    hb = _record(odla, with_table)
    p1, p2 = str(tmp_path / "a.odla"), str(tmp_path / "b.odla")
    loc1, k1 = odla.path_location(p1)
    assert L.odla_StoreComputation(loc1, hb.comp) == 0
    blob = open(p1, "rb").read()
    assert blob[:8] == b"ODLAHIP3" and len(blob) > 8 * 3 * 3 * 3 * 4

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
    for bad in (b"", b"ODLAHIP1", b"ODLAHIP2" + blob[8:], blob[:len(blob) // 2], b"X" + blob[1:],
                blob[:40] + b"\xff" * 64 + blob[104:], blob[:-1], blob + b"\0"):
        comp = ctypes.c_void_p()
        bloc, bk = odla.memory_location(bad) if bad else (odla.ResourceLocation(odla.ODLA_LOCATION_MEMORY, None, 0), None)
        assert L.odla_LoadComputation(bloc, ctypes.byref(comp)) != 0 and not comp.value
    missing, mk2 = odla.path_location(str(tmp_path / "nope.odla"))
    comp = ctypes.c_void_p()
    assert L.odla_LoadComputation(missing, ctypes.byref(comp)) != 0
    uri = odla.ResourceLocation(odla.ODLA_LOCATION_URI, ctypes.cast(keep, ctypes.c_void_p), 0)
    assert L.odla_LoadComputation(uri, ctypes.byref(comp)) != 0


# ---------------------------------------------------------------------------
# Files that pass the integrity hash but hold records the planner could not
# index safely: every one of them must be refused with ODLA_INVALID_PARAM when
# it is loaded, not crash later when a context is created.

def _fnv1a(data):
    h = 1469598103934665603
    for b in data:
        h = ((h ^ b) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


class _Stored:
    """Offsets of the records of a stored computation (the layout serialize.cc writes)."""

    def __init__(self, blob):
        import struct
        self.buf = bytearray(blob[:-8])
        self.pos = 8 + 8 * 8
        i64 = lambda: self._i64()
        nq = i64()
        for _ in range(nq):
            self.pos += 8 + self._peek_len()      # name
            self.pos += 8 + 4 * 4
        self.values = []                           # per value: offsets of kind, etype, rank, dims
        nv = i64()
        for _ in range(nv):
            o = {"kind": self.pos, "etype": self.pos + 8, "rank": self.pos + 16, "dims": self.pos + 24}
            kind = i64(); i64(); rank = i64()
            self.pos += 8 * rank
            self.pos += 8 + self._peek_len()
            o["producer"] = self.pos + 16
            self.pos += 8 * 4
            if kind == 1:
                nbytes = i64()
                self.pos += nbytes
            self.values.append(o)
        for _ in range(2):
            n = i64()
            self.pos += 8 * n
        self.nodes = []                            # per node: op, offsets of the operand list, results, attributes
        nn = i64()
        for _ in range(nn):
            o = {"op_at": self.pos}
            o["op"] = i64()
            o["nin_at"] = self.pos
            nin = i64()
            o["in_at"] = self.pos
            self.pos += 8 * nin
            o["out_at"], o["out2_at"] = self.pos, self.pos + 8
            self.pos += 16
            o["i_at"] = self.pos
            self.pos += 8 * 24 + 4 * 8
            o["niv_at"] = self.pos
            niv = i64()
            o["iv_at"] = self.pos
            self.pos += 8 * niv
            self.nodes.append(o)
        assert self.pos == len(self.buf)
        self.struct = struct

    def _peek_len(self):
        import struct
        return struct.unpack_from("<q", self.buf, self.pos)[0]

    def _i64(self):
        import struct
        v = struct.unpack_from("<q", self.buf, self.pos)[0]
        self.pos += 8
        return v

    def patched(self, at, value):
        b = bytearray(self.buf)
        self.struct.pack_into("<q", b, at, value)
        return bytes(b) + self.struct.pack("<Q", _fnv1a(b))

    def node(self, op):
        return next(n for n in self.nodes if n["op"] == op)


OP_CONV, OP_GEMM, OP_REDUCE, OP_SOFTMAX, OP_GATHER, OP_RESHAPE, OP_TRANSPOSE, OP_TOPK, OP_AXISOP = 0, 1, 7, 8, 11, 12, 15, 22, 26
AX_GATHER_ELEMENTS, AX_CUMSUM, AX_HARDMAX, AX_COMPRESS = range(4)


def test_well_hashed_files_with_malformed_records_are_refused(odla, tmp_path):
    L = odla.load_library()
    hb = _record(odla)
    p = str(tmp_path / "a.odla")
    loc, keep = odla.path_location(p)
    assert L.odla_StoreComputation(loc, hb.comp) == 0
    hb.destroy()
    blob = open(p, "rb").read()
    st = _Stored(blob)

    def load(data):
        comp = ctypes.c_void_p()
        mloc, mk = odla.memory_location(data)
        rc = L.odla_LoadComputation(mloc, ctypes.byref(comp))
        if rc == 0:
            L.odla_DestroyComputation(comp)
        return rc

    assert load(st.patched(8, 1)) == 0                       # the re-hashed, unchanged payload still loads
    conv, gemm, tr, topk = st.node(OP_CONV), st.node(OP_GEMM), st.node(OP_TRANSPOSE), st.node(OP_TOPK)
    axis_nodes = {st.struct.unpack_from("<q", st.buf, n["i_at"])[0]: n for n in st.nodes if n["op"] == OP_AXISOP}
    assert sorted(axis_nodes) == [AX_GATHER_ELEMENTS, AX_CUMSUM, AX_HARDMAX, AX_COMPRESS]
    arg_dims = st.values[0]["dims"]
    bad = {
        "extent 0": st.patched(arg_dims, 0),
        "negative extent": st.patched(arg_dims + 8, -3),
        "unknown element type": st.patched(st.values[0]["etype"], 99),
        "temporary without producer": st.patched(st.values[-1]["producer"], -1),
        "producer out of range": st.patched(st.values[-1]["producer"], 10 ** 6),
        "unknown operator": st.patched(conv["op_at"], 77),
        "conv without kernel": st.patched(conv["in_at"] + 8, -1),
        "conv with two operand slots": None,                 # changes record sizes: covered by the parse check below
        "conv stride 0": st.patched(conv["i_at"] + 8 * 3, 0),
        "conv group 0": st.patched(conv["i_at"] + 8 * 1, 0),
        "conv negative padding": st.patched(conv["i_at"] + 8 * 7, -1),
        "operand computed later": st.patched(conv["in_at"], st.struct.unpack_from("<q", st.buf, topk["out_at"])[0]),
        "result of another node": st.patched(gemm["out_at"], st.struct.unpack_from("<q", st.buf, conv["out_at"])[0]),
        "transpose: not a permutation": st.patched(tr["iv_at"], 0),
        "transpose: axis out of range": st.patched(tr["iv_at"], 5),
        "topk without its second result": st.patched(topk["out2_at"], -1),
        "topk: K beyond the extent": st.patched(topk["i_at"], 1000),
        "topk: axis out of range": st.patched(topk["i_at"] + 16, 7),
        "softmax: axis out of range": st.patched(st.node(OP_SOFTMAX)["i_at"], 9),
        "gather: axis out of range": st.patched(st.node(OP_GATHER)["i_at"], -4),
        "reduce: axis out of range": st.patched(st.node(OP_REDUCE)["iv_at"], 4),
        "axis operator: unknown kind": st.patched(axis_nodes[AX_CUMSUM]["i_at"], 9),
        "cumsum: axis out of range": st.patched(axis_nodes[AX_CUMSUM]["i_at"] + 8, 2),
        "hardmax: negative axis": st.patched(axis_nodes[AX_HARDMAX]["i_at"] + 8, -1),
        "gather elements without indices": st.patched(axis_nodes[AX_GATHER_ELEMENTS]["in_at"] + 8, -1),
        "compress: more conditions than the axis is long": st.patched(axis_nodes[AX_COMPRESS]["i_at"] + 16, 4),
        "compress: flat form with an axis": st.patched(axis_nodes[AX_COMPRESS]["i_at"] + 24, 1),
        "reshape changes the element count": st.patched(st.values[
            st.struct.unpack_from("<q", st.buf, st.node(OP_RESHAPE)["out_at"])[0]]["dims"], 3),
    }
    for what, data in bad.items():
        if data is not None:
            assert load(data) == odla.ODLA_INVALID_PARAM, what
    # an operand count that no longer matches the bytes that follow
    assert load(st.patched(conv["nin_at"], 2)) == odla.ODLA_INVALID_PARAM
    assert load(st.patched(tr["niv_at"], 1)) == odla.ODLA_INVALID_PARAM


def test_concat_with_a_missing_operand_beyond_slot_32_is_refused(odla, tmp_path):
    """A Concat may have up to 64 operands; every slot is required, also those beyond the 32
    the per-operator mask has a bit for (a well-hashed file with slot 32 empty used to pass
    validation and crash in the shape checks)."""
    L = odla.load_library()
    hb = odla.HipBuilder()
    x = hb.arg("x", (1, 2, 4))
    parts = [hb.relu(x, name="r%d" % i) for i in range(33)]
    hb.output(hb.concat(parts, 1, name="cat"), "cat")
    p = str(tmp_path / "cat.odla")
    loc, keep = odla.path_location(p)
    assert L.odla_StoreComputation(loc, hb.comp) == 0
    hb.destroy()
    st = _Stored(open(p, "rb").read())
    OP_CONCAT = 10
    cat = st.node(OP_CONCAT)

    def load(data):
        comp = ctypes.c_void_p()
        mloc, mk = odla.memory_location(data)
        rc = L.odla_LoadComputation(mloc, ctypes.byref(comp))
        if rc == 0:
            L.odla_DestroyComputation(comp)
        return rc

    assert load(st.patched(8, 1)) == 0
    assert load(st.patched(cat["in_at"] + 8 * 32, -1)) == odla.ODLA_INVALID_PARAM
    assert load(st.patched(cat["in_at"] + 8 * 5, -1)) == odla.ODLA_INVALID_PARAM
