"""Readers for the weight containers a HALO-compiled model ships with, so that a
harness can hand real constants to ``odla_CreateConstant``:

  * the C source written by ``-emit-data-as-c``
    (``extern <type> const <name>[d0*d1*...] = {...};`` per constant,
    lib/target/generic_cpp/generic_cxx_constant_writer.cc:24-36 of the
    reference tree),
  * the relocatable ELF object ``<model>.bin`` (one data symbol per constant),
  * a frozen TensorFlow GraphDef (``Const`` nodes), read with a minimal
    protobuf wire-format parser - enough for
    models/vision/classification/mnist_simple/mnist_simple.pb.

Pure host code: nothing here touches the GPU.
"""
import re
import struct

import numpy as np

_C_TYPES = {
    "float": np.float32, "double": np.float64, "int8_t": np.int8, "uint8_t": np.uint8, "int16_t": np.int16,
    "uint16_t": np.uint16, "int32_t": np.int32, "uint32_t": np.uint32, "int64_t": np.int64, "uint64_t": np.uint64,
    "int": np.int32, "unsigned": np.uint32, "bool": np.bool_, "odla_float16": np.float16,
}


def read_c_arrays(text):
    """name -> ndarray for every ``extern T const name[dims] = {values};`` in `text`."""
    out = {}
    pat = re.compile(r"extern\s+(?:const\s+)?([A-Za-z_]\w*)\s+(?:const\s+)?([A-Za-z_]\w*)\s*\[([^\]]*)\]\s*=\s*\{([^}]*)\}\s*;")
    for m in pat.finditer(text):
        ctype, name, dims, body = m.groups()
        if ctype not in _C_TYPES:
            raise ValueError("constant %s has unsupported element type %s" % (name, ctype))
        dt = np.dtype(_C_TYPES[ctype])
        shape = tuple(int(d) for d in dims.split("*") if d.strip())
        toks = [t for t in body.replace("\n", " ").split(",") if t.strip()]
        if dt.kind == "f":
            vals = np.array([float(t.strip().rstrip("fF")) for t in toks], dtype=dt)
        elif dt.kind == "b":
            vals = np.array([t.strip() in ("1", "true") for t in toks], dtype=dt)
        else:
            vals = np.array([int(t.strip().rstrip("uUlL"), 0) for t in toks], dtype=dt)
        if shape and int(np.prod(shape)) != vals.size:
            raise ValueError("constant %s: %d values for shape %s" % (name, vals.size, shape))
        out[name] = vals.reshape(shape) if shape else vals
    return out


def read_elf_symbols(data):
    """name -> bytes of every sized data symbol of a little-endian ELF64 object."""
    if data[:4] != b"\x7fELF" or data[4] != 2 or data[5] != 1:
        raise ValueError("not a little-endian ELF64 file")
    e_shoff, = struct.unpack_from("<Q", data, 0x28)
    e_shentsize, e_shnum, _ = struct.unpack_from("<HHH", data, 0x3A)
    secs = []
    for i in range(e_shnum):
        name, typ, flags, addr, off, size, link, info, align, entsize = struct.unpack_from("<IIQQQQIIQQ", data, e_shoff + i * e_shentsize)
        secs.append(dict(type=typ, off=off, size=size, link=link, entsize=entsize))
    out = {}
    for s in secs:
        if s["type"] != 2:  # SHT_SYMTAB
            continue
        strtab = secs[s["link"]]
        for k in range(s["size"] // 24):
            st_name, st_info, _, st_shndx, st_value, st_size = struct.unpack_from("<IBBHQQ", data, s["off"] + k * 24)
            if (st_info & 0xF) != 1 or st_size == 0 or st_shndx == 0 or st_shndx >= len(secs):  # STT_OBJECT in a section
                continue
            end = data.index(b"\0", strtab["off"] + st_name)
            name = data[strtab["off"] + st_name:end].decode()
            sec = secs[st_shndx]
            if sec["type"] == 8:  # SHT_NOBITS: zero-initialised
                out[name] = bytes(st_size)
            else:
                out[name] = bytes(data[sec["off"] + st_value:sec["off"] + st_value + st_size])
    return out


# ---------------------------------------------------------------- protobuf --
def _varint(buf, pos):
    v, shift = 0, 0
    while True:
        b = buf[pos]
        pos += 1
        v |= (b & 0x7F) << shift
        if not b & 0x80:
            return v, pos
        shift += 7


def _fields(buf):
    """Yields (field number, wire type, value) of one protobuf message."""
    pos, n = 0, len(buf)
    while pos < n:
        key, pos = _varint(buf, pos)
        fn, wt = key >> 3, key & 7
        if wt == 0:
            v, pos = _varint(buf, pos)
        elif wt == 1:
            v = buf[pos:pos + 8]
            pos += 8
        elif wt == 2:
            ln, pos = _varint(buf, pos)
            v = buf[pos:pos + ln]
            pos += ln
        elif wt == 5:
            v = buf[pos:pos + 4]
            pos += 4
        else:
            raise ValueError("unsupported protobuf wire type %d" % wt)
        yield fn, wt, v


_TF_DTYPES = {1: np.float32, 2: np.float64, 3: np.int32, 4: np.uint8, 5: np.int16, 6: np.int8, 9: np.int64, 10: np.bool_}


def _tensor_proto(buf):
    dtype, shape, content, floats, ints = None, [], None, [], []
    for fn, wt, v in _fields(buf):
        if fn == 1:
            dtype = v
        elif fn == 2:  # TensorShapeProto { repeated Dim dim = 2 { int64 size = 1 } }
            for f2, _, d in _fields(v):
                if f2 == 2:
                    size = 0
                    for f3, _, s in _fields(d):
                        if f3 == 1:
                            size = s
                    shape.append(size)
        elif fn == 4:
            content = bytes(v)
        elif fn == 5:  # float_val, packed or not
            floats += list(struct.unpack("<%df" % (len(v) // 4), v)) if wt == 2 else [struct.unpack("<f", v)[0]]
        elif fn in (7, 10):  # int_val / int64_val
            if wt == 2:
                pos = 0
                while pos < len(v):
                    x, pos = _varint(v, pos)
                    ints.append(x)
            else:
                ints.append(v)
    if dtype not in _TF_DTYPES:
        return None
    dt = np.dtype(_TF_DTYPES[dtype])
    n = int(np.prod(shape)) if shape else 1
    if content is not None:
        arr = np.frombuffer(content, dtype=dt)
    else:
        vals = floats if dt.kind == "f" else ints
        if not vals:
            arr = np.zeros(n, dt)
        else:
            arr = np.array(vals, dtype=dt)
            if arr.size == 1 and n > 1:   # a single value stands for the whole tensor
                arr = np.full(n, arr[0], dt)
    return arr.reshape(shape).copy()


def read_graphdef_constants(data):
    """name -> ndarray for every Const node of a serialized TensorFlow GraphDef."""
    out = {}
    for fn, wt, node in _fields(data):
        if fn != 1 or wt != 2:
            continue
        name, op, tensor = None, None, None
        for f2, w2, v in _fields(node):
            if f2 == 1:
                name = bytes(v).decode()
            elif f2 == 2:
                op = bytes(v).decode()
            elif f2 == 5:  # map<string, AttrValue> entry { key = 1, value = 2 }
                key, val = None, None
                for f3, _, x in _fields(v):
                    if f3 == 1:
                        key = bytes(x).decode()
                    elif f3 == 2:
                        val = x
                if key == "value" and val is not None:
                    for f4, _, t in _fields(val):
                        if f4 == 8:  # AttrValue.tensor
                            tensor = _tensor_proto(t)
        if op == "Const" and name and tensor is not None:
            out[name] = tensor
    return out
