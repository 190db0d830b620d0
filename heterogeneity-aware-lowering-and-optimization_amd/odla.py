"""ctypes host side of libodla_hip.so.

Mirrors what the reference's Python harness does through ctypes
(python/halo/odla.py:54-176 of the reference tree): create a computation,
build the graph by calling the ``odla_<Op>`` builders exactly as HALO-generated
C code would, create a context, bind numpy buffers, execute.  Enumerator values
are taken from include/odla_hip.h (the reference harness's own integer
constants are stale with respect to its headers).

``HipBuilder`` exposes one method per ODLA operator; model descriptions written
against it can be replayed on the CPU oracle, which offers the same methods.
The library is required: there is no CPU fallback on this side.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# ODLA_HIP_LIBRARY names another build of the library (the sanitizer build of the host code)
LIB_PATH = os.environ.get("ODLA_HIP_LIBRARY") or os.path.join(_HERE, "libodla_hip.so")

# ---- enums (include/odla_hip.h) ---------------------------------------------
(ODLA_INT8, ODLA_INT16, ODLA_INT32, ODLA_INT64, ODLA_UINT8, ODLA_UINT16, ODLA_UINT32, ODLA_UINT64,
 ODLA_QINT8, ODLA_QINT16, ODLA_QINT32, ODLA_QINT64, ODLA_QUINT8, ODLA_QUINT16, ODLA_QUINT32,
 ODLA_QUINT64, ODLA_FLOAT16, ODLA_BFLOAT16, ODLA_FLOAT32, ODLA_FLOAT64, ODLA_BOOL, ODLA_STRING) = range(22)
ODLA_SUCCESS = 0
ODLA_INVALID_PARAM = 3
ODLA_COMPUTE_INFERENCE = 1
(ODLA_DYNAMIC_BATCH, ODLA_MIN_BATCH_SIZE, ODLA_MAX_BATCH_SIZE, ODLA_OPT_BATCH_SIZE, ODLA_RUN_BATCH_SIZE,
 ODLA_DYNAMIC_SHAPE, ODLA_MIN_SHAPE, ODLA_MAX_SHAPE, ODLA_OPT_SHAPE, ODLA_DYNAMIC_VALUE, ODLA_MIN_VALUE,
 ODLA_MAX_VALUE, ODLA_OPT_VALUE, ODLA_BF16_MODE, ODLA_FP16_MODE, ODLA_USE_SIM_MODE, ODLA_PROCESSOR_NUM,
 ODLA_BATCHES_PER_STEP, ODLA_USE_DATA_TYPE, ODLA_LOAD_ENGINE_MODE, ODLA_USE_DLA_CORE, ODLA_QUANT_TABLE,
 ODLA_QUANT_TABLE_SIZE, ODLA_AGGREGATE_OPS, ODLA_ENABLE_ENGINE_CACHE, ODLA_CACHE_DIR,
 ODLA_ASYNC_CALLBACK_FUNC, ODLA_ASYNC_CALLBACK_ARG) = range(28)
ODLA_HIP_ITEM_RAW_INT32_ACC = 1000
BF16_DISABLE, BF16_ACCURACY_MODE, BF16_PERFORMACE_MODE, BF16_AUTO_MODE = range(4)
ODLA_CHANNELS_FIRST, ODLA_CHANNELS_LAST, ODLA_SIO, ODLA_SOI, ODLA_OIS, ODLA_IOS = range(6)
ODLA_NEAREST, ODLA_LINEAR, ODLA_CUBIC = range(3)
ODLA_ASSYMMETRIC, ODLA_HALF_PIXEL, ODLA_HALF_PIXEL_TF, ODLA_ALIGN_CORNERS = range(4)
ODLA_MEMCPY_H2H, ODLA_MEMCPY_H2D, ODLA_MEMCPY_D2H, ODLA_MEMCPY_D2D = range(4)
ODLA_DEVICE_INFO_TOTAL_MEMORY, ODLA_DEVICE_INFO_USED_MEMORY = 7, 8

ODLA_MAX_DIMENSION = 10
ODLA_MAX_OUTPUTS = 64

_NP_TO_ODLA = {
    np.dtype(np.float32): ODLA_FLOAT32, np.dtype(np.float16): ODLA_FLOAT16,
    np.dtype(np.int32): ODLA_INT32, np.dtype(np.int64): ODLA_INT64,
    np.dtype(np.int8): ODLA_INT8, np.dtype(np.uint8): ODLA_UINT8, np.dtype(np.bool_): ODLA_BOOL,
    np.dtype(np.uint32): ODLA_UINT32, np.dtype(np.uint64): ODLA_UINT64,
}
_ODLA_TO_NP = {v: k for k, v in _NP_TO_ODLA.items()}


class ValueShape(ctypes.Structure):
    _fields_ = [("size", ctypes.c_int32), ("dims", ctypes.c_int64 * ODLA_MAX_DIMENSION)]


class ValueType(ctypes.Structure):
    _fields_ = [("element_type", ctypes.c_int32), ("shape", ValueShape)]


class Values(ctypes.Structure):
    _fields_ = [("size", ctypes.c_size_t), ("values", ctypes.c_void_p * ODLA_MAX_OUTPUTS)]


class ValueIds(ctypes.Structure):
    _fields_ = [("size", ctypes.c_size_t), ("value_ids", ctypes.c_char_p * ODLA_MAX_OUTPUTS)]


class ResourceLocation(ctypes.Structure):
    _fields_ = [("location_type", ctypes.c_int32), ("location", ctypes.c_void_p), ("size", ctypes.c_size_t)]


ODLA_LOCATION_PATH, ODLA_LOCATION_MEMORY, ODLA_LOCATION_URI = range(3)


def path_location(path):
    """(location, keep-alive object) for a file path."""
    buf = ctypes.create_string_buffer(path.encode())
    return ResourceLocation(ODLA_LOCATION_PATH, ctypes.cast(buf, ctypes.c_void_p), 0), buf


def memory_location(data):
    buf = ctypes.create_string_buffer(bytes(data), len(data))
    return ResourceLocation(ODLA_LOCATION_MEMORY, ctypes.cast(buf, ctypes.c_void_p), len(data)), buf


class PlanSummary(ctypes.Structure):
    """odla_hip_plan_summary."""
    _fields_ = [("launches", ctypes.c_int32), ("init_launches", ctypes.c_int32),
                ("arena_bytes", ctypes.c_uint64), ("constant_bytes", ctypes.c_uint64)]


class QuantInfo(ctypes.Structure):
    _fields_ = [("value_id", ctypes.c_char_p), ("ch_idx", ctypes.c_int), ("scale", ctypes.c_float),
                ("offset", ctypes.c_float), ("min", ctypes.c_float), ("max", ctypes.c_float)]


assert ctypes.sizeof(ValueShape) == 88 and ctypes.sizeof(ValueType) == 96
assert ctypes.sizeof(Values) == 520 and ctypes.sizeof(QuantInfo) == 32


def make_shape(dims):
    s = ValueShape()
    s.size = len(dims)
    for i, d in enumerate(dims):
        s.dims[i] = int(d)
    return s


def undefined_shape():
    s = ValueShape()
    s.size = -1
    return s


def make_type(np_dtype, dims):
    t = ValueType()
    t.element_type = _NP_TO_ODLA[np.dtype(np_dtype)]
    t.shape = make_shape(dims)
    return t


_lib = None


def load_library(path=None):
    """Load libodla_hip.so and declare the prototypes of include/odla_hip.h."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    path = path or LIB_PATH
    if not os.path.exists(path):
        raise RuntimeError("%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`" % path)
    L = ctypes.CDLL(path)
    vp, u32, i32, f32, sz = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int32, ctypes.c_float, ctypes.c_size_t
    pu32 = ctypes.POINTER(ctypes.c_uint32)
    pi32 = ctypes.POINTER(ctypes.c_int32)
    cid = ctypes.c_char_p
    S, T = ValueShape, ValueType

    def proto(name, res, args):
        f = getattr(L, name)
        f.restype = res
        f.argtypes = args

    proto("odla_CreateComputation", i32, [ctypes.POINTER(vp)])
    proto("odla_DestroyComputation", i32, [vp])
    proto("odla_SetComputationItem", i32, [vp, i32, vp])
    proto("odla_CreateContext", i32, [ctypes.POINTER(vp)])
    proto("odla_DestroyContext", i32, [vp])
    proto("odla_SetContextItem", i32, [vp, i32, vp])
    proto("odla_BindToArgument", i32, [vp, vp, vp])
    proto("odla_BindToArgumentById", i32, [cid, vp, vp])
    proto("odla_BindToOutput", i32, [vp, vp, vp])
    proto("odla_BindToOutputById", i32, [cid, vp, vp])
    proto("odla_ExecuteComputation", i32, [vp, vp, i32, vp])
    proto("odla_hip_ExecuteComputationStatic", i32, [vp, vp, i32, vp])
    proto("odla_hip_PlanSummary", i32, [vp, ctypes.POINTER(PlanSummary)])
    proto("odla_GetNumOfArgsFromComputation", i32, [vp, pu32])
    proto("odla_GetArgFromComputationByIdx", i32, [vp, u32, ctypes.POINTER(vp)])
    proto("odla_GetNumOfOutputsFromComputation", i32, [vp, pu32])
    proto("odla_GetOutputFromComputationByIdx", i32, [vp, u32, ctypes.POINTER(vp)])
    proto("odla_GetRuntimeShape", i32, [vp, vp, ctypes.POINTER(S)])
    proto("odla_SetRuntimeShape", i32, [vp, vp, S])
    proto("odla_SetRuntimeValueType", i32, [vp, vp, T])
    proto("odla_GetRuntimeValueType", i32, [vp, vp, ctypes.POINTER(T)])
    proto("odla_GetValueType", i32, [vp, ctypes.POINTER(T)])
    proto("odla_GetValueId", i32, [vp, ctypes.POINTER(cid)])
    proto("odla_FindValueById", i32, [cid, ctypes.POINTER(vp)])
    proto("odla_SetValueAsOutput", i32, [vp])
    proto("odla_SetValuesAsOutput", i32, [Values])
    proto("odla_SetValueAsOutputById", i32, [cid])
    proto("odla_GetValueData", i32, [vp, vp, vp])
    proto("odla_ReleaseValue", i32, [vp])
    proto("odla_CreateValue", vp, [T, cid])
    proto("odla_SetValueData", i32, [vp, vp])
    proto("odla_SetValueDataById", i32, [cid, vp])
    proto("odla_GetValueDataById", i32, [cid, vp])
    proto("odla_CreateArgument", vp, [T, cid])
    proto("odla_CreateConstant", vp, [T, vp, cid])
    proto("odla_AllocateDevice", i32, [vp, i32, i32, ctypes.POINTER(vp)])
    proto("odla_GetDeviceInfo", i32, [vp, i32, vp])
    proto("odla_SetCurrentDevice", i32, [vp])
    proto("odla_DestroyDevice", i32, [vp])
    proto("odla_AllocateDeviceMemory", i32, [ctypes.POINTER(vp), sz])
    proto("odla_FreeDeviceMemory", i32, [vp])
    proto("odla_AllocateHostMemory", i32, [ctypes.POINTER(vp), sz])
    proto("odla_FreeHostMemory", i32, [vp])
    proto("odla_CopyMemory", i32, [vp, vp, sz, i32])
    proto("odla_SetLogLevel", i32, [i32])
    proto("odla_SetLogger", i32, [vp])
    proto("odla_GetLogger", vp, [])
    proto("odla_GetVersionString", ctypes.c_char_p, [])

    proto("odla_Conv", vp, [vp, i32, u32, vp, i32, pu32, pu32, pu32, pu32, vp, S, cid])
    proto("odla_Gemm", vp, [vp, u32, vp, u32, f32, f32, vp, S, cid])
    proto("odla_BatchMatMul", vp, [vp, u32, vp, u32, S, cid])
    for n in ("Add", "Sub", "Mul", "Div", "Max", "Min"):
        proto("odla_" + n, vp, [vp, vp, cid])
    for n in ("Relu", "Sigmoid", "Tanh", "Exp", "Log", "Sqrt", "Rsqrt", "Erf", "Abs", "Neg", "Round"):
        proto("odla_" + n, vp, [vp, cid])
    proto("odla_LeakyRelu", vp, [vp, f32, cid])
    proto("odla_Clamp", vp, [vp, f32, f32, cid])
    proto("odla_Gelu", vp, [vp, u32, cid])
    proto("odla_BatchNormalization", vp, [vp, i32, vp, vp, f32, vp, vp, f32, f32, cid])
    proto("odla_LayerNorm", vp, [vp, sz, pi32, f32, vp, vp, cid])
    proto("odla_MaxPool", vp, [vp, i32, pu32, pu32, pu32, pu32, S, cid])
    proto("odla_AveragePool", vp, [vp, i32, pu32, pu32, pu32, pu32, u32, S, cid])
    for n in ("ReduceMean", "ReduceSum", "ReduceMax"):
        proto("odla_" + n, vp, [vp, sz, pu32, u32, S, cid])
    proto("odla_Softmax", vp, [vp, i32, cid])
    proto("odla_LogSoftmax", vp, [vp, i32, cid])
    proto("odla_Cast", vp, [vp, i32, cid])
    proto("odla_Concat", vp, [Values, i32, S, cid])
    proto("odla_Gather", vp, [vp, vp, i32, S, cid])
    proto("odla_Reshape", vp, [vp, S, cid])
    proto("odla_Resize", vp, [vp, i32, i32, u32, S, cid])
    proto("odla_Slice", vp, [vp, pi32, pi32, pi32, S, cid])
    proto("odla_Transpose", vp, [vp, S, S, cid])
    proto("odla_Quantize", vp, [vp, vp, vp, i32, i32, cid])
    proto("odla_Dequantize", vp, [vp, vp, vp, i32, i32, cid])
    proto("odla_NMS", vp, [vp, vp, u32, f32, f32, T, cid])
    RL = ResourceLocation
    proto("odla_StoreComputation", i32, [RL, vp])
    proto("odla_LoadComputation", i32, [RL, ctypes.POINTER(vp)])
    proto("odla_CompileComputation", i32, [vp, vp, ctypes.POINTER(vp)])
    proto("odla_StoreExecutable", i32, [RL, vp])
    proto("odla_LoadExecutable", i32, [RL, vp, ctypes.POINTER(vp)])
    proto("odla_LaunchExecutable", i32, [vp, vp])
    proto("odla_GetNumOfArgsFromExecutable", i32, [vp, pu32])
    proto("odla_GetArgFromExecutableByIdx", i32, [vp, u32, ctypes.POINTER(vp)])
    proto("odla_GetNumOfOutputsFromExecutable", i32, [vp, pu32])
    proto("odla_GetOutputFromExecutableByIdx", i32, [vp, u32, ctypes.POINTER(vp)])
    proto("odla_DestroyExecutable", i32, [vp])
    i64 = ctypes.c_int64
    for n in ("Reciprocal", "Ceil", "Floor", "Sign", "Sin", "Cos", "Tan", "ASin", "ACos", "ATan", "Sinh", "Cosh",
              "ASinh", "ACosh", "ATanh", "Softplus", "Softsign", "Not", "IsNaN"):
        proto("odla_" + n, vp, [vp, cid])
    for n in ("Elu", "Celu", "ThresholdedRelu"):
        proto("odla_" + n, vp, [vp, f32, cid])
    for n in ("Selu", "HardSigmoid", "Shrink"):
        proto("odla_" + n, vp, [vp, f32, f32, cid])
    for n in ("Pow", "SquaredDifference", "PRelu", "Equal", "NotEqual", "Less", "LessOrEqual", "Greater",
              "GreaterOrEqual", "And", "Or", "Xor"):
        proto("odla_" + n, vp, [vp, vp, cid])
    proto("odla_Mod", vp, [vp, vp, i64, cid])
    proto("odla_Mean", vp, [Values, cid])
    proto("odla_IsInf", vp, [vp, u32, u32, cid])
    proto("odla_Select", vp, [vp, vp, vp, S, cid])
    proto("odla_GatherElements", vp, [vp, vp, i32, S, cid])
    proto("odla_CumSum", vp, [vp, vp, u32, u32, cid])
    proto("odla_Hardmax", vp, [vp, i32, cid])
    proto("odla_Compress", vp, [vp, vp, i32, S, cid])
    proto("odla_Shift", vp, [vp, vp, u32, cid])
    for n in ("ReduceMin", "ReduceProd", "ReduceSumSquare", "ReduceLogSum", "ReduceLogSumExp"):
        proto("odla_" + n, vp, [vp, sz, pu32, u32, S, cid])
    for n in ("ReduceL1", "ReduceL2"):
        proto("odla_" + n, vp, [vp, sz, pu32, u32, f32, S, cid])
    proto("odla_ArgMax", vp, [vp, i32, u32, u32, T, cid])
    proto("odla_ArgMin", vp, [vp, i32, u32, u32, T, cid])
    proto("odla_TopK", Values, [vp, u32, u32, u32, u32, T, T, ValueIds])
    proto("odla_PostProcess", Values, [vp, vp, vp, vp, vp, cid])
    proto("odla_Pad", vp, [vp, pu32, pu32, S, cid])
    proto("odla_Tile", vp, [vp, pu32, S, cid])
    proto("odla_ExpandDims", vp, [vp, S, cid])
    proto("odla_Squeeze", vp, [vp, sz, pu32, S, cid])
    proto("odla_Stack", vp, [Values, i32, S, cid])
    proto("odla_LRN", vp, [vp, i32, i32, f32, f32, f32, cid])
    proto("odla_InstanceNormalization", vp, [vp, i32, f32, vp, vp, f32, f32, cid])
    proto("odla_DeConv", vp, [vp, i32, u32, vp, i32, pu32, pu32, pu32, pu32, vp, S, cid])
    if path == LIB_PATH:
        _lib = L
    return L


def exported_symbols_declared_in_header():
    """Names of all functions declared in include/odla_hip.h."""
    import re
    hdr = os.path.join(os.path.dirname(_HERE), "include", "odla_hip.h")
    text = open(hdr).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = set(re.findall(r"\b(odla_[A-Z]\w*)\s*\(", text))
    names |= set(re.findall(r"^void\s+([A-Z]\w*)\s*\(", text, flags=re.M))  # profiler control functions
    return sorted(names)


def _u32(vals):
    return (ctypes.c_uint32 * len(vals))(*[int(v) for v in vals])


def _i32(vals):
    return (ctypes.c_int32 * len(vals))(*[int(v) for v in vals])


def _cid(name):
    return name.encode() if name else None


class OdlaError(RuntimeError):
    pass


def _check(st, what):
    if st != ODLA_SUCCESS:
        raise OdlaError("%s failed with odla_status %d" % (what, st))


class HipBuilder:
    """Builds an ODLA computation on libodla_hip.so; one method per operator."""

    def __init__(self, fp16=False, bf16=False, quant_table=None, raw_acc=False, lib=None, max_batch=0, min_batch=1):
        """max_batch > 0 records a dynamic-batch computation: arguments declared with a
        leading extent of -1 are planned at max_batch and a Session may run any
        batch min_batch..max_batch (Session.set_batch)."""
        self.L = lib or load_library()
        self.comp = ctypes.c_void_p()
        _check(self.L.odla_CreateComputation(ctypes.byref(self.comp)), "odla_CreateComputation")
        self.max_batch = int(max_batch)
        if self.max_batch > 0:
            t = ctypes.c_bool(True)
            _check(self.L.odla_SetComputationItem(self.comp, ODLA_DYNAMIC_BATCH, ctypes.byref(t)), "DYNAMIC_BATCH")
            for item, n in ((ODLA_MIN_BATCH_SIZE, int(min_batch)), (ODLA_MAX_BATCH_SIZE, self.max_batch),
                            (ODLA_OPT_BATCH_SIZE, self.max_batch)):
                v = ctypes.c_int(n)
                _check(self.L.odla_SetComputationItem(self.comp, item, ctypes.byref(v)), "BATCH_SIZE item")
        self._keep = []      # numpy arrays / ctypes objects that must outlive the computation
        self.args = {}       # name -> (handle, shape, dtype)
        self.outs = {}       # name -> (handle, shape, dtype)
        self._shapes = {}    # handle value -> tuple shape (for convenience)
        if fp16:
            b = ctypes.c_bool(True)
            _check(self.L.odla_SetComputationItem(self.comp, ODLA_FP16_MODE, ctypes.byref(b)), "FP16_MODE")
        if bf16:
            # True / "performance": every FLOAT32 value is stored as bf16; "accuracy": values stay fp32 and
            # only the operands of Conv / Gemm are rounded to bf16 (the reference's two bf16 modes)
            m = ctypes.c_int32(BF16_ACCURACY_MODE if bf16 == "accuracy" else BF16_PERFORMACE_MODE)
            _check(self.L.odla_SetComputationItem(self.comp, ODLA_BF16_MODE, ctypes.byref(m)), "BF16_MODE")
        if quant_table is not None:
            tbl = (QuantInfo * len(quant_table))(*quant_table)
            n = ctypes.c_int(len(quant_table))
            t = ctypes.c_int32(ODLA_INT8)
            self._keep += [tbl, n, t, quant_table]
            _check(self.L.odla_SetComputationItem(self.comp, ODLA_QUANT_TABLE, ctypes.cast(tbl, ctypes.c_void_p)), "QUANT_TABLE")
            _check(self.L.odla_SetComputationItem(self.comp, ODLA_QUANT_TABLE_SIZE, ctypes.byref(n)), "QUANT_TABLE_SIZE")
            _check(self.L.odla_SetComputationItem(self.comp, ODLA_USE_DATA_TYPE, ctypes.byref(t)), "USE_DATA_TYPE")
        if raw_acc:
            b = ctypes.c_bool(True)
            _check(self.L.odla_SetComputationItem(self.comp, ODLA_HIP_ITEM_RAW_INT32_ACC, ctypes.byref(b)), "RAW_ACC")

    # -- helpers --
    def _ret(self, h, what):
        if not h:
            raise OdlaError("%s returned NULL (see the library log)" % what)
        return h

    def shape_of(self, h):
        t = ValueType()
        _check(self.L.odla_GetValueType(h, ctypes.byref(t)), "odla_GetValueType")
        return tuple(t.shape.dims[i] for i in range(t.shape.size)), _ODLA_TO_NP[t.element_type]

    # -- graph inputs --
    def arg(self, name, shape, dtype=np.float32):
        h = self._ret(self.L.odla_CreateArgument(make_type(dtype, shape), _cid(name)), "odla_CreateArgument")
        if shape and shape[0] < 0:          # the dynamic batch: recorded at the largest one
            shape = (self.max_batch,) + tuple(shape[1:])
        self.args[name] = (h, tuple(shape), np.dtype(dtype))
        return h

    def const(self, name, array):
        a = np.ascontiguousarray(array)
        self._keep.append(a)
        shape = a.shape if a.ndim > 0 else ()
        return self._ret(self.L.odla_CreateConstant(make_type(a.dtype, shape), a.ctypes.data_as(ctypes.c_void_p),
                                                    _cid(name)), "odla_CreateConstant")

    def output(self, v, name):
        _check(self.L.odla_SetValueAsOutput(v), "odla_SetValueAsOutput")
        shape, dt = self.shape_of(v)
        self.outs[name] = (v, shape, np.dtype(dt))

    # -- operators --
    def conv(self, x, w, bias=None, stride=(1, 1), pad=(0, 0, 0, 0), dilation=(1, 1), group=1, name=None):
        return self._ret(self.L.odla_Conv(x, ODLA_CHANNELS_FIRST, group, w, ODLA_OIS, _u32(stride), _u32(dilation),
                                          _u32(pad[:2]), _u32(pad[2:]), bias, undefined_shape(), _cid(name)), "odla_Conv")

    def gemm(self, a, b, c=None, ta=False, tb=False, alpha=1.0, beta=1.0, name=None):
        return self._ret(self.L.odla_Gemm(a, int(ta), b, int(tb), alpha, beta, c, undefined_shape(), _cid(name)), "odla_Gemm")

    def batch_matmul(self, a, b, ta=False, tb=False, name=None):
        return self._ret(self.L.odla_BatchMatMul(a, int(ta), b, int(tb), undefined_shape(), _cid(name)), "odla_BatchMatMul")

    def _bin(self, fn, a, b, name):
        return self._ret(getattr(self.L, "odla_" + fn)(a, b, _cid(name)), "odla_" + fn)

    def add(self, a, b, name=None): return self._bin("Add", a, b, name)
    def sub(self, a, b, name=None): return self._bin("Sub", a, b, name)
    def mul(self, a, b, name=None): return self._bin("Mul", a, b, name)
    def div(self, a, b, name=None): return self._bin("Div", a, b, name)
    def max(self, a, b, name=None): return self._bin("Max", a, b, name)
    def min(self, a, b, name=None): return self._bin("Min", a, b, name)

    def _un(self, fn, x, name):
        return self._ret(getattr(self.L, "odla_" + fn)(x, _cid(name)), "odla_" + fn)

    def relu(self, x, name=None): return self._un("Relu", x, name)
    def sigmoid(self, x, name=None): return self._un("Sigmoid", x, name)
    def tanh(self, x, name=None): return self._un("Tanh", x, name)
    def exp(self, x, name=None): return self._un("Exp", x, name)
    def log(self, x, name=None): return self._un("Log", x, name)
    def sqrt(self, x, name=None): return self._un("Sqrt", x, name)
    def rsqrt(self, x, name=None): return self._un("Rsqrt", x, name)
    def erf(self, x, name=None): return self._un("Erf", x, name)
    def abs(self, x, name=None): return self._un("Abs", x, name)
    def neg(self, x, name=None): return self._un("Neg", x, name)
    def round(self, x, name=None): return self._un("Round", x, name)

    def leaky_relu(self, x, alpha, name=None):
        return self._ret(self.L.odla_LeakyRelu(x, alpha, _cid(name)), "odla_LeakyRelu")

    def clamp(self, x, lo, hi, name=None):
        return self._ret(self.L.odla_Clamp(x, lo, hi, _cid(name)), "odla_Clamp")

    def gelu(self, x, approx=False, name=None):
        return self._ret(self.L.odla_Gelu(x, int(approx), _cid(name)), "odla_Gelu")

    def batchnorm(self, x, mean, var, eps, scale=None, offset=None, scalar_scale=1.0, scalar_offset=0.0, name=None):
        return self._ret(self.L.odla_BatchNormalization(x, ODLA_CHANNELS_FIRST, mean, var, eps, scale, offset,
                                                        scalar_scale, scalar_offset, _cid(name)), "odla_BatchNormalization")

    def layernorm(self, x, n_axes, eps, scale=None, offset=None, name=None):
        axes = _i32([-(i + 1) for i in range(n_axes)][::-1])
        return self._ret(self.L.odla_LayerNorm(x, n_axes, axes, eps, scale, offset, _cid(name)), "odla_LayerNorm")

    def maxpool(self, x, window, stride, pad, out_hw=None, name=None):
        od = undefined_shape()
        if out_hw is not None:
            s, _ = self.shape_of(x)
            od = make_shape([s[0], s[1], out_hw[0], out_hw[1]])
        return self._ret(self.L.odla_MaxPool(x, ODLA_CHANNELS_FIRST, _u32(window), _u32(stride), _u32(pad[:2]),
                                             _u32(pad[2:]), od, _cid(name)), "odla_MaxPool")

    def avgpool(self, x, window, stride, pad, count_include_pad=False, out_hw=None, name=None):
        od = undefined_shape()
        if out_hw is not None:
            s, _ = self.shape_of(x)
            od = make_shape([s[0], s[1], out_hw[0], out_hw[1]])
        return self._ret(self.L.odla_AveragePool(x, ODLA_CHANNELS_FIRST, _u32(window), _u32(stride), _u32(pad[:2]),
                                                 _u32(pad[2:]), int(count_include_pad), od, _cid(name)), "odla_AveragePool")

    def _reduce(self, fn, x, axes, keep_dims, name):
        return self._ret(getattr(self.L, "odla_" + fn)(x, len(axes), _u32(axes), int(keep_dims), undefined_shape(),
                                                       _cid(name)), "odla_" + fn)

    def reduce_mean(self, x, axes, keep_dims=True, name=None): return self._reduce("ReduceMean", x, axes, keep_dims, name)
    def reduce_sum(self, x, axes, keep_dims=True, name=None): return self._reduce("ReduceSum", x, axes, keep_dims, name)
    def reduce_max(self, x, axes, keep_dims=True, name=None): return self._reduce("ReduceMax", x, axes, keep_dims, name)

    def softmax(self, x, axis=-1, log=False, name=None):
        f = self.L.odla_LogSoftmax if log else self.L.odla_Softmax
        return self._ret(f(x, axis, _cid(name)), "odla_Softmax")

    def cast(self, x, dtype, name=None):
        return self._ret(self.L.odla_Cast(x, _NP_TO_ODLA[np.dtype(dtype)], _cid(name)), "odla_Cast")

    def concat(self, xs, axis, name=None):
        vs = Values()
        vs.size = len(xs)
        for i, v in enumerate(xs):
            vs.values[i] = v
        return self._ret(self.L.odla_Concat(vs, axis, undefined_shape(), _cid(name)), "odla_Concat")

    def gather(self, x, idx, axis=0, name=None):
        return self._ret(self.L.odla_Gather(x, idx, axis, undefined_shape(), _cid(name)), "odla_Gather")

    def gather_elements(self, x, idx, axis=0, name=None):
        return self._ret(self.L.odla_GatherElements(x, idx, axis, undefined_shape(), _cid(name)), "odla_GatherElements")

    def cumsum(self, x, axis, exclusive=False, reverse=False, name=None):
        ax = self.const((name or "cumsum") + ".axis", np.array([axis], np.int32))
        return self._ret(self.L.odla_CumSum(x, ax, int(exclusive), int(reverse), _cid(name)), "odla_CumSum")

    def hardmax(self, x, axis=-1, name=None):
        return self._ret(self.L.odla_Hardmax(x, axis, _cid(name)), "odla_Hardmax")

    def compress(self, x, cond, axis, max_shape, name=None):
        """axis None: x is taken as one flat axis (the C API's INT_MAX)."""
        return self._ret(self.L.odla_Compress(x, cond, 2 ** 31 - 1 if axis is None else axis, make_shape(max_shape), _cid(name)),
                         "odla_Compress")

    def shift(self, x, amount, left=True, name=None):
        return self._ret(self.L.odla_Shift(x, amount, int(left), _cid(name)), "odla_Shift")

    def reshape(self, x, shape, name=None):
        return self._ret(self.L.odla_Reshape(x, make_shape(shape), _cid(name)), "odla_Reshape")

    def transpose(self, x, perm, name=None):
        return self._ret(self.L.odla_Transpose(x, make_shape(perm), undefined_shape(), _cid(name)), "odla_Transpose")

    def slice(self, x, start, end, stride=None, name=None):
        stride = stride or [1] * len(start)
        return self._ret(self.L.odla_Slice(x, _i32(start), _i32(end), _i32(stride), undefined_shape(), _cid(name)), "odla_Slice")

    def resize_nearest(self, x, out_hw, name=None):
        s, _ = self.shape_of(x)
        return self._ret(self.L.odla_Resize(x, ODLA_NEAREST, ODLA_ASSYMMETRIC, 0,
                                            make_shape([s[0], s[1], out_hw[0], out_hw[1]]), _cid(name)), "odla_Resize")

    def resize_linear(self, x, out_hw, name=None):
        s, _ = self.shape_of(x)
        return self._ret(self.L.odla_Resize(x, ODLA_LINEAR, ODLA_HALF_PIXEL, 0,
                                            make_shape([s[0], s[1], out_hw[0], out_hw[1]]), _cid(name)), "odla_Resize")

    def quantize(self, x, scale, zp=None, axis=-1, signed=False, name=None):
        sc = self.const(None, np.asarray(scale, np.float32).reshape(-1))
        z = None if zp is None else self.const(None, np.asarray(zp, np.int8 if signed else np.uint8).reshape(-1))
        return self._ret(self.L.odla_Quantize(x, sc, z, axis, ODLA_INT8 if signed else ODLA_UINT8, _cid(name)), "odla_Quantize")

    def dequantize(self, q, scale, zp=None, axis=-1, name=None, zp_dtype=np.uint8):
        sc = self.const(None, np.asarray(scale, np.float32).reshape(-1))
        z = None if zp is None else self.const(None, np.asarray(zp, zp_dtype).reshape(-1))
        return self._ret(self.L.odla_Dequantize(q, sc, z, axis, ODLA_FLOAT32, _cid(name)), "odla_Dequantize")

    def nms(self, boxes, scores, max_out, iou_thr, score_thr, name=None):
        return self._ret(self.L.odla_NMS(boxes, scores, max_out, iou_thr, score_thr, make_type(np.int32, [1]), _cid(name)), "odla_NMS")

    # -- wider operator surface --
    def _values(self, xs):
        vs = Values()
        vs.size = len(xs)
        for i, v in enumerate(xs):
            vs.values[i] = v
        return vs

    def reciprocal(self, x, name=None): return self._un("Reciprocal", x, name)
    def ceil(self, x, name=None): return self._un("Ceil", x, name)
    def floor(self, x, name=None): return self._un("Floor", x, name)
    def sign(self, x, name=None): return self._un("Sign", x, name)
    def sin(self, x, name=None): return self._un("Sin", x, name)
    def cos(self, x, name=None): return self._un("Cos", x, name)
    def tan(self, x, name=None): return self._un("Tan", x, name)
    def asin(self, x, name=None): return self._un("ASin", x, name)
    def acos(self, x, name=None): return self._un("ACos", x, name)
    def atan(self, x, name=None): return self._un("ATan", x, name)
    def sinh(self, x, name=None): return self._un("Sinh", x, name)
    def cosh(self, x, name=None): return self._un("Cosh", x, name)
    def asinh(self, x, name=None): return self._un("ASinh", x, name)
    def acosh(self, x, name=None): return self._un("ACosh", x, name)
    def atanh(self, x, name=None): return self._un("ATanh", x, name)
    def softplus(self, x, name=None): return self._un("Softplus", x, name)
    def softsign(self, x, name=None): return self._un("Softsign", x, name)
    def logical_not(self, x, name=None): return self._un("Not", x, name)
    def isnan(self, x, name=None): return self._un("IsNaN", x, name)

    def isinf(self, x, pos=True, neg=True, name=None):
        return self._ret(self.L.odla_IsInf(x, int(pos), int(neg), _cid(name)), "odla_IsInf")

    def elu(self, x, alpha, name=None): return self._ret(self.L.odla_Elu(x, alpha, _cid(name)), "odla_Elu")
    def celu(self, x, alpha, name=None): return self._ret(self.L.odla_Celu(x, alpha, _cid(name)), "odla_Celu")

    def thresholded_relu(self, x, alpha, name=None):
        return self._ret(self.L.odla_ThresholdedRelu(x, alpha, _cid(name)), "odla_ThresholdedRelu")

    def selu(self, x, alpha, gamma, name=None):
        return self._ret(self.L.odla_Selu(x, alpha, gamma, _cid(name)), "odla_Selu")

    def hard_sigmoid(self, x, alpha, beta, name=None):
        return self._ret(self.L.odla_HardSigmoid(x, alpha, beta, _cid(name)), "odla_HardSigmoid")

    def shrink(self, x, bias, lambd, name=None):
        return self._ret(self.L.odla_Shrink(x, bias, lambd, _cid(name)), "odla_Shrink")

    def pow(self, a, b, name=None): return self._bin("Pow", a, b, name)
    def squared_difference(self, a, b, name=None): return self._bin("SquaredDifference", a, b, name)
    def prelu(self, x, slope, name=None): return self._bin("PRelu", x, slope, name)
    def equal(self, a, b, name=None): return self._bin("Equal", a, b, name)
    def not_equal(self, a, b, name=None): return self._bin("NotEqual", a, b, name)
    def less(self, a, b, name=None): return self._bin("Less", a, b, name)
    def less_equal(self, a, b, name=None): return self._bin("LessOrEqual", a, b, name)
    def greater(self, a, b, name=None): return self._bin("Greater", a, b, name)
    def greater_equal(self, a, b, name=None): return self._bin("GreaterOrEqual", a, b, name)
    def logical_and(self, a, b, name=None): return self._bin("And", a, b, name)
    def logical_or(self, a, b, name=None): return self._bin("Or", a, b, name)
    def logical_xor(self, a, b, name=None): return self._bin("Xor", a, b, name)

    def mod(self, a, b, fmod=False, name=None):
        return self._ret(self.L.odla_Mod(a, b, int(fmod), _cid(name)), "odla_Mod")

    def mean(self, xs, name=None):
        return self._ret(self.L.odla_Mean(self._values(xs), _cid(name)), "odla_Mean")

    def select(self, cond, a, b, name=None):
        return self._ret(self.L.odla_Select(cond, a, b, undefined_shape(), _cid(name)), "odla_Select")

    def reduce_min(self, x, axes, keep_dims=True, name=None): return self._reduce("ReduceMin", x, axes, keep_dims, name)
    def reduce_prod(self, x, axes, keep_dims=True, name=None): return self._reduce("ReduceProd", x, axes, keep_dims, name)
    def reduce_sum_square(self, x, axes, keep_dims=True, name=None): return self._reduce("ReduceSumSquare", x, axes, keep_dims, name)
    def reduce_log_sum(self, x, axes, keep_dims=True, name=None): return self._reduce("ReduceLogSum", x, axes, keep_dims, name)
    def reduce_log_sum_exp(self, x, axes, keep_dims=True, name=None): return self._reduce("ReduceLogSumExp", x, axes, keep_dims, name)

    def _reduce_eps(self, fn, x, axes, keep_dims, eps, name):
        return self._ret(getattr(self.L, "odla_" + fn)(x, len(axes), _u32(axes), int(keep_dims), eps, undefined_shape(),
                                                       _cid(name)), "odla_" + fn)

    def reduce_l1(self, x, axes, keep_dims=True, eps=0.0, name=None): return self._reduce_eps("ReduceL1", x, axes, keep_dims, eps, name)
    def reduce_l2(self, x, axes, keep_dims=True, eps=0.0, name=None): return self._reduce_eps("ReduceL2", x, axes, keep_dims, eps, name)

    def _arg(self, fn, x, axis, keep_dims, last, dtype, name):
        return self._ret(getattr(self.L, "odla_" + fn)(x, axis, int(keep_dims), int(last), make_type(dtype, [1]),
                                                       _cid(name)), "odla_" + fn)

    def argmax(self, x, axis, keep_dims=True, last=False, dtype=np.int32, name=None):
        return self._arg("ArgMax", x, axis, keep_dims, last, dtype, name)

    def argmin(self, x, axis, keep_dims=True, last=False, dtype=np.int32, name=None):
        return self._arg("ArgMin", x, axis, keep_dims, last, dtype, name)

    def topk(self, x, k, axis, largest=True, index_dtype=np.int32, names=(None, None)):
        ids = ValueIds()
        ids.size = 2
        for i, n in enumerate(names):
            ids.value_ids[i] = _cid(n)
        r = self.L.odla_TopK(x, k, int(largest), 1, axis, make_type(np.float32, [1]), make_type(index_dtype, [1]), ids)
        if r.size != 2:
            raise OdlaError("odla_TopK failed (see the library log)")
        return r.values[0], r.values[1]

    def yolo_postprocess(self, img_w, img_h, bb13, bb26, bb52, name=None):
        """-> (rows [classes, N/169, 5], rows kept [classes]); the values are named name+"0" / name+"1"."""
        r = self.L.odla_PostProcess(img_w, img_h, bb13, bb26, bb52, _cid(name))
        if r.size != 2:
            raise OdlaError("odla_PostProcess failed (see the library log)")
        return r.values[0], r.values[1]

    def pad(self, x, front, back, name=None):
        return self._ret(self.L.odla_Pad(x, _u32(front), _u32(back), undefined_shape(), _cid(name)), "odla_Pad")

    def tile(self, x, repeat, name=None):
        return self._ret(self.L.odla_Tile(x, _u32(repeat), undefined_shape(), _cid(name)), "odla_Tile")

    def broadcast_to(self, x, shape, name=None):
        return self._ret(self.L.odla_ExpandDims(x, make_shape(shape), _cid(name)), "odla_ExpandDims")

    def squeeze(self, x, axes, name=None):
        return self._ret(self.L.odla_Squeeze(x, len(axes), _u32(axes), undefined_shape(), _cid(name)), "odla_Squeeze")

    def stack(self, xs, axis, name=None):
        return self._ret(self.L.odla_Stack(self._values(xs), axis, undefined_shape(), _cid(name)), "odla_Stack")

    def lrn(self, x, window, alpha, beta, bias, name=None):
        return self._ret(self.L.odla_LRN(x, ODLA_CHANNELS_FIRST, window, alpha, beta, bias, _cid(name)), "odla_LRN")

    def instance_norm(self, x, eps, scale=None, offset=None, scalar_scale=1.0, scalar_offset=0.0, name=None):
        return self._ret(self.L.odla_InstanceNormalization(x, ODLA_CHANNELS_FIRST, eps, scale, offset, scalar_scale,
                                                           scalar_offset, _cid(name)), "odla_InstanceNormalization")

    def deconv(self, x, w, bias=None, stride=(1, 1), pad=(0, 0, 0, 0), group=1, out_hw=None, name=None):
        """w in the ONNX ConvTranspose order [C_in, C_out / group, kH, kW]."""
        od = undefined_shape()
        if out_hw is not None:
            s, _ = self.shape_of(x)
            ws, _ = self.shape_of(w)
            od = make_shape([s[0], ws[1] * group, out_hw[0], out_hw[1]])
        return self._ret(self.L.odla_DeConv(x, ODLA_CHANNELS_FIRST, group, w, ODLA_IOS, _u32(stride), _u32((1, 1)),
                                            _u32(pad[:2]), _u32(pad[2:]), bias, od, _cid(name)), "odla_DeConv")

    # -- execution --
    def session(self, use_graph=True):
        return Session(self, use_graph)

    def plan_summary(self):
        """odla_hip_PlanSummary: lowers the recorded graph on the host (no device
        needed) and returns its launch count and device-memory needs."""
        ps = PlanSummary()
        _check(self.L.odla_hip_PlanSummary(self.comp, ctypes.byref(ps)), "odla_hip_PlanSummary")
        return {"launches": ps.launches, "init_launches": ps.init_launches, "arena_bytes": ps.arena_bytes,
                "constant_bytes": ps.constant_bytes}

    def destroy(self):
        if self.comp:
            self.L.odla_DestroyComputation(self.comp)
            self.comp = None


class Session:
    """One odla_context: bind numpy (host) or device buffers, execute."""

    def __init__(self, builder, use_graph=True):
        self.b = builder
        self.L = builder.L
        self.ctx = ctypes.c_void_p()
        _check(self.L.odla_CreateContext(ctypes.byref(self.ctx)), "odla_CreateContext")
        if not use_graph:
            f = ctypes.c_bool(False)
            _check(self.L.odla_SetContextItem(self.ctx, ODLA_AGGREGATE_OPS, ctypes.byref(f)), "AGGREGATE_OPS")
        self._dev = []

    def set_batch(self, batch):
        """Run the following executions at `batch` (dynamic-batch computations)."""
        v = ctypes.c_int(int(batch))
        _check(self.L.odla_SetContextItem(self.ctx, ODLA_RUN_BATCH_SIZE, ctypes.byref(v)), "RUN_BATCH_SIZE")

    def runtime_shape(self, h):
        """Shape of a value at the batch this session runs at."""
        s = ValueShape()
        _check(self.L.odla_GetRuntimeShape(self.ctx, h, ctypes.byref(s)), "odla_GetRuntimeShape")
        return tuple(s.dims[i] for i in range(s.size))

    def run(self, feeds):
        """feeds: name -> numpy array.  Returns name -> numpy array."""
        keep = []
        for name, (h, shape, dt) in self.b.args.items():
            a = np.ascontiguousarray(feeds[name], dtype=dt)
            assert tuple(a.shape) == self.runtime_shape(h), (name, a.shape, self.runtime_shape(h))
            keep.append(a)
            _check(self.L.odla_BindToArgument(h, a.ctypes.data_as(ctypes.c_void_p), self.ctx), "odla_BindToArgument")
        outs = {}
        for name, (h, shape, dt) in self.b.outs.items():
            o = np.empty(self.runtime_shape(h), dt)
            outs[name] = o
            _check(self.L.odla_BindToOutput(h, o.ctypes.data_as(ctypes.c_void_p), self.ctx), "odla_BindToOutput")
        _check(self.L.odla_ExecuteComputation(self.b.comp, self.ctx, ODLA_COMPUTE_INFERENCE, None), "odla_ExecuteComputation")
        return outs

    def bind_device_io(self, feeds):
        """Copy `feeds` into device memory once and bind device buffers for every
        argument and output, so that execute() moves no data across PCIe."""
        self.dev_out = {}
        for name, (h, shape, dt) in self.b.args.items():
            a = np.ascontiguousarray(feeds[name], dtype=dt)
            p = ctypes.c_void_p()
            _check(self.L.odla_AllocateDeviceMemory(ctypes.byref(p), a.nbytes), "odla_AllocateDeviceMemory")
            _check(self.L.odla_CopyMemory(p, a.ctypes.data_as(ctypes.c_void_p), a.nbytes, ODLA_MEMCPY_H2D), "odla_CopyMemory")
            self._dev.append(p)
            _check(self.L.odla_BindToArgument(h, p, self.ctx), "odla_BindToArgument")
        for name, (h, shape, dt) in self.b.outs.items():
            nbytes = int(np.prod(shape)) * dt.itemsize
            p = ctypes.c_void_p()
            _check(self.L.odla_AllocateDeviceMemory(ctypes.byref(p), nbytes), "odla_AllocateDeviceMemory")
            self._dev.append(p)
            self.dev_out[name] = (p, shape, dt)
            _check(self.L.odla_BindToOutput(h, p, self.ctx), "odla_BindToOutput")

    def bind_host_io(self, feeds, pinned=False):
        """Bind HOST buffers for every argument and output, so that execute() copies the
        arguments to the device and the results back, as a caller of the reference's
        harness pays it (python/halo/odla.py:172-175 times odla_ExecuteComputation on host
        arrays).  pinned=False: ordinary (pageable) numpy arrays; True: page-locked
        buffers from odla_AllocateHostMemory.  Returns name -> numpy view of each output."""
        self._host_keep = []
        self._host_pinned = getattr(self, "_host_pinned", [])

        def buffer(nbytes, dt, shape):
            if not pinned:
                return np.empty(shape, dt)
            p = ctypes.c_void_p()
            _check(self.L.odla_AllocateHostMemory(ctypes.byref(p), max(nbytes, 1)), "odla_AllocateHostMemory")
            self._host_pinned.append(p)
            raw = (ctypes.c_uint8 * max(nbytes, 1)).from_address(p.value)
            return np.frombuffer(raw, dtype=dt, count=int(np.prod(shape))).reshape(shape)

        for name, (h, shape, dt) in self.b.args.items():
            src = np.ascontiguousarray(feeds[name], dtype=dt)
            a = buffer(src.nbytes, dt, src.shape)
            a[...] = src
            self._host_keep.append(a)
            _check(self.L.odla_BindToArgument(h, a.ctypes.data_as(ctypes.c_void_p), self.ctx), "odla_BindToArgument")
        outs = {}
        for name, (h, shape, dt) in self.b.outs.items():
            o = buffer(int(np.prod(shape)) * dt.itemsize, dt, tuple(shape))
            outs[name] = o
            self._host_keep.append(o)
            _check(self.L.odla_BindToOutput(h, o.ctypes.data_as(ctypes.c_void_p), self.ctx), "odla_BindToOutput")
        return outs

    def execute(self):
        _check(self.L.odla_ExecuteComputation(self.b.comp, self.ctx, ODLA_COMPUTE_INFERENCE, None), "odla_ExecuteComputation")

    def execute_static(self):
        """The same step through the entry point that allocates nothing (temporaries in the
        library's static device scratch); returns the status code."""
        return self.L.odla_hip_ExecuteComputationStatic(self.b.comp, self.ctx, ODLA_COMPUTE_INFERENCE, None)

    def fetch_device_outputs(self):
        outs = {}
        for name, (p, shape, dt) in self.dev_out.items():
            o = np.empty(shape, dt)
            _check(self.L.odla_CopyMemory(o.ctypes.data_as(ctypes.c_void_p), p, o.nbytes, ODLA_MEMCPY_D2H), "odla_CopyMemory")
            outs[name] = o
        return outs

    def close(self):
        for p in self._dev:
            self.L.odla_FreeDeviceMemory(p)
        self._dev = []
        for p in getattr(self, "_host_pinned", []):
            self.L.odla_FreeHostMemory(p)
        self._host_pinned = []
        self._host_keep = []
        if self.ctx:
            self.L.odla_DestroyContext(self.ctx)
            self.ctx = None


class ScalarValue(ctypes.Structure):
    _fields_ = [("data_type", ctypes.c_int32), ("val_int64", ctypes.c_int64)]


def used_device_memory(L=None):
    """Bytes in use on the default device (odla_GetDeviceInfo, ODLA_DEVICE_INFO_USED_MEMORY)."""
    L = L or load_library()
    dev = ctypes.c_void_p()
    _check(L.odla_AllocateDevice(None, 0, 0, ctypes.byref(dev)), "odla_AllocateDevice")
    val = ScalarValue()
    _check(L.odla_GetDeviceInfo(dev, ODLA_DEVICE_INFO_USED_MEMORY, ctypes.byref(val)), "odla_GetDeviceInfo")
    L.odla_DestroyDevice(dev)
    return int(val.val_int64)


def quant_table(entries):
    """entries: list of (name, scale, zero_point, min, max, channel_minmax or None).
    Emits records in the reference writer's format (utils/halo_pgq.py:308-332):
    one tensor record with ch_idx = -channels, then one record per channel."""
    recs = []
    for name, scale, zp, mn, mx, ch in entries:
        nch = len(ch) if ch is not None else 1
        recs.append(QuantInfo(name.encode(), -nch, float(scale), float(zp), float(mn), float(mx)))
        if ch is not None:
            for c, (cmn, cmx) in enumerate(ch):
                recs.append(QuantInfo(name.encode(), c, 0.0, 0.0, float(cmn), float(cmx)))
    return recs
