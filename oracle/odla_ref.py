"""CPU oracle for the ODLA hot path -- TEST INFRASTRUCTURE ONLY.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the shipped library never does.

``RefBuilder`` offers the same builder vocabulary as the GPU-side
``HipBuilder`` (one method per ``odla_<Op>``) but evaluates every operator
eagerly on numpy arrays in fp32, restating what the reference CPU backend
computes.  Each method cites the reference code it follows; paths are relative
to the reference tree.  Heavy loops live in ``odla_ref.c`` (built to
``libodla_ref.so`` by ``oracle/Makefile``).

Pin status (what fixes each function independently of this file):
  conv2d / gemm (plain and batched) / pools / softmax / batchnorm
      reference-held known-answer vectors (odla_popart/test), the reference's
      own fp32 kernels built to ``oracle/_ref/libsn_rt.so``, float64 brute force.
  reduce_mean / argmax (first maximum) / slice / gather / transpose / pad /
      erf / add, sub, mul, div with broadcasting   vectors of the same
      reference kernels (runtime/generic/*.cc) held in tests/golden.
  quantize / dequantize   ONNX QuantizeLinear published example (passes on the
      reference CPU backend), exhaustive half-integer rounding check.
  layernorm / gelu / concat   closed forms and library routines (math.erf, numpy).
  resize_nearest   hand-listed source indices for non-integer ratios and the
      loops of the reference's portable backend (odla_eigen.cc:619-631) restated
      in plain Python.
  cast_like_reference   hand-listed roundings (ties to even), saturation ends
      and narrowing cases; behaviour at |x| >= 2^31 and for NaN is this build's
      choice: PARITY UNPINNED there.
  qadd (residual add of two 8-bit tensors)   hand-worked levels with exact
      power-of-two scales: both ties, both clamps, the fused ReLU clamp.
  nms   ONNX NonMaxSuppression published examples, O(n^2) brute force.
  wider operator surface (trigonometric / hyperbolic functions, Elu family,
      comparisons, Select, Mod, reductions, ArgMax, TopK, Pad, Tile, LRN,
      InstanceNormalization, DeConv)   numpy / math library routines and
      the scatter definition of the transposed convolution (``deconv2d``); cross-checked in
      tests against torch's CPU operators.  TopK tie order (ascending index) is
      this build's choice: the reference's portable TopK is not implemented
      (``dnnl_utils.h:52-56``), so ties are PARITY UNPINNED.
  yolo_decode / yolo_class_walk / yolo_postprocess   closed forms of the
      decode (float64 sigmoid / exp), the same boxes from the Sigmoid / Exp
      graph of the package's YOLOv3 builder, hand-worked walks that separate
      "compare with the box kept last" from greedy suppression.  The order of
      equal scores (ascending row) and the stop at N/169 rows per class are
      this build's choices where the reference leaves the result open
      (unstable sort; writes past the end): PARITY UNPINNED for those two.
  int8 convolution + requantisation (``qconv`` ...)   PARITY UNPINNED by the
      reference: it has no int8 convolution of its own.  The int32 accumulators
      are pinned by int64 brute force; the requantisation formula is this
      build's definition.
"""
import ctypes
import math
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def lib():
    """libodla_ref.so, loaded on first use."""
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libodla_ref.so")
        if not os.path.exists(path):
            raise RuntimeError("oracle/libodla_ref.so is missing: run `make -C oracle`")
        _LIB = ctypes.CDLL(path)
        _LIB.odla_ref_num_threads.restype = ctypes.c_int
    return _LIB


def num_threads():
    return int(lib().odla_ref_num_threads())


def _p(a, t):
    return a.ctypes.data_as(ctypes.POINTER(t))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def round_to_storage(a, storage):
    """The fp32 array `a` with every element rounded (to nearest, ties to even) to
    the nearest value of a 16-bit storage type, still held as fp32.  "bf16": the
    upper 16 bits of the fp32 pattern; "fp16": IEEE binary16 (values beyond its
    range become infinities, as in a hardware conversion)."""
    a = _f32(a)
    if storage == "bf16":
        u = a.view(np.uint32).astype(np.uint64)
        r = ((u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000).astype(np.uint32).view(np.float32)
        return np.where(np.isnan(a), a, r).astype(np.float32).reshape(a.shape)
    if storage == "fp16":
        with np.errstate(over="ignore"):
            return a.astype(np.float16).astype(np.float32)
    raise ValueError("unknown storage type %r" % (storage,))


# --------------------------------------------------------------------------
# Heavy kernels (C)
# --------------------------------------------------------------------------
def conv_out_dim(i, k, s, pf, pb, d=1):
    return (i + pf + pb - ((k - 1) * d + 1)) // s + 1


def conv2d(x, w, bias=None, stride=(1, 1), pad=(0, 0, 0, 0), dilation=(1, 1), group=1):
    """NCHW x OIHW cross-correlation.  pad = (top, left, bottom, right).
    [ref: ODLA/platforms/dnnl/odla_dnnl.cc:1014-1129]"""
    x, w = _f32(x), _f32(w)
    N, C, H, W = x.shape
    O, I, R, S = w.shape
    assert C == I * group and O % group == 0
    Ho = conv_out_dim(H, R, stride[0], pad[0], pad[2], dilation[0])
    Wo = conv_out_dim(W, S, stride[1], pad[1], pad[3], dilation[1])
    y = np.empty((N, O, Ho, Wo), np.float32)
    b = None if bias is None else _f32(bias).reshape(-1)
    lib().odla_ref_conv2d_f32(
        _p(x, ctypes.c_float), _p(w, ctypes.c_float),
        _p(b, ctypes.c_float) if b is not None else None, _p(y, ctypes.c_float),
        N, C, H, W, O, R, S, group, stride[0], stride[1], dilation[0], dilation[1],
        pad[0], pad[1], Ho, Wo)
    return y


def pool2d(x, window, stride, pad, out_hw=None, is_max=True, count_include_pad=False):
    """NCHW pooling.  [ref: odla_dnnl.cc:1360-1446]: max pooling ignores padding;
    average pooling divides by the in-bounds count (oneDNN pooling_avg ==
    exclude-padding) unless count_include_pad."""
    x = _f32(x)
    N, C, H, W = x.shape
    Ho = conv_out_dim(H, window[0], stride[0], pad[0], pad[2]) if out_hw is None else out_hw[0]
    Wo = conv_out_dim(W, window[1], stride[1], pad[1], pad[3]) if out_hw is None else out_hw[1]
    y = np.empty((N, C, Ho, Wo), np.float32)
    lib().odla_ref_pool2d_f32(_p(x, ctypes.c_float), _p(y, ctypes.c_float), N, C, H, W,
                              window[0], window[1], stride[0], stride[1], pad[0], pad[1], Ho, Wo,
                              1 if is_max else 0, 1 if count_include_pad else 0)
    return y


def conv2d_q8_acc(xq, zp_x, wq, bias_i32=None, stride=(1, 1), pad=(0, 0, 0, 0)):
    """int32 accumulators of a u8 x s8 convolution (see odla_ref.c)."""
    xq = np.ascontiguousarray(xq, dtype=np.uint8)
    wq = np.ascontiguousarray(wq, dtype=np.int8)
    N, C, H, W = xq.shape
    O, I, R, S = wq.shape
    assert C == I
    Ho = conv_out_dim(H, R, stride[0], pad[0], pad[2])
    Wo = conv_out_dim(W, S, stride[1], pad[1], pad[3])
    acc = np.empty((N, O, Ho, Wo), np.int32)
    b = None if bias_i32 is None else np.ascontiguousarray(bias_i32, dtype=np.int32)
    lib().odla_ref_conv2d_q8(_p(xq, ctypes.c_uint8), int(zp_x), _p(wq, ctypes.c_int8),
                             _p(b, ctypes.c_int32) if b is not None else None,
                             _p(acc, ctypes.c_int32), N, C, H, W, O, R, S,
                             stride[0], stride[1], pad[0], pad[1], Ho, Wo)
    return acc


def requant_q8(acc, mul, zp, lo=0, res=None, r_mul=0.0, r_add=0.0):
    """q = sat8(max(fma(float32(acc), mul[o], add), lo)) with add = zp, or, with a
    residual `res` (uint8 levels shaped like acc), add = fma(float32(res), r_mul, r_add).
    fma = one fused multiply-add in float32 (C fmaf); sat8 = round half to even,
    saturate to [0, 255].  This is the int8 plan's own definition (PARITY UNPINNED by
    the reference, which has no int8 convolution)."""
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    N, O = acc.shape[0], acc.shape[1]
    HW = int(np.prod(acc.shape[2:])) if acc.ndim > 2 else 1
    mul = _f32(mul).reshape(-1)
    assert mul.size == O
    q = np.empty(acc.shape, np.uint8)
    f = lib().odla_ref_requant_q8
    f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_float, ctypes.c_void_p, ctypes.c_float,
                  ctypes.c_float, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
    f.restype = None
    rp = None
    if res is not None:
        res = np.ascontiguousarray(res, dtype=np.uint8)
        assert res.shape == acc.shape
        rp = res.ctypes.data
    f(acc.ctypes.data, mul.ctypes.data, float(np.float32(zp)), float(np.float32(lo)), rp, float(np.float32(r_mul)),
      float(np.float32(r_add)), q.ctypes.data, N, O, HW)
    return q


# --------------------------------------------------------------------------
# Quantisation scheme of the int8 plan
# [ref: utils/halo_pgq.py:283-297 (activations), lib/quantizer/weights_quantizer.cc:35-64,
#  126-176 (zero-point clamp, bias)]
# --------------------------------------------------------------------------
def act_qparams(mn, mx):
    """Asymmetric u8: scale = (max-min)/255, zp = clip(rne(-min/scale), 0, 255).
    The range is widened to contain 0 so that 0 is exactly representable."""
    mn = np.float32(min(float(mn), 0.0))
    mx = np.float32(max(float(mx), 0.0))
    scale = np.float32((mx - mn) / np.float32(255.0))
    if not scale > 0:
        scale = np.float32(1.0)
    zp = int(np.clip(np.rint(np.float32(-mn) / scale), 0, 255))
    return scale, zp


def weight_qparams(w):
    """Symmetric per-output-channel s8: scale[o] = max|w_o| / 127."""
    w = _f32(w)
    m = np.abs(w.reshape(w.shape[0], -1)).max(axis=1).astype(np.float32)
    s = (m / np.float32(127.0)).astype(np.float32)
    s[m == 0] = np.float32(1.0)
    return s


def quantize_weights(w, s):
    w = _f32(w)
    q = np.rint(w / s.reshape((-1,) + (1,) * (w.ndim - 1)).astype(np.float32))
    return np.clip(q, -127, 127).astype(np.int8)


def quantize_bias(b, s_x, s_w):
    """int32 bias = rne(b / (s_x * s_w[o]))."""
    bs = (np.float32(s_x) * s_w.astype(np.float32)).astype(np.float32)
    r = np.rint(_f32(b).reshape(-1) / bs)
    return np.clip(r, -2147483648.0, 2147483520.0).astype(np.int64).astype(np.int32)


def quantize_act(x, scale, zp):
    """q = clamp(rne(x / scale) + zp, 0, 255)   [ref: odla_dnnl_quantization.cc:61-90]"""
    t = np.rint(_f32(x) / np.float32(scale)) + np.float32(zp)
    return np.clip(t, 0, 255).astype(np.uint8)


def dequantize_act(q, scale, zp):
    """x = (q - zp) * scale   [ref: odla_dnnl_quantization.cc:33-59]"""
    return ((q.astype(np.float32) - np.float32(zp)) * np.float32(scale)).astype(np.float32)


def qconv(xq, x_qp, w, bias, out_qp, stride, pad, relu=False, residual=None):
    """int8 convolution with fused requantisation, as the int8 plan defines it:
    ONE requantisation to out_qp behind everything fused into the convolution - the
    ReLU (a lower clamp at the zero point) and, when `residual` = (levels, (scale,
    zp)) is given, the residual add: its levels enter the fused multiply-add as
    fma(float(r), s_r / s_y, zp_y - zp_r * (s_r / s_y)).
    Returns (q_out u8, acc int32)."""
    s_x, zp_x = x_qp
    s_w = weight_qparams(w)
    wq = quantize_weights(w, s_w)
    bi = None if bias is None else quantize_bias(bias, s_x, s_w)
    acc = conv2d_q8_acc(xq, zp_x, wq, bi, stride, pad)
    s_y, zp_y = out_qp
    mul = ((np.float32(s_x) * s_w).astype(np.float32) / np.float32(s_y)).astype(np.float32)
    lo = zp_y if relu else 0
    if residual is None:
        return requant_q8(acc, mul, zp_y, lo), acc
    rq, (s_r, zp_r) = residual
    r_mul = np.float32(s_r) / np.float32(s_y)
    r_add = np.float32(zp_y) - np.float32(zp_r) * r_mul
    return requant_q8(acc, mul, zp_y, lo, rq, r_mul, r_add), acc


def cast_like_reference(x, dtype):
    """odla_Cast: a oneDNN reorder between f32 / s32 / s8 / u8 / bf16
    [ref: ODLA/platforms/dnnl/odla_dnnl_cast.cc:232-258].  A floating-point value
    that becomes an integer is rounded to nearest, ties to even, and saturates
    at the ends of the target range (2147483520, the largest float below 2^31,
    stands in for the upper end of int32); an integer that becomes a narrower
    integer saturates; anything that becomes a bool is "!= 0".  Half-precision
    targets round to nearest even (the reference's own fp16 conversion
    truncates the mantissa, ``:49-104``; that defect is not reproduced).
    Behaviour at |x| >= 2^31 and for NaN (-> 0) is this build's choice:
    PARITY UNPINNED there."""
    x = np.asarray(x)
    dt = np.dtype(dtype)
    if dt == np.bool_:
        return x != 0
    if dt.kind in "iu":
        info = np.iinfo(dt)
        if x.dtype.kind == "f":
            v = x.astype(np.float32)
            hi = {8: 9223371487098961920.0, 4: 2147483520.0}.get(dt.itemsize, float(info.max))
            v = np.where(np.isnan(v), np.float32(0), v)
            v = np.clip(v, np.float32(info.min), np.float32(hi))
            return np.rint(v).astype(dt)
        if x.dtype == np.bool_:
            return x.astype(dt)
        return np.clip(x.astype(np.int64), info.min, info.max).astype(dt)
    return x.astype(dt)


def qadd(aq, a_qp, bq, b_qp, out_qp, relu=False):
    """Residual add in the quantised domain: dequantise both, add in fp32,
    requantise with a multiply by float32(1/s_out)."""
    fa = dequantize_act(aq, *a_qp)
    fb = dequantize_act(bq, *b_qp)
    f = (fa + fb).astype(np.float32)
    s_y, zp_y = out_qp
    inv = np.float32(1.0) / np.float32(s_y)
    q = np.rint(f * inv).astype(np.int64) + int(zp_y)
    return np.clip(q, zp_y if relu else 0, 255).astype(np.uint8)


# --------------------------------------------------------------------------
# NMS  [ref: ODLA/platforms/dnnl/dnnl_utils_avx512.h:977-1079, selection rule as intended]
# --------------------------------------------------------------------------
def deconv2d(x, w, bias=None, stride=(1, 1), pad=(0, 0, 0, 0), group=1, out_hw=None):
    """Transposed convolution by its definition: every input element scatters its
    kernel-weighted copy into the output, y[n, o, hi*s - p + r, wi*s - p + q] +=
    x[n, c, hi, wi] * w[c, o_in_group, r, q]  (w in [C_in, C_out/group, kH, kW]
    order; dnnl deconvolution_direct [ref: odla_dnnl.cc:1131-1232])."""
    x = _f32(x).astype(np.float64)
    w = _f32(w).astype(np.float64)
    N, C, H, W = x.shape
    Cin, Og, R, S = w.shape
    assert Cin == C and C % group == 0
    Cg = C // group
    Ho = (H - 1) * stride[0] - pad[0] - pad[2] + R
    Wo = (W - 1) * stride[1] - pad[1] - pad[3] + S
    if out_hw is not None:
        Ho, Wo = out_hw
    full = np.zeros((N, Og * group, (H - 1) * stride[0] + R + stride[0], (W - 1) * stride[1] + S + stride[1]))
    for g in range(group):
        xg = x[:, g * Cg:(g + 1) * Cg]
        wg = w[g * Cg:(g + 1) * Cg]
        for r in range(R):
            for q in range(S):
                contrib = np.einsum("nchw,co->nohw", xg, wg[:, :, r, q])
                full[:, g * Og:(g + 1) * Og, r:r + (H - 1) * stride[0] + 1:stride[0],
                     q:q + (W - 1) * stride[1] + 1:stride[1]] += contrib
    y = full[:, :, pad[0]:pad[0] + Ho, pad[1]:pad[1] + Wo]
    if bias is not None:
        y = y + _f32(bias).astype(np.float64).reshape(1, -1, 1, 1)
    return np.ascontiguousarray(y).astype(np.float32)


def _iou_one_to_many(box, others):
    f = np.float32
    y1 = np.minimum(box[0], box[2]); x1 = np.minimum(box[1], box[3])
    y2 = np.maximum(box[0], box[2]); x2 = np.maximum(box[1], box[3])
    oy1 = np.minimum(others[:, 0], others[:, 2]); ox1 = np.minimum(others[:, 1], others[:, 3])
    oy2 = np.maximum(others[:, 0], others[:, 2]); ox2 = np.maximum(others[:, 1], others[:, 3])
    area_i = ((oy2 - oy1) * (ox2 - ox1)).astype(f)
    area_j = f((y2 - y1) * (x2 - x1))
    ih = np.maximum(np.minimum(oy2, y2) - np.maximum(oy1, y1), f(0)).astype(f)
    iw = np.maximum(np.minimum(ox2, x2) - np.maximum(ox1, x1), f(0)).astype(f)
    inter = (ih * iw).astype(f)
    with np.errstate(divide="ignore", invalid="ignore"):
        iou = (inter / ((area_i + area_j).astype(f) - inter).astype(f)).astype(f)
    iou[(area_i <= 0) | (area_j <= 0)] = 0
    return iou


def nms(boxes, scores, max_out, iou_thr, score_thr):
    """boxes [N,B,4] (y1,x1,y2,x2), scores [N,C,B] -> int32 [N*max_out,3] rows
    {image, class, box}, -1 padded."""
    boxes, scores = _f32(boxes), _f32(scores)
    N, B, _ = boxes.shape
    out = np.full((N, max_out, 3), -1, np.int32)
    for n in range(N):
        sc = scores[n]                      # [C,B]
        cls = np.argmax(sc, axis=0)         # first maximum
        best = sc[cls, np.arange(B)]
        cand = np.nonzero(best > np.float32(score_thr))[0]
        if cand.size == 0 or max_out == 0:
            continue
        order = cand[np.lexsort((cand, -best[cand].astype(np.float64)))]
        alive = np.ones(order.size, bool)
        kept = 0
        for i in range(order.size):
            if not alive[i]:
                continue
            if kept >= max_out:
                break
            bi = order[i]
            out[n, kept] = (n, cls[bi], bi)
            kept += 1
            rest = np.nonzero(alive[i + 1:])[0] + i + 1
            if rest.size:
                iou = _iou_one_to_many(boxes[n, bi], boxes[n, order[rest]])
                alive[rest[iou >= np.float32(iou_thr)]] = False
    return out.reshape(N * max_out, 3)


# --------------------------------------------------------------------------
# YOLOv3 post-processing of one image
#   [ref: models/vision/detection/yolo/yolov3_postproc.cc:34-88 (decode), :90-153 (per-class
#    walk); ODLA/platforms/odla_popart/custom_ops/codelets_nms.cpp:24-125 and
#    custom_ops/postprocess.cc:139-290 (the same two steps behind odla_PostProcess)]
# --------------------------------------------------------------------------
YOLO_ANCHORS = (10, 13, 16, 30, 33, 23, 30, 61, 62, 45, 59, 119, 116, 90, 156, 198, 373, 326)
YOLO_ANCHOR_MASKS = ((6, 7, 8), (3, 4, 5), (0, 1, 2))   # heads with 13, 26 and 52 cells a side


def yolo_decode(img_w, img_h, head, mask):
    """head [1, 3*(5+C), dim, dim] -> rows [dim*dim*3, 5+C] in the reference's order
    (cell row, cell column, anchor): {y min, x min, y max, x max, objectness, class scores}.
    Arithmetic in the reference's mix of float and double: its locals are floats, the
    literals 416.0 and 2.0 make the sub-expressions around them double."""
    f32, f64 = np.float32, np.float64
    head = _f32(head)
    _, ch, dim, _ = head.shape
    C = ch // 3 - 5
    scale = f32(min(416.0 / img_h, 416.0 / img_w))
    # std::round rounds halves away from zero
    rnd = lambda v: f32(math.floor(abs(float(v)) + 0.5) * (1 if v >= 0 else -1))
    new_h, new_w = rnd(f32(img_h) * scale), rnd(f32(img_w) * scale)
    offset_h = f32(f64(f32(416) - new_h) / 2.0 / 416)
    offset_w = f32(f64(f32(416) - new_w) / 2.0 / 416)
    scale_h, scale_w = f32(416) / new_h, f32(416) / new_w
    t = np.exp(head[0].transpose(1, 2, 0).reshape(dim, dim, 3, 5 + C)).astype(f32)   # channels last, all through exp
    out = np.empty_like(t)
    gx = np.arange(dim, dtype=f32).reshape(1, dim, 1)
    gy = np.arange(dim, dtype=f32).reshape(dim, 1, 1)
    aw = np.array([YOLO_ANCHORS[2 * m] for m in mask], f32).reshape(1, 1, 3)
    ah = np.array([YOLO_ANCHORS[2 * m + 1] for m in mask], f32).reshape(1, 1, 3)
    dx = ((t[..., 0] / (t[..., 0] + f32(1))) + gx) / f32(dim)
    dx = (dx - offset_w) * scale_w
    dy = ((t[..., 1] / (t[..., 1] + f32(1))) + gy) / f32(dim)
    dy = (dy - offset_h) * scale_h
    dw = (t[..., 2] * aw) / f32(416) * scale_w
    dh = (t[..., 3] * ah) / f32(416) * scale_h
    out[..., 0] = ((dy.astype(f64) - dh.astype(f64) / 2.0) * img_h).astype(f32)
    out[..., 1] = ((dx.astype(f64) - dw.astype(f64) / 2.0) * img_w).astype(f32)
    out[..., 2] = ((dy.astype(f64) + dh.astype(f64) / 2.0) * img_h).astype(f32)
    out[..., 3] = ((dx.astype(f64) + dw.astype(f64) / 2.0) * img_w).astype(f32)
    conf = t[..., 4] / (t[..., 4] + f32(1))
    out[..., 4] = conf
    out[..., 5:] = t[..., 5:] / (t[..., 5:] + f32(1)) * conf[..., None]
    return out.reshape(dim * dim * 3, 5 + C)


def yolo_overlapping(sel, cur, iou_thr):
    f32 = np.float32
    y_top, x_left = max(sel[0], cur[0]), max(sel[1], cur[1])
    y_bot, x_right = min(sel[2], cur[2]), min(sel[3], cur[3])
    if x_right < x_left or y_bot < y_top:
        return False
    common = f32(x_right - x_left) * f32(y_bot - y_top)
    sel_area = f32(sel[2] - sel[0]) * f32(sel[3] - sel[1])
    cur_area = f32(cur[2] - cur[0]) * f32(cur[3] - cur[1])
    with np.errstate(divide="ignore", invalid="ignore"):
        return bool(common / f32(f32(sel_area + cur_area) - common) > f32(iou_thr))


def yolo_class_walk(rows, cls, iou_thr=0.45, score_thr=0.3):
    """Rows of one class that survive: score >= threshold, by falling score (equal
    scores by rising row - the reference's sort leaves their order open), a row is
    kept when it does not overlap the row kept last."""
    sc = rows[:, 5 + cls]
    cand = np.nonzero(sc >= np.float32(score_thr))[0]
    order = cand[np.lexsort((cand, -sc[cand].astype(np.float64)))]
    kept, sel = [], -1
    for i in order:
        if sel < 0 or not yolo_overlapping(rows[sel, :4], rows[i, :4], iou_thr):
            sel = i
            kept.append(int(i))
    return kept


def yolo_postprocess(img_w, img_h, bb13, bb26, bb52, iou_thr=0.45, score_thr=0.3):
    """-> (info [C, N/169, 5] zero padded, num [C]): the two results of odla_PostProcess.
    A class keeps at most N/169 rows (the reference writes past the end beyond that)."""
    rows = np.concatenate([yolo_decode(img_w, img_h, h, m)
                           for h, m in zip((bb13, bb26, bb52), YOLO_ANCHOR_MASKS)], axis=0)
    N, C = rows.shape[0], rows.shape[1] - 5
    cap = N // 169
    info = np.zeros((C, cap, 5), np.float32)
    num = np.zeros((C,), np.uint32)
    for c in range(C):
        kept = yolo_class_walk(rows, c, iou_thr, score_thr)[:cap]
        for k, i in enumerate(kept):
            info[c, k, :4] = rows[i, :4]
            info[c, k, 4] = rows[i, 5 + c]
        num[c] = len(kept)
    return info, num


# --------------------------------------------------------------------------
# Reference-style broadcast alignment  [ref: ODLA/platforms/dnnl/odla_dnnl.h:301-343]
# --------------------------------------------------------------------------
def align_like_reference(src_shape, dst_shape):
    sn, dn = len(src_shape), len(dst_shape)
    for j in range(dn - 1, sn - 2, -1):
        ok = all(dst_shape[j - k] == src_shape[sn - 1 - k] or dst_shape[j - k] == 1 or src_shape[sn - 1 - k] == 1
                 for k in range(sn))
        if ok:
            r = [1] * dn
            for k in range(sn):
                r[j - k] = src_shape[sn - 1 - k]
            return tuple(r)
    raise ValueError("shapes %s and %s do not broadcast" % (src_shape, dst_shape))


_erf = np.vectorize(math.erf, otypes=[np.float64])


# ---------------------------------------------------------------------------
# Operators along one axis.  Each follows the reference's loop over the tensor seen as
# [i][j][k] (j = the axis); the pins compare them with the operator examples the
# reference's own test names point at and with independent numpy formulations.

def _ijk(shape, axis):
    i = int(np.prod(shape[:axis], dtype=np.int64))
    k = int(np.prod(shape[axis + 1:], dtype=np.int64))
    return i, int(shape[axis]), k


def gather_elements(data, indices, axis):
    """out[i][j][k] = data[i][indices[i][j][k]][k]
    [ref: ODLA/platforms/dnnl/odla_dnnl.cc:509-522 do_gather_elements, :525-567].  A negative
    index counts from the end of the axis (the reference adds the extent BEHIND the axis
    instead, which is the same for the square operands of its test; the operator's
    definition is followed here); an index outside the axis is clamped into it (the reference
    reads outside the tensor)."""
    data = np.asarray(data)
    indices = np.asarray(indices)
    axis = axis % data.ndim
    di, dj, dk = _ijk(data.shape, axis)
    ii, ij, ik = _ijk(indices.shape, axis)
    flat = data.reshape(-1)
    idx = indices.reshape(ii, ij, ik).astype(np.int64)
    out = np.empty((ii, ij, ik), data.dtype)
    for i in range(ii):
        for j in range(ij):
            v = idx[i, j]
            v = np.where(v < 0, v + dj, v)
            v = np.clip(v, 0, dj - 1)
            out[i, j] = flat[i * dj * dk + v * dk + np.arange(ik)]
    return out.reshape(indices.shape)


def cumsum(x, axis, exclusive=False, reverse=False):
    """Running sum along the axis, accumulated in order in fp32
    [ref: ODLA/platforms/dnnl/odla_dnnl_statistics.cc:147-170 DoCumSum]."""
    x = np.asarray(x, np.float32)
    axis = axis % x.ndim
    ni, nj, nk = _ijk(x.shape, axis)
    src = x.reshape(ni, nj, nk)
    out = np.empty_like(src)
    acc = np.zeros((ni, nk), np.float32)
    order = range(nj - 1, -1, -1) if reverse else range(nj)
    for j in order:
        cur = src[:, j, :]
        out[:, j, :] = acc if exclusive else acc + cur
        acc = acc + cur
    return out.reshape(x.shape)


def hardmax(x, axis):
    """1 at the first largest element along the axis, 0 elsewhere
    [ref: ODLA/platforms/dnnl/odla_dnnl.cc:1688-1727 (ArgMax without return_last_index, then
    DoHardmax); odla_dnnl_statistics.cc:203-232 for the comparison: strictly greater replaces]."""
    x = np.asarray(x, np.float32)
    axis = axis % x.ndim
    ni, nj, nk = _ijk(x.shape, axis)
    src = x.reshape(ni, nj, nk)
    best = src[:, 0, :].copy()
    arg = np.zeros((ni, nk), np.int64)
    for j in range(1, nj):
        cur = src[:, j, :]
        take = cur > best
        best = np.where(take, cur, best)
        arg = np.where(take, j, arg)
    out = (np.arange(nj)[None, :, None] == arg[:, None, :]).astype(np.float32)
    return out.reshape(x.shape)


def compress(x, condition, axis, max_shape):
    """Slices of x along the axis whose condition is set, packed densely from the start of a
    buffer of the declared maximum shape ([outer][selected][inner], outer after outer); the
    rest is zero here and undefined in the reference.  axis None: x is taken as one flat axis
    [ref: ODLA/platforms/dnnl/odla_dnnl.cc:1280-1328]."""
    x = np.asarray(x)
    cond = np.asarray(condition).astype(bool).reshape(-1)
    n_out = int(np.prod(max_shape, dtype=np.int64))
    if axis is None:
        src = x.reshape(1, -1, 1)
        used = min(cond.size, n_out, src.shape[1])
    else:
        axis = axis % x.ndim
        src = x.reshape(_ijk(x.shape, axis))
        used = min(cond.size, src.shape[1])
    out = np.zeros(n_out, x.dtype)
    pos = 0
    for i in range(src.shape[0]):
        for j in range(used):
            if cond[j]:
                out[pos:pos + src.shape[2]] = src[i, j]
                pos += src.shape[2]
    return out.reshape(max_shape)


def shift(x, amount, left):
    """Logical shift of unsigned integers; a shift by the width or more gives 0 (undefined
    in the reference) [ref: ODLA/platforms/dnnl/odla_dnnl.cc:947-1010]."""
    x = np.asarray(x)
    amount = np.asarray(amount)
    assert x.dtype.kind == "u" and amount.dtype == x.dtype
    bits = x.dtype.itemsize * 8
    wide = x.astype(np.uint64)
    s = np.minimum(amount.astype(np.uint64), np.uint64(63))
    r = (wide << s) if left else (wide >> s)
    if bits < 64:
        r = r & np.uint64((1 << bits) - 1)
    r = np.where(amount.astype(np.uint64) >= bits, np.uint64(0), r)
    return r.astype(x.dtype)



class RefBuilder:
    """Eager evaluation of an ODLA graph on the CPU.

    Default: every operator in fp32 (the arithmetic of the reference CPU backend).

    Reduced-precision emulation, for networks that a device runs with 16-bit
    tensors: the same fp32 graph with values rounded to `storage` ("bf16" or
    "fp16") at chosen points, so that a device result can be told apart from
    what the storage type alone costs.
      emulate="operands"  only where a matrix unit must round: both operands of
          every Conv / Gemm (the reference's BF16_ACCURACY_MODE: operands cast,
          fp32 results, ODLA/platforms/dnnl/odla_dnnl.cc:1024-1026, 1780-1802);
          everything else stays fp32.
      emulate="stored"    at every tensor a 16-bit plan stores: arguments and
          constants when an operator reads them, every operator's result -
          except inside the chains one launch computes in fp32: Conv / Gemm with
          a per-channel constant Add / Sub / Mul / Div, one same-shape residual
          Add and one activation behind it (an Add behind the activation too),
          an Add whose only reader is a Softmax, a Softmax that is a graph
          output; the scores of an attention block with head size 64 and at most
          128 keys (q . k^T, scale and mask stay fp32 up to the Softmax, whose
          probabilities are stored).  Parameters that stay fp32 on the device (Conv / Gemm bias,
          LayerNorm and BatchNorm parameters) are not rounded.
    """

    _ACTS = ("relu", "leaky_relu", "clamp", "gelu", "sigmoid", "tanh")

    def __init__(self, feeds, emulate=None, storage=None):
        assert emulate in (None, "operands", "stored")
        assert (emulate is None) == (storage is None)
        self.feeds = feeds
        self.outputs = {}
        self.values = {}
        self.emulate, self.storage = emulate, storage
        self._open = {}      # id -> (array, stage): computed in fp32, not yet rounded to storage
        self._consts = {}    # id -> array handed out by const()
        self._rounded_const = {}
        if emulate == "stored":
            special = {"arg", "const", "output", "conv", "gemm", "batch_matmul", "add", "sub", "mul", "div",
                       "softmax", "layernorm", "batchnorm"} | set(self._ACTS)
            for attr in dir(type(self)):
                if attr.startswith("_") or attr in special or not callable(getattr(type(self), attr)):
                    continue
                setattr(self, attr, self._stored_op(getattr(self, attr)))

    def _name(self, name, v):
        if name:
            self.values[name] = v
        return v

    # reduced-precision emulation -------------------------------------------
    def _rs(self, a):
        return round_to_storage(a, self.storage)

    def _is_f32(self, v):
        return isinstance(v, np.ndarray) and v.dtype == np.float32

    def _closed(self, v):
        """`v` as an operator that reads stored tensors sees it."""
        if self.emulate != "stored" or not self._is_f32(v):
            return v
        ent = self._open.pop(id(v), None)
        if ent is not None:          # first reader outside its launch: the tensor is stored now
            v[...] = self._rs(v)
            return v
        if id(v) in self._consts:    # constants are converted to the storage type when uploaded
            r = self._rounded_const.get(id(v))
            if r is None:
                r = self._rounded_const[id(v)] = self._rs(v)
            return r
        return v

    def _store(self, v):
        """Result of an operator that writes a stored tensor."""
        if self.emulate == "stored" and self._is_f32(v) and v.flags.writeable:
            v[...] = self._rs(v)
        return v

    def _mark_open(self, v, stage):
        if self.emulate == "stored" and self._is_f32(v):
            self._open[id(v)] = (v, stage)
        return v

    def _stage(self, v):
        ent = self._open.get(id(v)) if isinstance(v, np.ndarray) else None
        return None if ent is None else ent[1]

    def _stored_op(self, f):
        def close(a):
            if isinstance(a, np.ndarray):
                return self._closed(a)
            if isinstance(a, (list, tuple)) and any(isinstance(e, np.ndarray) for e in a):
                return type(a)(close(e) for e in a)
            return a

        def run(*args, **kw):
            out = f(*[close(a) for a in args], **{k: close(a) for k, a in kw.items()})
            if isinstance(out, tuple):
                return tuple(self._store(o) for o in out)
            return self._store(out)
        return run

    def _operand(self, v):
        """A Conv / Gemm operand: rounded to the storage type in both emulations."""
        if self.emulate == "operands":
            return self._rs(v) if self._is_f32(np.asarray(v)) else v
        return self._closed(v)

    # graph inputs -----------------------------------------------------------
    def arg(self, name, shape, dtype=np.float32):
        v = np.ascontiguousarray(self.feeds[name], dtype=dtype)
        assert tuple(v.shape) == tuple(shape), (name, v.shape, shape)
        if self.emulate == "stored" and v.dtype == np.float32:
            v = self._rs(v)          # converted on its way into the plan
        return self._name(name, v)

    def const(self, name, array):
        v = np.ascontiguousarray(array)
        self._consts[id(v)] = v
        return self._name(name, v)

    def output(self, v, name):
        st = self._stage(v)
        if st is not None and st[0] == "softmax":
            self._open.pop(id(v))    # written in fp32 by the Softmax launch itself
        self.outputs[name] = self._closed(v)

    # heavy operators --------------------------------------------------------
    def conv(self, x, w, bias=None, stride=(1, 1), pad=(0, 0, 0, 0), dilation=(1, 1), group=1, name=None):
        y = conv2d(self._operand(x), self._operand(w), bias, stride, pad, dilation, group)
        return self._name(name, self._mark_open(y, ("acc", 1)))

    def gemm(self, a, b, c=None, ta=False, tb=False, alpha=1.0, beta=1.0, name=None):
        """alpha * op(A) op(B) + beta * C; leading dims of A are batch dims.
        [ref: odla_dnnl.cc:1730-1866]"""
        a, b = _f32(self._operand(a)), _f32(self._operand(b))
        if ta:
            a = np.swapaxes(a, -1, -2)
        if tb:
            b = np.swapaxes(b, -1, -2)
        y = np.matmul(a.astype(np.float64), b.astype(np.float64))
        y = y * float(alpha)
        stage = "acc"
        if c is not None and beta != 0:
            if id(c) not in self._consts:   # a run-time matrix rides as the launch's residual operand
                c = self._closed(c)
                stage = "res"
            y = y + float(beta) * _f32(c).astype(np.float64)
        y = y.astype(np.float32)
        # q . k^T of an attention block that a 16-bit plan runs as one launch (head size 64, up to
        # 128 keys in blocks of 32): the scores then never leave the launch, see _bin
        attn = (y.ndim == 4 and tb and not ta and c is None and a.shape[-1] == 64 and y.shape[-1] == y.shape[-2]
                and y.shape[-1] % 32 == 0 and y.shape[-1] <= 128)
        return self._name(name, self._mark_open(y, (stage, y.ndim - 1, attn)))

    def batch_matmul(self, a, b, ta=False, tb=False, name=None):
        """op(A) op(B) over matching leading batch dims [ref: ops/odla_ops_math.h:337-339;
        the code generator emits odla_Gemm with alpha = 1 for it, matmul.cc:45-70]"""
        return self.gemm(a, b, None, ta, tb, 1.0, 0.0, name=name)

    def maxpool(self, x, window, stride, pad, out_hw=None, name=None):
        return self._name(name, pool2d(x, window, stride, pad, out_hw, True))

    def avgpool(self, x, window, stride, pad, count_include_pad=False, out_hw=None, name=None):
        return self._name(name, pool2d(x, window, stride, pad, out_hw, False, count_include_pad))

    # element-wise -----------------------------------------------------------
    def _bin(self, f, a, b, name):
        a, b = (v if isinstance(v, np.ndarray) else np.asarray(v) for v in (a, b))
        ra, rb = a, b   # as given: identity matters for the emulation's bookkeeping
        if a.ndim != b.ndim:
            if a.ndim < b.ndim:
                a = a.reshape(align_like_reference(a.shape, b.shape))
            else:
                b = b.reshape(align_like_reference(b.shape, a.shape))
        if a.dtype.kind in "iu" and a.dtype == b.dtype:  # integer arithmetic [ref: odla_dnnl.cc:567-610]
            return self._name(name, f(a, b).astype(a.dtype))
        if self.emulate != "stored":
            return self._name(name, f(a.astype(np.float32), b.astype(np.float32)).astype(np.float32))
        # ---- 16-bit storage: what joins the launch of an open Conv / Gemm stays fp32
        out_shape = np.broadcast_shapes(a.shape, b.shape)
        for cur, other, c_al, o_al, lhs in ((ra, rb, a, b, True), (rb, ra, b, a, False)):
            st = self._stage(cur)
            if st is None or st[0] not in ("acc", "act") or tuple(c_al.shape) != tuple(out_shape):
                continue
            stage, ch = st[0], st[1]
            attn = len(st) > 2 and st[2]
            is_const = id(other) in self._consts
            per_channel = o_al.size == 1 or (o_al.size == out_shape[ch] and o_al.shape[ch] == o_al.size)
            res = None
            if stage == "acc" and is_const and per_channel and (
                    f is np.add or f is np.multiply or (f is np.subtract and lhs) or (f is np.divide and lhs and o_al.size == 1)):
                res, nxt = (f(c_al, o_al.astype(np.float32)) if lhs else f(o_al.astype(np.float32), c_al)), ("acc", ch, attn)
            elif f is np.add and not is_const and tuple(o_al.shape) == tuple(out_shape):
                o_cl = self._closed(other).reshape(o_al.shape)
                res, nxt = c_al + o_cl, (("res", ch) if stage == "acc" else ("done", ch))
            elif (f is np.add and not is_const and attn and stage == "acc" and o_al.ndim == 4
                  and o_al.shape[1] == 1 and o_al.shape[2] == 1 and o_al.shape[3] == out_shape[3]):
                # the mask of an attention block: added to fp32 scores inside the one launch
                o_cl = self._closed(other).reshape(o_al.shape)
                res, nxt = (c_al + o_cl).astype(np.float32), ("bin", ch)
            if res is not None:
                self._open.pop(id(cur), None)
                return self._name(name, self._mark_open(res.astype(np.float32), nxt))
        a = self._closed(ra).reshape(a.shape).astype(np.float32)
        b = self._closed(rb).reshape(b.shape).astype(np.float32)
        y = f(a, b).astype(np.float32)
        if f is np.add:   # an attention mask in front of a Softmax is added inside the Softmax launch
            return self._name(name, self._mark_open(y, ("bin", y.ndim - 1)))
        return self._name(name, self._store(y))

    def _act(self, f, x, name):
        """Activation: joins the launch of an open Conv / Gemm, else reads and writes stored tensors."""
        st = self._stage(x)
        if st is not None and st[0] in ("acc", "res"):
            self._open.pop(id(x))
            return self._name(name, self._mark_open(f(x), ("act" if st[0] == "acc" else "done", st[1])))
        return self._name(name, self._store(f(_f32(self._closed(x)))))

    def add(self, a, b, name=None): return self._bin(np.add, a, b, name)
    def sub(self, a, b, name=None): return self._bin(np.subtract, a, b, name)
    def mul(self, a, b, name=None): return self._bin(np.multiply, a, b, name)
    def div(self, a, b, name=None): return self._bin(np.divide, a, b, name)
    def max(self, a, b, name=None): return self._bin(np.maximum, a, b, name)
    def min(self, a, b, name=None): return self._bin(np.minimum, a, b, name)

    def relu(self, x, name=None): return self._act(lambda v: np.maximum(_f32(v), np.float32(0)), x, name)

    def leaky_relu(self, x, alpha, name=None):
        return self._act(lambda v: np.where(_f32(v) > 0, _f32(v), np.float32(alpha) * _f32(v)).astype(np.float32), x, name)

    def _unary64(self, f, x, name):
        return self._name(name, f(_f32(x).astype(np.float64)).astype(np.float32))

    def _act64(self, f, x, name):
        return self._act(lambda v: f(_f32(v).astype(np.float64)).astype(np.float32), x, name)

    def sigmoid(self, x, name=None): return self._act64(lambda v: 1.0 / (1.0 + np.exp(-v)), x, name)
    def tanh(self, x, name=None): return self._act64(np.tanh, x, name)
    def exp(self, x, name=None): return self._unary64(np.exp, x, name)
    def log(self, x, name=None): return self._unary64(np.log, x, name)
    def sqrt(self, x, name=None): return self._unary64(np.sqrt, x, name)
    def rsqrt(self, x, name=None): return self._unary64(lambda v: 1.0 / np.sqrt(v), x, name)
    def erf(self, x, name=None): return self._unary64(_erf, x, name)
    def abs(self, x, name=None): return self._name(name, np.abs(_f32(x)))
    def neg(self, x, name=None): return self._name(name, -_f32(x))
    def round(self, x, name=None): return self._name(name, np.rint(_f32(x)))

    def clamp(self, x, lo, hi, name=None):
        return self._act(lambda v: np.clip(_f32(v), np.float32(lo), np.float32(hi)), x, name)

    def gelu(self, x, approx=False, name=None):
        """[ref: odla_dnnl.cc:1868-1876]"""
        if approx:
            f = lambda v: 0.5 * v * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (v + 0.044715 * v ** 3)))
        else:
            f = lambda v: 0.5 * v * (1.0 + _erf(v / math.sqrt(2.0)))
        return self._act64(f, x, name)

    # normalisation ----------------------------------------------------------
    def batchnorm(self, x, mean, var, eps, scale=None, offset=None, scalar_scale=1.0, scalar_offset=0.0,
                  name=None):
        """y = scale * (x - mean) / sqrt(var + eps) + offset over channel axis 1.
        [ref: odla_dnnl.cc:1448-1524]"""
        st = self._stage(x)
        folded = st is not None and st[0] == "acc" and st[1] == 1   # folded into the Conv in front of it
        if folded:
            self._open.pop(id(x))
        else:
            x = self._closed(x)
        x = _f32(x)
        C = x.shape[1]
        sh = (1, C) + (1,) * (x.ndim - 2)
        g = np.full(C, scalar_scale, np.float64) if scale is None else _f32(scale).astype(np.float64)
        b = np.full(C, scalar_offset, np.float64) if offset is None else _f32(offset).astype(np.float64)
        m = g / np.sqrt(_f32(var).astype(np.float64) + float(np.float32(eps)))
        y = (x.astype(np.float64) * m.reshape(sh) + (b - _f32(mean).astype(np.float64) * m).reshape(sh)).astype(np.float32)
        return self._name(name, self._mark_open(y, ("acc", 1)) if folded else self._store(y))

    def layernorm(self, x, n_axes, eps, scale=None, offset=None, name=None):
        """Biased variance over the trailing n_axes axes, eps inside the root.
        [ref: lib/transforms/fusion.cc:296-313]"""
        x64 = _f32(self._closed(x)).astype(np.float64)
        ax = tuple(range(x64.ndim - n_axes, x64.ndim))
        mu = x64.mean(axis=ax, keepdims=True)
        var = ((x64 - mu) ** 2).mean(axis=ax, keepdims=True)
        y = (x64 - mu) / np.sqrt(var + float(np.float32(eps)))
        if scale is not None:
            y = y * _f32(scale).astype(np.float64).reshape(x64.shape[-n_axes:])
        if offset is not None:
            y = y + _f32(offset).astype(np.float64).reshape(x64.shape[-n_axes:])
        return self._name(name, self._store(y.astype(np.float32)))

    def softmax(self, x, axis=-1, log=False, name=None):
        """[ref: odla_dnnl.cc:1628-1669]; every negative axis means the last one."""
        st = self._stage(x)
        last = axis in (-1, np.ndim(x) - 1)
        if st is not None and last and (st[0] == "bin" or (st[0] == "acc" and len(st) > 2 and st[2])):
            self._open.pop(id(x))    # the Add in front ran inside this launch / the scores of an attention block
        else:
            x = self._closed(x)
        x64 = _f32(x).astype(np.float64)
        if axis < 0:
            axis = x64.ndim - 1
        z = x64 - x64.max(axis=axis, keepdims=True)
        e = np.exp(z)
        s = e.sum(axis=axis, keepdims=True)
        y = (z - np.log(s) if log else e / s).astype(np.float32)
        return self._name(name, self._mark_open(y, ("softmax", axis)))

    def reduce_mean(self, x, axes, keep_dims=True, name=None):
        """[ref: odla_dnnl_statistics.cc:20-46,111-117]"""
        y = _f32(x).astype(np.float64).mean(axis=tuple(axes), keepdims=bool(keep_dims))
        return self._name(name, y.astype(np.float32))

    def reduce_sum(self, x, axes, keep_dims=True, name=None):
        y = _f32(x).astype(np.float64).sum(axis=tuple(axes), keepdims=bool(keep_dims))
        return self._name(name, y.astype(np.float32))

    def reduce_max(self, x, axes, keep_dims=True, name=None):
        return self._name(name, _f32(x).max(axis=tuple(axes), keepdims=bool(keep_dims)))

    # wider operator surface ---------------------------------------------------
    # unary [ref: ODLA/platforms/dnnl/odla_dnnl_unary.cc:61-137; odla_dnnl.cc:409-430]
    def reciprocal(self, x, name=None): return self._unary64(lambda v: 1.0 / v, x, name)
    def ceil(self, x, name=None): return self._name(name, np.ceil(_f32(x)))
    def floor(self, x, name=None): return self._name(name, np.floor(_f32(x)))
    def sign(self, x, name=None): return self._name(name, np.sign(_f32(x)))
    def sin(self, x, name=None): return self._unary64(np.sin, x, name)
    def cos(self, x, name=None): return self._unary64(np.cos, x, name)
    def tan(self, x, name=None): return self._unary64(np.tan, x, name)
    def asin(self, x, name=None): return self._unary64(np.arcsin, x, name)
    def acos(self, x, name=None): return self._unary64(np.arccos, x, name)
    def atan(self, x, name=None): return self._unary64(np.arctan, x, name)
    def sinh(self, x, name=None): return self._unary64(np.sinh, x, name)
    def cosh(self, x, name=None): return self._unary64(np.cosh, x, name)
    def asinh(self, x, name=None): return self._unary64(np.arcsinh, x, name)
    def acosh(self, x, name=None): return self._unary64(np.arccosh, x, name)
    def atanh(self, x, name=None): return self._unary64(np.arctanh, x, name)

    def softplus(self, x, name=None):
        """log(exp(x) + 1)  [ref: odla_dnnl.cc:1671-1678]"""
        return self._unary64(lambda v: np.log(np.exp(v) + 1.0), x, name)

    def softsign(self, x, name=None):
        """x / (|x| + 1)  [ref: odla_dnnl.cc:1680-1687]"""
        return self._unary64(lambda v: v / (np.abs(v) + 1.0), x, name)

    def elu(self, x, alpha, name=None):
        """dnnl eltwise_elu: x > 0 ? x : alpha (exp(x) - 1)  [ref: odla_dnnl.cc:720-723]"""
        return self._unary64(lambda v: np.where(v > 0, v, alpha * np.expm1(v)), x, name)

    def selu(self, x, alpha, gamma, name=None):
        """gamma * elu(x, alpha)  [ref: odla_dnnl.cc:725-732]"""
        return self._unary64(lambda v: gamma * np.where(v > 0, v, alpha * np.expm1(v)), x, name)

    def celu(self, x, alpha, name=None):
        """relu(x) - relu(-elu(x / alpha, alpha))  [ref: odla_dnnl.cc:734-748]"""
        def f(v):
            e = np.where(v / alpha > 0, v / alpha, alpha * np.expm1(v / alpha))
            return np.maximum(v, 0.0) - np.maximum(-e, 0.0)
        return self._unary64(f, x, name)

    def hard_sigmoid(self, x, alpha, beta, name=None):
        """clamp(alpha x + beta, 0, 1)  [ref: odla_dnnl.cc:660-686]"""
        return self._unary64(lambda v: np.clip(alpha * v + beta, 0.0, 1.0), x, name)

    def thresholded_relu(self, x, alpha, name=None):
        """x > alpha ? x : 0  [ref: odla_dnnl.cc:750-774]"""
        x = _f32(x)
        return self._name(name, np.where(x > np.float32(alpha), x, np.float32(0)).astype(np.float32))

    def shrink(self, x, bias, lambd, name=None):
        """[ref: odla_dnnl.cc:776-789]"""
        x = _f32(x)
        b = np.float32(bias)
        y = np.where(x > lambd, x - b, np.where(x < -lambd, x + b, np.float32(0)))
        return self._name(name, y.astype(np.float32))

    def isnan(self, x, name=None): return self._name(name, np.isnan(_f32(x)))

    def isinf(self, x, pos=True, neg=True, name=None):
        """[ref: odla_dnnl_unary.cc:143-155,229-238]: neither flag means the negative test"""
        x = _f32(x)
        if pos and neg:
            return self._name(name, np.isinf(x))
        return self._name(name, np.isposinf(x) if pos else np.isneginf(x))

    def logical_not(self, x, name=None): return self._name(name, np.logical_not(np.asarray(x, bool)))

    # binary [ref: odla_dnnl_binary.cc:41-141]
    def _bin_typed(self, f, a, b, name, out_bool=False):
        a, b = np.asarray(a), np.asarray(b)
        assert a.dtype == b.dtype
        if a.ndim != b.ndim:
            if a.ndim < b.ndim:
                a = a.reshape(align_like_reference(a.shape, b.shape))
            else:
                b = b.reshape(align_like_reference(b.shape, a.shape))
        r = f(a, b)
        return self._name(name, r.astype(bool) if out_bool else r.astype(a.dtype))

    def pow(self, a, b, name=None):
        return self._bin_typed(lambda l, r: np.power(l.astype(np.float64), r.astype(np.float64)) if l.dtype.kind == "f" else np.power(l, r), a, b, name)

    def squared_difference(self, a, b, name=None): return self._bin_typed(lambda l, r: (l - r) * (l - r), a, b, name)

    def prelu(self, x, slope, name=None):
        """x < 0 ? x * slope : x  [ref: odla_dnnl.cc:698-718]"""
        return self._bin_typed(lambda l, r: np.where(l < 0, l * r, l), x, slope, name)

    def mod(self, a, b, fmod=False, name=None):
        """[ref: odla_dnnl_binary.cc:104-127]: quotient from a double division, floor (mod) or
        truncation through int32 (fmod), then l - r * quo in the operand type."""
        def f(l, r):
            t = l.astype(np.float64) / r.astype(np.float64)
            if fmod:
                q = np.where(t > 0, np.floor(t), np.ceil(t)).astype(np.int32).astype(l.dtype)
            else:
                q = np.floor(t).astype(l.dtype)
            return l - r * q
        return self._bin_typed(f, a, b, name)

    def equal(self, a, b, name=None): return self._bin_typed(np.equal, a, b, name, True)
    def not_equal(self, a, b, name=None): return self._bin_typed(np.not_equal, a, b, name, True)
    def less(self, a, b, name=None): return self._bin_typed(np.less, a, b, name, True)
    def less_equal(self, a, b, name=None): return self._bin_typed(np.less_equal, a, b, name, True)
    def greater(self, a, b, name=None): return self._bin_typed(np.greater, a, b, name, True)
    def greater_equal(self, a, b, name=None): return self._bin_typed(np.greater_equal, a, b, name, True)
    def logical_and(self, a, b, name=None): return self._bin_typed(np.logical_and, a, b, name, True)
    def logical_or(self, a, b, name=None): return self._bin_typed(np.logical_or, a, b, name, True)
    def logical_xor(self, a, b, name=None): return self._bin_typed(np.logical_xor, a, b, name, True)

    def mean(self, xs, name=None):
        """((x0 + x1) + x2 ...) / n  [ref: odla_dnnl.cc:2432-2441]"""
        acc = _f32(xs[0])
        for v in xs[1:]:
            acc = (acc + _f32(v)).astype(np.float32)
        return self._name(name, (acc / np.float32(len(xs))).astype(np.float32))

    def select(self, cond, a, b, name=None):
        """[ref: odla_dnnl.cc:2372-2430]"""
        cond, a, b = np.asarray(cond, bool), np.asarray(a), np.asarray(b)
        hi = max((cond, a, b), key=lambda v: v.ndim).shape
        al = [v if v.ndim == len(hi) else v.reshape(align_like_reference(v.shape, hi)) for v in (cond, a, b)]
        return self._name(name, np.where(al[0], al[1], al[2]).astype(a.dtype))

    # reductions [ref: odla_dnnl_statistics.cc:48-160]
    def _red64(self, f, x, axes, keep_dims, name):
        return self._name(name, f(_f32(x).astype(np.float64), tuple(axes), bool(keep_dims)).astype(np.float32))

    def reduce_min(self, x, axes, keep_dims=True, name=None):
        return self._name(name, _f32(x).min(axis=tuple(axes), keepdims=bool(keep_dims)))

    def reduce_prod(self, x, axes, keep_dims=True, name=None):
        return self._red64(lambda v, a, k: v.prod(axis=a, keepdims=k), x, axes, keep_dims, name)

    def reduce_sum_square(self, x, axes, keep_dims=True, name=None):
        return self._red64(lambda v, a, k: (v * v).sum(axis=a, keepdims=k), x, axes, keep_dims, name)

    def reduce_l1(self, x, axes, keep_dims=True, eps=0.0, name=None):
        """dnnl reduction_norm_lp_sum, p = 1: sum |x| + eps"""
        return self._red64(lambda v, a, k: np.abs(v).sum(axis=a, keepdims=k) + eps, x, axes, keep_dims, name)

    def reduce_l2(self, x, axes, keep_dims=True, eps=0.0, name=None):
        """dnnl reduction_norm_lp_sum, p = 2: sqrt(sum x^2 + eps)"""
        return self._red64(lambda v, a, k: np.sqrt((v * v).sum(axis=a, keepdims=k) + eps), x, axes, keep_dims, name)

    def reduce_log_sum(self, x, axes, keep_dims=True, name=None):
        return self._red64(lambda v, a, k: np.log(v.sum(axis=a, keepdims=k)), x, axes, keep_dims, name)

    def reduce_log_sum_exp(self, x, axes, keep_dims=True, name=None):
        def f(v, a, k):
            m = v.max(axis=a, keepdims=True)
            r = np.log(np.exp(v - m).sum(axis=a, keepdims=True)) + m
            return r if k else np.squeeze(r, axis=a)
        return self._red64(f, x, axes, keep_dims, name)

    def _arg(self, is_max, x, axis, keep_dims, last, dtype, name):
        """[ref: odla_dnnl_statistics.cc:203-232]: strict comparison keeps the first index,
        ``return_last_index`` also replaces on equality."""
        x = _f32(x)
        axis = axis % x.ndim
        v = x if is_max else -x
        if last:
            idx = x.shape[axis] - 1 - np.argmax(np.flip(v, axis=axis), axis=axis)
        else:
            idx = np.argmax(v, axis=axis)
        if keep_dims:
            idx = np.expand_dims(idx, axis)
        return self._name(name, idx.astype(dtype))

    def argmax(self, x, axis, keep_dims=True, last=False, dtype=np.int32, name=None):
        return self._arg(True, x, axis, keep_dims, last, dtype, name)

    def argmin(self, x, axis, keep_dims=True, last=False, dtype=np.int32, name=None):
        return self._arg(False, x, axis, keep_dims, last, dtype, name)

    def topk(self, x, k, axis, largest=True, index_dtype=np.int32, names=(None, None)):
        """Ordered, ties by ascending index (a stable sort of the keys)."""
        x = _f32(x)
        key = -x if largest else x
        order = np.argsort(key, axis=axis, kind="stable")
        idx = np.take(order, np.arange(k), axis=axis)
        vals = np.take_along_axis(x, idx, axis=axis)
        return self._name(names[0], vals), self._name(names[1], idx.astype(index_dtype))

    def pad(self, x, front, back, name=None):
        return self._name(name, np.pad(np.asarray(x), list(zip(front, back))))

    def tile(self, x, repeat, name=None): return self._name(name, np.tile(np.asarray(x), repeat))

    def broadcast_to(self, x, shape, name=None):
        x = np.asarray(x)
        if x.ndim != len(shape):
            x = x.reshape(align_like_reference(x.shape, shape))
        return self._name(name, np.ascontiguousarray(np.broadcast_to(x, shape)))

    def squeeze(self, x, axes, name=None):
        return self._name(name, np.squeeze(np.asarray(x), axis=tuple(axes) if len(axes) else None))

    def stack(self, xs, axis, name=None): return self._name(name, np.stack(xs, axis=axis))

    def lrn(self, x, window, alpha, beta, bias, name=None):
        """dnnl lrn_across_channels: x / (bias + alpha / size * sum_window x^2)^beta
        [ref: odla_dnnl.cc:1553-1581]"""
        x64 = _f32(x).astype(np.float64)
        half = (window - 1) // 2
        C = x64.shape[1]
        sq = x64 * x64
        acc = np.zeros_like(x64)
        for c in range(C):
            lo, hi = max(0, c - half), min(C - 1, c + half)
            acc[:, c] = sq[:, lo:hi + 1].sum(axis=1)
        y = x64 / np.power(bias + alpha / (2 * half + 1) * acc, beta)
        return self._name(name, y.astype(np.float32))

    def instance_norm(self, x, eps, scale=None, offset=None, scalar_scale=1.0, scalar_offset=0.0, name=None):
        """(x - mean) / sqrt(sum((x - mean)^2) / m + eps) * scale + offset over the spatial dims
        [ref: odla_dnnl.cc:1583-1626]"""
        x64 = _f32(x).astype(np.float64)
        ax = tuple(range(2, x64.ndim))
        d = x64 - x64.mean(axis=ax, keepdims=True)
        var = (d * d).mean(axis=ax, keepdims=True)
        shp = (1, -1) + (1,) * (x64.ndim - 2)
        g = np.asarray(scale, np.float64).reshape(shp) if scale is not None else scalar_scale
        b = np.asarray(offset, np.float64).reshape(shp) if offset is not None else scalar_offset
        return self._name(name, (d / np.sqrt(var + eps) * g + b).astype(np.float32))

    def deconv(self, x, w, bias=None, stride=(1, 1), pad=(0, 0, 0, 0), group=1, out_hw=None, name=None):
        return self._name(name, deconv2d(x, w, bias, stride, pad, group, out_hw))

    # data movement ----------------------------------------------------------
    def cast(self, x, dtype, name=None): return self._name(name, cast_like_reference(x, dtype))
    def concat(self, xs, axis, name=None): return self._name(name, np.concatenate(xs, axis=axis))
    def gather(self, x, idx, axis=0, name=None): return self._name(name, np.take(x, np.asarray(idx), axis=axis))
    def gather_elements(self, x, idx, axis=0, name=None): return self._name(name, gather_elements(x, idx, axis))
    def cumsum(self, x, axis, exclusive=False, reverse=False, name=None): return self._name(name, cumsum(x, axis, exclusive, reverse))
    def hardmax(self, x, axis=-1, name=None): return self._name(name, hardmax(x, axis))
    def compress(self, x, cond, axis, max_shape, name=None): return self._name(name, compress(x, cond, axis, max_shape))
    def shift(self, x, amount, left=True, name=None): return self._name(name, shift(x, amount, left))
    def reshape(self, x, shape, name=None): return self._name(name, np.reshape(x, shape))
    def transpose(self, x, perm, name=None): return self._name(name, np.ascontiguousarray(np.transpose(x, perm)))

    def slice(self, x, start, end, stride=None, name=None):
        stride = stride or [1] * len(start)
        sl = tuple(slice(s, e, t) for s, e, t in zip(start, end, stride))
        return self._name(name, np.ascontiguousarray(x[sl]))

    def resize_nearest(self, x, out_hw, name=None):
        """src index = floor(dst * in / out).  [ref: ODLA/platforms/odla_eigen.cc:602-632]"""
        x = np.asarray(x)
        H, W = x.shape[2], x.shape[3]
        hi = (np.arange(out_hw[0]) * H) // out_hw[0]
        wi = (np.arange(out_hw[1]) * W) // out_hw[1]
        return self._name(name, np.ascontiguousarray(x[:, :, hi][:, :, :, wi]))

    def resize_linear(self, x, out_hw, name=None):
        """Bilinear, pixel centres at half-integers, edges clamped: source coordinate
        s = (o + 0.5) * in / out - 0.5, neighbours floor(s) and floor(s) + 1 clamped
        into the image, weights 1 - frac and frac.  The reference calls oneDNN's
        resampling_linear for ODLA_LINEAR whatever coordinate mode is passed
        [ref: ODLA/platforms/dnnl/odla_dnnl.cc:1526-1551]; oneDNN (1.x / 2.x, not in
        the reference tree) documents exactly this formula for its linear algorithm."""
        x = np.asarray(x, np.float64)
        H, W = x.shape[2], x.shape[3]

        def taps(o_n, i_n):
            s = (np.arange(o_n, dtype=np.float64) + 0.5) * (i_n / o_n) - 0.5
            s = np.maximum(s, 0.0)
            i0 = np.minimum(np.floor(s).astype(np.int64), i_n - 1)
            i1 = np.minimum(i0 + 1, i_n - 1)
            return i0, i1, s - i0

        h0, h1, ah = taps(out_hw[0], H)
        w0, w1, aw = taps(out_hw[1], W)
        ah = ah.reshape(1, 1, -1, 1)
        aw = aw.reshape(1, 1, 1, -1)
        top = x[:, :, h0][:, :, :, w0] * (1 - aw) + x[:, :, h0][:, :, :, w1] * aw
        bot = x[:, :, h1][:, :, :, w0] * (1 - aw) + x[:, :, h1][:, :, :, w1] * aw
        return self._name(name, np.ascontiguousarray((top * (1 - ah) + bot * ah).astype(np.float32)))

    # quantisation -----------------------------------------------------------
    def quantize(self, x, scale, zp=None, axis=-1, signed=False, name=None):
        """[ref: odla_dnnl_quantization.cc:61-90]"""
        x = _f32(x)
        scale = _f32(scale).reshape(-1)
        sh = [1] * x.ndim
        if scale.size > 1:
            sh[axis] = scale.size
        t = np.rint(x / scale.reshape(sh))
        if zp is not None:
            t = t + np.asarray(zp, dtype=np.float32).reshape(sh)
        lo, hi, dt = (-128, 127, np.int8) if signed else (0, 255, np.uint8)
        return self._name(name, np.clip(t, lo, hi).astype(dt))

    def dequantize(self, q, scale, zp=None, axis=-1, name=None, zp_dtype=None):
        """[ref: odla_dnnl_quantization.cc:33-59]"""
        q = np.asarray(q)
        scale = _f32(scale).reshape(-1)
        sh = [1] * q.ndim
        if scale.size > 1:
            sh[axis] = scale.size
        f = q.astype(np.float32)
        if zp is not None:
            f = f - np.asarray(zp, dtype=np.float32).reshape(sh)
        return self._name(name, (f * scale.reshape(sh)).astype(np.float32))

    def yolo_postprocess(self, img_w, img_h, bb13, bb26, bb52, name=None):
        info, num = yolo_postprocess(int(np.asarray(img_w).reshape(-1)[0]), int(np.asarray(img_h).reshape(-1)[0]),
                                     bb13, bb26, bb52)
        name = name or ""
        return self._name(name + "0", info), self._name(name + "1", num)

    def nms(self, boxes, scores, max_out, iou_thr, score_thr, name=None):
        return self._name(name, nms(boxes, scores, max_out, iou_thr, score_thr))
