"""CPU oracle of the int8 ResNet plan -- TEST INFRASTRUCTURE ONLY.

Evaluates the post-training-quantised ResNet-50-shaped network with explicit
integer arithmetic (u8 activations, s8 weights, int32 accumulators) following
the fusion rules of the int8 plan:
  conv (+ ReLU)          -> requantise to the table entry of the last fused value
  conv + residual + ReLU -> likewise, ONE requantisation: the residual's levels
                            enter the fused multiply-add of the requantisation
                            (ref.qconv with `residual`)
  max-pool               -> keeps levels and its input's scale
  global average pool    -> fp32 (the head has no table entries)
PARITY UNPINNED by the reference for the requantisation formula (the reference
has no int8 convolution); the int32 accumulators are exact integer arithmetic.
"""
import numpy as np

import odla_ref as ref


def run(w, feeds, qp, stages, stem, batch, hw, record=None):
    """qp: name -> (scale, zp).  Returns dict with 'logits', 'prob' (fp32)."""
    def rec(name, q, acc=None):
        if record is not None:
            record[name] = q
            if acc is not None:
                record[name + "/acc"] = acc

    x = ref.quantize_act(feeds["input"], *qp["input"])
    cur_qp = qp["input"]
    rec("input", x)

    def conv(xq, x_qp, name, stride, pad, out_name, relu, residual=None):
        q, acc = ref.qconv(xq, x_qp, w[name + ".w"], w[name + ".b"], qp[out_name], (stride, stride),
                           (pad, pad, pad, pad), relu, residual)
        rec(out_name, q, acc)
        return q

    x = conv(x, cur_qp, "stem", 2, 3, "stem.relu", True)
    cur_qp = qp["stem.relu"]
    # max pooling on levels: monotone, keeps scale and zero point
    x = ref.pool2d(x.astype(np.float32), (3, 3), (2, 2), (1, 1, 1, 1), None, True).astype(np.uint8)
    rec("pool1", x)
    for si, (mid, blocks, stride) in enumerate(stages):
        for bi in range(blocks):
            s = stride if bi == 0 else 1
            p = "l%db%d" % (si + 1, bi)
            if bi == 0:
                ident = conv(x, cur_qp, p + "ds", s, 0, p + "ds", False)
                ident_qp = qp[p + "ds"]
            else:
                ident, ident_qp = x, cur_qp
            y = conv(x, cur_qp, p + "c1", 1, 0, p + "c1.relu", True)
            y = conv(y, qp[p + "c1.relu"], p + "c2", s, 1, p + "c2.relu", True)
            x = conv(y, qp[p + "c2.relu"], p + "c3", 1, 0, p + "out", True, (ident, ident_qp))
            cur_qp = qp[p + "out"]
    # global average pool -> fp32: ((sum q - n*zp) / n) * scale
    n = x.shape[2] * x.shape[3]
    isum = x.astype(np.int64).sum(axis=(2, 3)) - n * cur_qp[1]
    gap = ((isum.astype(np.float32) / np.float32(n)) * np.float32(cur_qp[0])).astype(np.float32)
    rb = ref.RefBuilder({})
    logits = rb.gemm(gap, w["fc.w"], w["fc.b"].reshape(1, -1))
    return {"logits": logits, "prob": rb.softmax(logits, -1), "gap": gap}
