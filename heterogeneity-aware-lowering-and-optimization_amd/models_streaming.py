"""Bandwidth-bound operators at the shapes they have in the benchmark
configurations, one graph of independent branches.  Used by
``bench.py --workload streaming_fp16`` to price every streaming kernel against
the HBM roofline: algorithmic bytes = (elements read + elements written) x
element size, each tensor once.
"""
import numpy as np


def _n(*s):
    return int(np.prod(s))


def streaming_cases(es=2):
    """[(launch name, description, algorithmic bytes)]; `es` = bytes per element of the storage type."""
    a = _n(256, 256, 56, 56)
    q = _n(256, 64, 56, 56)
    return [
        ("unary:s_relu", "ReLU [256,256,56,56]", 2 * a * es),
        ("binary:s_add", "Add (residual) [256,256,56,56]", 3 * a * es),
        ("bn:s_bn", "BatchNorm scale-shift [256,256,56,56]", 2 * a * es),
        ("maxpool:s_maxpool", "MaxPool 3x3 s2 p1 [256,64,112,112]", (_n(256, 64, 112, 112) + _n(256, 64, 56, 56)) * es),
        ("reduce:s_gap", "global AvgPool (ReduceMean) [256,2048,7,7]", (_n(256, 2048, 7, 7) + _n(256, 2048)) * es),
        ("avgpool:s_avgpool", "AveragePool 2x2 s2 [256,256,56,56]", (a + a // 4) * es),
        ("softmax:s_softmax_cls", "Softmax [8192,1000]", 2 * _n(8192, 1000) * es),
        ("softmax:s_softmax_att", "Softmax [64,12,128,128]", 2 * _n(64, 12, 128, 128) * es),
        ("layernorm:s_ln", "LayerNorm [64,128,768]", 2 * _n(64, 128, 768) * es),
        ("unary:s_gelu", "GELU(erf) [64,128,3072]", 2 * _n(64, 128, 3072) * es),
        ("resize:s_up", "Resize nearest 2x [16,256,52,52]", 5 * _n(16, 256, 52, 52) * es),
        ("concat:s_cat", "Concat channels [16,256,104,104]+[16,128,104,104]", 2 * _n(16, 384, 104, 104) * es),
        ("transpose:s_heads", "Transpose [64,128,12,64]->[64,12,128,64]", 2 * _n(64, 128, 768) * es),
        ("quantize:s_quant", "Quantize -> u8 [256,64,56,56]", q * (es + 1)),
        ("dequantize:s_dequant", "Dequantize u8 -> float [256,64,56,56]", q * (es + 1)),
        ("to_nhwc:img", "NCHW fp32 -> channels-last [256,3,224,224], C padded to 16 B",
         _n(256, 3, 224, 224) * 4 + _n(256, 224, 224) * 16),
        ("to_nchw:s_out_src", "channels-last -> NCHW fp32 [16,255,52,52]", _n(16, 255, 52, 52) * (es + 4)),
    ]


def streaming_input(seed=1234):
    rng = np.random.default_rng(seed)
    f = lambda *s: rng.standard_normal(s, dtype=np.float32)
    return {"a": f(256, 256, 56, 56), "p": f(256, 64, 112, 112), "g": f(256, 2048, 7, 7), "sc": f(8192, 1000),
            "sa": f(64, 12, 128, 128), "ln": f(64, 128, 768), "ge": f(64, 128, 3072), "u": f(16, 256, 52, 52),
            "k": f(16, 128, 104, 104), "h": f(64, 128, 12, 64), "q": f(256, 64, 56, 56), "img": f(256, 3, 224, 224),
            "o": f(16, 255, 52, 52)}


def build_streaming(b):
    """Every branch starts with a cheap producer so that the measured operator
    reads a device tensor in the library's internal type and layout, and ends in
    a small reduction so that only a few bytes leave the device."""
    rng = np.random.default_rng(5)

    def sink(v, name, rank):
        if rank == 4:
            r = b.reduce_mean(v, (2, 3), True, name=name + "_sink")
        else:
            r = b.reduce_max(v, tuple(range(1, rank)), False, name=name + "_sink")
        b.output(r, name)

    def channels_last(v, name):
        """1x1 max-pool: the cheapest operator that moves a tensor to channels-last."""
        return b.maxpool(v, (1, 1), (1, 1), (0, 0, 0, 0), name=name)

    a = channels_last(b.arg("a", (256, 256, 56, 56)), "a_cl")
    a2 = b.neg(a, name="a_neg")
    sink(b.relu(a, name="s_relu"), "o_relu", 4)
    sink(b.add(a, a2, name="s_add"), "o_add", 4)
    C = 256
    bn = b.batchnorm(a2, b.const("bn_m", rng.standard_normal(C).astype(np.float32)),
                     b.const("bn_v", (rng.random(C) + 0.5).astype(np.float32)), 1e-5,
                     b.const("bn_g", rng.standard_normal(C).astype(np.float32)),
                     b.const("bn_b", rng.standard_normal(C).astype(np.float32)), name="s_bn")
    sink(bn, "o_bn", 4)
    p = channels_last(b.arg("p", (256, 64, 112, 112)), "p_cl")
    sink(b.maxpool(p, (3, 3), (2, 2), (1, 1, 1, 1), name="s_maxpool"), "o_maxpool", 4)
    g = channels_last(b.arg("g", (256, 2048, 7, 7)), "g_cl")
    b.output(b.reduce_mean(g, (2, 3), True, name="s_gap"), "o_gap")
    sink(b.avgpool(a, (2, 2), (2, 2), (0, 0, 0, 0), name="s_avgpool"), "o_avgpool", 4)
    sc = b.neg(b.arg("sc", (8192, 1000)), name="sc_neg")
    sink(b.softmax(sc, -1, name="s_softmax_cls"), "o_sm_cls", 2)
    sa = b.neg(b.arg("sa", (64, 12, 128, 128)), name="sa_neg")
    sink(b.reshape(b.softmax(sa, -1, name="s_softmax_att"), (64, 12 * 128 * 128), name="sa_flat"), "o_sm_att", 2)
    ln = b.neg(b.arg("ln", (64, 128, 768)), name="ln_neg")
    y = b.layernorm(ln, 1, 1e-12, b.const("ln_g", rng.standard_normal(768).astype(np.float32)),
                    b.const("ln_b", rng.standard_normal(768).astype(np.float32)), name="s_ln")
    sink(y, "o_ln", 3)
    ge = b.neg(b.arg("ge", (64, 128, 3072)), name="ge_neg")
    sink(b.gelu(ge, False, name="s_gelu"), "o_gelu", 3)
    u = channels_last(b.arg("u", (16, 256, 52, 52)), "u_cl")
    up = b.resize_nearest(u, (104, 104), name="s_up")
    k = channels_last(b.arg("k", (16, 128, 104, 104)), "k_cl")
    sink(b.concat([up, k], 1, name="s_cat"), "o_cat", 4)
    h = b.neg(b.arg("h", (64, 128, 12, 64)), name="h_neg")
    sink(b.reshape(b.transpose(h, (0, 2, 1, 3), name="s_heads"), (64, 12 * 128 * 64), name="h_flat"), "o_heads", 2)
    q = b.reshape(b.neg(b.arg("q", (256, 64, 56, 56)), name="q_neg"), (256, 64 * 56 * 56), name="q_flat")
    qq = b.quantize(q, [0.05], [128], name="s_quant")
    sink(b.dequantize(qq, [0.05], [128], name="s_dequant"), "o_quant", 2)
    img = b.arg("img", (256, 3, 224, 224))
    w1 = b.const("w_in", (rng.standard_normal((8, 3, 1, 1)) * 0.1).astype(np.float32))
    sink(b.conv(img, w1, None, name="s_in"), "o_in", 4)
    o = channels_last(b.arg("o", (16, 255, 52, 52)), "o_cl")
    b.output(b.neg(o, name="s_out_src"), "o_out")   # output conversion: channels-last -> NCHW fp32
