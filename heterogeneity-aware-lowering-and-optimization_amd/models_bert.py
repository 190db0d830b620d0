"""C4: BERT-base encoder as the ODLA call sequence an ONNX export lowers to.

Embedding gather + position/type embeddings + LayerNorm, then per layer:
QKV projections (Gemm + bias), head split (Reshape/Transpose), scaled
Q.K^T (batched Gemm, Div), additive mask, Softmax, P.V (batched Gemm), head
merge, output projection + residual + LayerNorm, FFN (Gemm + bias + GELU,
Gemm + bias) + residual + LayerNorm.  Weights ~ N(0, 0.02), synthetic.
"""
import math

import numpy as np

BERT_BASE = dict(layers=12, hidden=768, heads=12, ffn=3072, vocab=30522, max_pos=512)
LN_EPS = 1e-12


def bert_weights(cfg=BERT_BASE, seed=42):
    rng = np.random.default_rng(seed)
    H, F = cfg["hidden"], cfg["ffn"]

    def n(*shape):
        return (rng.standard_normal(shape) * 0.02).astype(np.float32)

    w = {"emb.word": n(cfg["vocab"], H), "emb.pos": n(cfg["max_pos"], H), "emb.type": n(2, H),
         "emb.ln.g": np.ones(H, np.float32), "emb.ln.b": np.zeros(H, np.float32)}
    for l in range(cfg["layers"]):
        p = "l%d." % l
        for nm in ("q", "k", "v", "o"):
            w[p + nm + ".w"] = n(H, H)
            w[p + nm + ".b"] = n(H)
        w[p + "ln1.g"] = (1.0 + n(H)).astype(np.float32)
        w[p + "ln1.b"] = n(H)
        w[p + "f1.w"], w[p + "f1.b"] = n(H, F), n(F)
        w[p + "f2.w"], w[p + "f2.b"] = n(F, H), n(H)
        w[p + "ln2.g"] = (1.0 + n(H)).astype(np.float32)
        w[p + "ln2.b"] = n(H)
    return w


def bert_input(batch, seq, cfg=BERT_BASE, seed=1234):
    rng = np.random.default_rng(seed)
    return {"input_ids": rng.integers(0, cfg["vocab"], size=(batch, seq)).astype(np.int32),
            "attention_mask": np.ones((batch, 1, 1, seq), np.float32)}


def build_bert(b, w, batch, seq, cfg=BERT_BASE):
    H, nh = cfg["hidden"], cfg["heads"]
    dh = H // nh
    ids = b.arg("input_ids", (batch, seq), np.int32)
    mask = b.arg("attention_mask", (batch, 1, 1, seq))
    # additive mask: (1 - mask) * -10000
    mbias = b.mul(b.sub(b.const("one", np.ones((1,), np.float32)), mask, name="inv_mask"),
                  b.const("neg", np.full((1,), -10000.0, np.float32)), name="mask_bias")
    x = b.gather(b.const("emb.word", w["emb.word"]), ids, 0, name="word_emb")          # [B,S,H]
    pos = b.const("emb.pos_s", np.ascontiguousarray(w["emb.pos"][:seq] + w["emb.type"][0]))  # [S,H]
    x = b.add(x, pos, name="emb_sum")
    x = b.layernorm(x, 1, LN_EPS, b.const("emb.ln.g", w["emb.ln.g"]), b.const("emb.ln.b", w["emb.ln.b"]), name="emb_ln")
    for l in range(cfg["layers"]):
        p = "l%d." % l

        def proj(inp, nm):
            y = b.gemm(inp, b.const(p + nm + ".w", w[p + nm + ".w"]), None, False, False, 1.0, 0.0, name=p + nm + ".mm")
            return b.add(y, b.const(p + nm + ".b", w[p + nm + ".b"]), name=p + nm)

        def heads(t, nm):
            t = b.reshape(t, (batch, seq, nh, dh), name=p + nm + ".r")
            return b.transpose(t, (0, 2, 1, 3), name=p + nm + ".t")                       # [B,nh,S,dh]

        q, k, v = heads(proj(x, "q"), "q"), heads(proj(x, "k"), "k"), heads(proj(x, "v"), "v")
        s = b.gemm(q, k, None, False, True, 1.0, 0.0, name=p + "qk")                       # [B,nh,S,S]
        s = b.div(s, b.const(p + "scale", np.full((1,), math.sqrt(dh), np.float32)), name=p + "qk.s")
        s = b.add(s, mbias, name=p + "qk.m")
        pr = b.softmax(s, -1, name=p + "prob")
        c = b.gemm(pr, v, None, False, False, 1.0, 0.0, name=p + "ctx")                     # [B,nh,S,dh]
        c = b.reshape(b.transpose(c, (0, 2, 1, 3), name=p + "ctx.t"), (batch, seq, H), name=p + "ctx.r")
        a = b.add(proj(c, "o"), x, name=p + "res1")
        x = b.layernorm(a, 1, LN_EPS, b.const(p + "ln1.g", w[p + "ln1.g"]), b.const(p + "ln1.b", w[p + "ln1.b"]), name=p + "ln1")
        f = b.gemm(x, b.const(p + "f1.w", w[p + "f1.w"]), None, False, False, 1.0, 0.0, name=p + "f1.mm")
        f = b.gelu(b.add(f, b.const(p + "f1.b", w[p + "f1.b"]), name=p + "f1"), False, name=p + "gelu")
        f = b.gemm(f, b.const(p + "f2.w", w[p + "f2.w"]), None, False, False, 1.0, 0.0, name=p + "f2.mm")
        f = b.add(b.add(f, b.const(p + "f2.b", w[p + "f2.b"]), name=p + "f2"), x, name=p + "res2")
        x = b.layernorm(f, 1, LN_EPS, b.const(p + "ln2.g", w[p + "ln2.g"]), b.const(p + "ln2.b", w[p + "ln2.b"]), name=p + "ln2")
    b.output(x, "hidden")


def bert_gflop_per_sequence(seq, cfg=BERT_BASE):
    H, F, nh = cfg["hidden"], cfg["ffn"], cfg["heads"]
    mac = cfg["layers"] * (4 * seq * H * H + 2 * seq * H * F + 2 * nh * seq * seq * (H // nh))
    return 2.0 * mac / 1e9
