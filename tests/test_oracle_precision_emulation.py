"""Pins of the oracle's reduced-precision emulation (``RefBuilder(emulate=..., storage=...)``).

The rounding helper is pinned by hand-listed ties (round half to even), the ends of
the range, and an independent library's conversions (torch's bfloat16 / float16).
The two emulations are pinned by spelling out, operator by operator in numpy, where
each of them rounds - small graphs chosen so that every rule is exercised: operands
only; the fp32 chain of one launch (bias, residual, activation); constants that stay
fp32; the mask Add in front of a Softmax; a Softmax that is a graph output.
"""
import numpy as np
import pytest
import torch

import __graft_entry__ as entry


@pytest.fixture(scope="module")
def ref():
    return entry.load_oracle()


def test_round_to_storage_ties_and_range(ref):
    r = ref.round_to_storage
    # bf16 keeps 8 significant bits: neighbours of 1 are 2^-7 apart
    x = np.array([1.0, 1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8, 1 + 2.0 ** -8 + 2.0 ** -20, -1 - 2.0 ** -8, 3.0e38, 1e-40], np.float32)
    want = np.array([1.0, 1.0, 1 + 2.0 ** -6, 1 + 2.0 ** -7, -1.0, 3.0e38, 1e-40], np.float32)
    got = r(x, "bf16")
    assert np.array_equal(got[:5], want[:5])
    assert got[5] == np.float32(torch.tensor(3.0e38).to(torch.bfloat16).float().item())
    # fp16 keeps 11: neighbours of 1 are 2^-10 apart; 65520 is the first value that rounds to infinity
    x = np.array([1.0, 1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11, 65504.0, 65519.0, 65520.0, -70000.0, 2.0 ** -25], np.float32)
    want = np.array([1.0, 1.0, 1 + 2.0 ** -9, 65504.0, 65504.0, np.inf, -np.inf, 0.0], np.float32)
    assert np.array_equal(r(x, "fp16"), want)
    assert np.isnan(r(np.array([np.nan], np.float32), "bf16")[0])


@pytest.mark.parametrize("storage,tdt", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_round_to_storage_against_library_conversion(ref, storage, tdt):
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(200000) * s for s in (1e-6, 1e-2, 1.0, 300.0, 6e4)]).astype(np.float32)
    want = torch.from_numpy(x).to(tdt).to(torch.float32).numpy()
    assert np.array_equal(ref.round_to_storage(x, storage), want)


def _rs(ref, a, st):
    return ref.round_to_storage(np.asarray(a, np.float32), st)


@pytest.mark.parametrize("storage", ["bf16", "fp16"])
def test_operands_emulation_rounds_only_matrix_operands(ref, storage):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((6, 40)).astype(np.float32)
    w = rng.standard_normal((40, 24)).astype(np.float32)
    bias = rng.standard_normal(24).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(24)).astype(np.float32)
    rb = ref.RefBuilder({"x": x}, emulate="operands", storage=storage)
    xv = rb.arg("x", x.shape)
    y = rb.add(rb.gemm(xv, rb.const("w", w), None, False, False, 1.0, 0.0), rb.const("b", bias))
    z = rb.layernorm(rb.gelu(y), 1, 1e-5, rb.const("g", g), None)
    rb.output(z, "z")
    # spelled out: operands rounded, everything else fp32
    y0 = (_rs(ref, x, storage).astype(np.float64) @ _rs(ref, w, storage).astype(np.float64)).astype(np.float32) + bias
    plain = ref.RefBuilder({})
    z0 = plain.layernorm(plain.gelu(y0), 1, 1e-5, g, None)
    assert np.array_equal(rb.outputs["z"], z0)
    # and it differs from the fp32 graph (the rounding is really there)
    plain2 = ref.RefBuilder({"x": x})
    y1 = plain2.add(plain2.gemm(x, w, None, False, False, 1.0, 0.0), bias)
    assert not np.array_equal(y1, y0)


@pytest.mark.parametrize("storage", ["bf16", "fp16"])
def test_stored_emulation_conv_chain_rounds_once(ref, storage):
    """conv + bias + residual + ReLU is one launch: fp32 inside, one rounding at its store;
    the argument, the kernel and the residual are read as stored tensors, the bias is fp32."""
    rng = np.random.default_rng(7)
    x = rng.standard_normal((2, 8, 6, 6)).astype(np.float32)
    w = (rng.standard_normal((8, 8, 3, 3)) * 0.2).astype(np.float32)
    b = rng.standard_normal(8).astype(np.float32)
    rb = ref.RefBuilder({"x": x}, emulate="stored", storage=storage)
    xv = rb.arg("x", x.shape)
    c = rb.conv(xv, rb.const("w", w), rb.const("b", b), (1, 1), (1, 1, 1, 1))
    y = rb.relu(rb.add(c, xv))
    out = rb.maxpool(y, (2, 2), (2, 2), (0, 0, 0, 0))
    rb.output(out, "y")
    xr, wr = _rs(ref, x, storage), _rs(ref, w, storage)
    y0 = _rs(ref, np.maximum(ref.conv2d(xr, wr, b, (1, 1), (1, 1, 1, 1)) + xr, 0), storage)
    want = ref.pool2d(y0, (2, 2), (2, 2), (0, 0, 0, 0), None, True)
    assert np.array_equal(rb.outputs["y"], want)
    # rounding the convolution before the add (two launches) would give another result
    two = _rs(ref, np.maximum(_rs(ref, ref.conv2d(xr, wr, b, (1, 1), (1, 1, 1, 1)), storage) + xr, 0), storage)
    assert not np.array_equal(two, y0)


def test_stored_emulation_attention_rules(ref):
    """Scaled scores are stored; the mask Add runs inside the Softmax launch; probabilities
    are stored; a Softmax that is a graph output is written in fp32."""
    st = "bf16"
    rng = np.random.default_rng(9)
    q = rng.standard_normal((2, 3, 8, 16)).astype(np.float32)
    k = rng.standard_normal((2, 3, 8, 16)).astype(np.float32)
    mask = np.where(rng.random((2, 1, 1, 8)) < 0.3, -10000.0, 0.0).astype(np.float32)
    rb = ref.RefBuilder({"q": q, "k": k, "m": mask}, emulate="stored", storage=st)
    qv, kv, mv = rb.arg("q", q.shape), rb.arg("k", k.shape), rb.arg("m", mask.shape)
    s = rb.div(rb.gemm(qv, kv, None, False, True, 1.0, 0.0), rb.const("scale", np.full((1,), 4.0, np.float32)))
    p = rb.softmax(rb.add(s, mv), -1)
    ctx = rb.gemm(p, kv, None, False, False, 1.0, 0.0)
    rb.output(ctx, "ctx")
    rb.output(rb.softmax(ctx, -1), "sm_out")
    qr, kr, mr = _rs(ref, q, st), _rs(ref, k, st), _rs(ref, mask, st)
    s0 = _rs(ref, (qr.astype(np.float64) @ np.swapaxes(kr, -1, -2).astype(np.float64)).astype(np.float32) / np.float32(4.0), st)
    plain = ref.RefBuilder({})
    p0 = _rs(ref, plain.softmax(s0 + mr, -1), st)
    ctx0 = _rs(ref, (p0.astype(np.float64) @ kr.astype(np.float64)).astype(np.float32), st)
    assert np.array_equal(rb.outputs["ctx"], ctx0)
    sm0 = plain.softmax(ctx0, -1)
    assert np.array_equal(rb.outputs["sm_out"], sm0)          # fp32: not rounded
    assert not np.array_equal(_rs(ref, sm0, st), sm0)


def test_stored_emulation_attention_block_keeps_scores_fp32(ref):
    """Head size 64 and a multiple of 32 keys (at most 128): the block is one launch in a 16-bit
    plan, so scale, mask and Softmax see fp32 scores; the probabilities are stored."""
    st = "bf16"
    rng = np.random.default_rng(10)
    q = rng.standard_normal((2, 2, 32, 64)).astype(np.float32)
    k = rng.standard_normal((2, 2, 32, 64)).astype(np.float32)
    v = rng.standard_normal((2, 2, 32, 64)).astype(np.float32)
    mask = np.where(rng.random((2, 1, 1, 32)) < 0.3, -10000.0, 0.0).astype(np.float32)
    rb = ref.RefBuilder({"q": q, "k": k, "v": v, "m": mask}, emulate="stored", storage=st)
    qv, kv, vv, mv = (rb.arg(n, a.shape) for n, a in (("q", q), ("k", k), ("v", v), ("m", mask)))
    s = rb.div(rb.gemm(qv, kv, None, False, True, 1.0, 0.0), rb.const("scale", np.full((1,), 8.0, np.float32)))
    ctx = rb.gemm(rb.softmax(rb.add(s, mv), -1), vv, None, False, False, 1.0, 0.0)
    rb.output(ctx, "ctx")
    qr, kr, vr, mr = (_rs(ref, a, st) for a in (q, k, v, mask))
    s0 = (qr.astype(np.float64) @ np.swapaxes(kr, -1, -2).astype(np.float64)).astype(np.float32) / np.float32(8.0)
    plain = ref.RefBuilder({})
    p0 = _rs(ref, plain.softmax(s0 + mr, -1), st)
    ctx0 = _rs(ref, (p0.astype(np.float64) @ vr.astype(np.float64)).astype(np.float32), st)
    assert np.array_equal(rb.outputs["ctx"], ctx0)
    # with stored (rounded) scores the result differs: the rule matters
    p1 = _rs(ref, plain.softmax(_rs(ref, s0, st) + mr, -1), st)
    assert not np.array_equal(p1, p0)


def test_stored_emulation_keeps_normalisation_parameters_fp32(ref):
    st = "bf16"
    rng = np.random.default_rng(11)
    x = rng.standard_normal((4, 32)).astype(np.float32)
    g = (1 + 0.01 * rng.standard_normal(32)).astype(np.float32)   # not representable in bf16
    b = (0.01 * rng.standard_normal(32)).astype(np.float32)
    rb = ref.RefBuilder({"x": x}, emulate="stored", storage=st)
    y = rb.layernorm(rb.arg("x", x.shape), 1, 1e-5, rb.const("g", g), rb.const("b", b))
    rb.output(y, "y")
    plain = ref.RefBuilder({})
    assert np.array_equal(rb.outputs["y"], _rs(ref, plain.layernorm(_rs(ref, x, st), 1, 1e-5, g, b), st))
    # a constant read by an ordinary operator is a stored tensor
    rb2 = ref.RefBuilder({"x": x}, emulate="stored", storage=st)
    z = rb2.mul(rb2.arg("x", x.shape), rb2.const("g", g))
    rb2.output(z, "z")
    assert np.array_equal(rb2.outputs["z"], _rs(ref, _rs(ref, x, st) * _rs(ref, g, st), st))


def test_default_oracle_is_unchanged_by_the_emulation_code(ref, ):
    """emulate=None: plain fp32, nothing is tracked."""
    rng = np.random.default_rng(13)
    x = rng.standard_normal((3, 20)).astype(np.float32)
    w = rng.standard_normal((20, 10)).astype(np.float32)
    rb = ref.RefBuilder({"x": x})
    y = rb.relu(rb.add(rb.gemm(rb.arg("x", x.shape), rb.const("w", w), None, False, False, 1.0, 0.0), rb.const("b", np.ones(10, np.float32))))
    rb.output(y, "y")
    want = np.maximum((x.astype(np.float64) @ w.astype(np.float64)).astype(np.float32) + np.float32(1), 0)
    assert np.array_equal(rb.outputs["y"], want) and not rb._open
