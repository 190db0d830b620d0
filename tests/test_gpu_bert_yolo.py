"""Whole-graph parity for the BERT encoder (config 4) and YOLOv3 + NMS (config 3)
at reduced sizes the CPU oracle evaluates in seconds."""
import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, max_rel_err, run_hip, run_ref, run_ref_emulated

pytestmark = pytest.mark.gpu

SMALL_BERT = dict(layers=2, hidden=128, heads=4, ffn=256, vocab=1000, max_pos=64)


@pytest.mark.parametrize("mode", ["fp32", "bf16"])
def test_small_bert_encoder(mode):
    announce("small bert %s" % mode)
    mb = entry.load().models_bert
    w = mb.bert_weights(SMALL_BERT, seed=3)
    feeds = mb.bert_input(4, 32, SMALL_BERT, seed=4)
    feeds["attention_mask"][1, 0, 0, 20:] = 0.0   # one padded sequence exercises the additive mask
    build = lambda b: mb.build_bert(b, w, 4, 32, SMALL_BERT)
    got = run_hip(build, feeds, bf16=(mode == "bf16"))["hidden"]
    want = run_ref(build, feeds)["hidden"]
    assert got.shape == want.shape == (4, 32, 128)
    if mode == "fp32":
        assert max_rel_err(got, want) <= 1e-4
    else:
        # bf16 storage (8 significant bits) of O(1) LayerNorm outputs
        assert np.max(np.abs(got - want)) <= 2e-2 * max(1.0, float(np.max(np.abs(want))))


def test_small_bert_encoder_bf16_accuracy_mode():
    """BF16_ACCURACY_MODE against the oracle that rounds only the Gemm operands; a padded sequence
    exercises the mask, which stays fp32 in this mode."""
    announce("small bert bf16, accuracy mode")
    mb = entry.load().models_bert
    w = mb.bert_weights(SMALL_BERT, seed=3)
    feeds = mb.bert_input(4, 32, SMALL_BERT, seed=4)
    feeds["attention_mask"][1, 0, 0, 20:] = 0.0
    build = lambda b: mb.build_bert(b, w, 4, 32, SMALL_BERT)
    got = run_hip(build, feeds, bf16="accuracy")["hidden"]
    want = run_ref(build, feeds)["hidden"]
    emu = run_ref_emulated(build, feeds, "operands", "bf16")["hidden"]
    floor, e, d = (float(np.max(np.abs(a - b))) for a, b in ((emu, want), (got, want), (got, emu)))
    announce("small bert bf16 accuracy mode: operands floor %.3e, GPU vs fp32 %.3e, GPU vs emulated %.3e" % (floor, e, d))
    assert e <= 2e-2 and e <= 1.5 * floor and d <= floor


def test_small_yolov3_heads_and_detections():
    """Heads within tolerance; decode + NMS on the same head tensors gives identical detections."""
    announce("small yolov3")
    my = entry.load().models_yolo
    width, classes, hw, batch = 0.125, 5, 96, 2
    feeds = my.yolov3_input(batch, hw, seed=5)
    w0 = my.yolov3_weights(width, classes, seed=6)
    build0 = lambda b: my.build_yolov3(b, w0, batch, hw, width, classes, postprocess=False)
    heads0 = run_hip(build0, feeds)
    scales, bias = my.calibrate_heads([heads0["head%d" % i] for i in range(3)], classes, target=0.02)
    w = my.yolov3_weights(width, classes, seed=6, head_bias=bias, head_scale=scales)
    build = lambda b: my.build_yolov3(b, w, batch, hw, width, classes, postprocess=True, max_out=20)
    got = run_hip(build, feeds)
    want = run_ref(build, feeds)
    for i in range(3):
        assert max_rel_err(got["head%d" % i], want["head%d" % i]) <= 1e-4, i
    # fp16 network
    got16 = run_hip(build, feeds, fp16=True)
    for i in range(3):
        k = "head%d" % i
        assert np.max(np.abs(got16[k] - want[k])) <= 2e-2 * max(1.0, float(np.max(np.abs(want[k])))), i

    # post-processing on identical inputs (the fp16 network's heads): fp32 decode + NMS
    pfeeds = {"head%d" % i: got16["head%d" % i] for i in range(3)}
    pbuild = lambda b: my.build_yolo_postprocess(b, batch, hw, classes, max_out=20)
    pg = run_hip(pbuild, pfeeds)
    pw = run_ref(pbuild, pfeeds)
    assert max_rel_err(pg["boxes"], pw["boxes"]) <= 1e-5
    assert max_rel_err(pg["scores"], pw["scores"]) <= 1e-5
    n_det = int((pw["detections"][:, 2] >= 0).sum())
    assert n_det > 0, "calibration produced no detections"
    # NMS itself on bit-identical inputs: feed the GPU's decoded boxes/scores to the oracle rule
    ref = entry.load_oracle()
    want_det = ref.nms(pg["boxes"], pg["scores"], 20, 0.45, 0.3)
    assert np.array_equal(pg["detections"], want_det)


def test_bert_encoder_random_sizes():
    """Encoders of random (small) sizes: sequence lengths that are no multiple of any
    tile, one head, heads of 8 .. 64 features, batch 1 - the masked-softmax fusion, the
    split-K rule and the batched attention GEMMs have size conditions of their own."""
    mb = entry.load().models_bert
    r = np.random.default_rng(17)
    for i in range(14):
        heads = int(r.choice([1, 2, 3, 4, 12]))
        dh = int(r.choice([8, 16, 32, 64]))
        cfg = dict(layers=int(r.integers(1, 3)), hidden=heads * dh, heads=heads, ffn=heads * dh * int(r.choice([1, 2, 4])),
                   vocab=int(r.integers(50, 500)), max_pos=160)
        batch, seq = int(r.integers(1, 5)), int(r.choice([1, 5, 16, 33, 64, 128, 150]))
        announce("bert #%d %s batch %d seq %d" % (i, cfg, batch, seq))
        w = mb.bert_weights(cfg, seed=100 + i)
        feeds = mb.bert_input(batch, seq, cfg, seed=200 + i)
        if seq > 3:
            feeds["attention_mask"][0, 0, 0, seq - seq // 3:] = 0.0
        build = lambda b: mb.build_bert(b, w, batch, seq, cfg)
        want = run_ref(build, feeds)["hidden"]
        got = run_hip(build, feeds)["hidden"]
        assert max_rel_err(got, want) <= 2e-4, (i, cfg, batch, seq)
        got = run_hip(build, feeds, bf16=True)["hidden"]
        assert np.max(np.abs(got - want)) <= 3e-2 * max(1.0, float(np.max(np.abs(want)))), (i, cfg, batch, seq)
