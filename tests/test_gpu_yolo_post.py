"""odla_PostProcess (YOLOv3 decode + per-class suppression walk of one image) on the
GPU against the oracle's restatement of the reference's post-processor."""
import numpy as np
import pytest

import __graft_entry__ as entry
from util import announce, run_hip, run_ref

pytestmark = pytest.mark.gpu


def heads_for(seed, classes, dims, obj_bias, cls_bias, spread=1.0, size_bias=0.0, geo_spread=None):
    r = np.random.default_rng(seed)
    heads = []
    for d in dims:
        h = (r.standard_normal((1, 3 * (5 + classes), d, d)) * spread).astype(np.float32)
        t = h.reshape(1, 3, 5 + classes, d, d)
        if geo_spread is not None:
            t[:, :, 0:4] *= geo_spread / spread
        t[:, :, 2:4] += size_bias          # larger boxes overlap more often
        t[:, :, 4] += obj_bias
        t[:, :, 5:] += cls_bias
        heads.append(h)
    return heads


def build_for(heads):
    def build(b):
        w = b.arg("src_w", (1,), np.uint32)
        h = b.arg("src_h", (1,), np.uint32)
        hs = [b.arg("bb%d" % i, x.shape) for i, x in enumerate(heads)]
        info, num = b.yolo_postprocess(w, h, hs[0], hs[1], hs[2], name="post")
        b.output(info, "post0")
        b.output(num, "post1")
    return build


def check(got, want, classes):
    assert got["post1"].dtype == np.uint32 and got["post1"].shape == (classes,)
    assert np.array_equal(got["post1"], want["post1"])
    assert got["post0"].shape == want["post0"].shape
    scale = max(float(np.abs(want["post0"]).max()), 1.0)
    assert float(np.abs(got["post0"] - want["post0"]).max()) <= 1e-4 * scale
    for c in range(classes):
        assert np.all(got["post0"][c, int(got["post1"][c]):] == 0)


@pytest.mark.parametrize("size", [(416, 416), (640, 480), (375, 1242)])
def test_postprocess_coco_shape(size):
    classes = 80
    announce("yolo postprocess 80 classes, image %dx%d" % size)
    heads = heads_for(11, classes, (13, 26, 52), obj_bias=-1.5, cls_bias=-3.2, spread=1.5, size_bias=2.5, geo_spread=0.3)
    feeds = {"src_w": np.array([size[0]], np.uint32), "src_h": np.array([size[1]], np.uint32)}
    feeds.update({"bb%d" % i: h for i, h in enumerate(heads)})
    got = run_hip(build_for(heads), feeds, repeats=2)
    want = run_ref(build_for(heads), feeds)
    kept = want["post1"].astype(int)
    assert kept.sum() > 2000 and kept.max() < 63     # a real walk, below the row limit
    check(got, want, classes)


def test_postprocess_crowded_classes_stop_at_their_rows():
    classes = 3
    announce("yolo postprocess crowded")
    heads = heads_for(12, classes, (13, 26, 52), obj_bias=3.0, cls_bias=1.0, spread=0.7)
    heads[0].reshape(1, 3, 5 + classes, 13, 13)[:, :, 7] -= 30.0     # nothing of the last class passes in head 0 ...
    heads[1].reshape(1, 3, 5 + classes, 26, 26)[:, :, 7] -= 30.0
    heads[2].reshape(1, 3, 5 + classes, 52, 52)[:, :, 7] -= 30.0     # ... or anywhere
    feeds = {"src_w": np.array([500], np.uint32), "src_h": np.array([333], np.uint32)}
    feeds.update({"bb%d" % i: h for i, h in enumerate(heads)})
    got = run_hip(build_for(heads), feeds)
    want = run_ref(build_for(heads), feeds)
    assert want["post1"].tolist() == [63, 63, 0]
    check(got, want, classes)


def test_postprocess_small_heads_fp16_and_equal_scores():
    """Other head sizes (rows per class = boxes / 169), half-precision plan (the heads
    reach the operator as fp16 values), and repeated cells, whose equal scores are
    ordered by box index."""
    classes = 2
    announce("yolo postprocess small fp16")
    heads = heads_for(13, classes, (4, 8, 16), obj_bias=1.0, cls_bias=0.0)
    for h in heads:
        h[...] = h.astype(np.float16).astype(np.float32)
        h[:, :, 1] = h[:, :, 0]                  # second cell row = first: equal scores, far-apart boxes
    feeds = {"src_w": np.array([416], np.uint32), "src_h": np.array([416], np.uint32)}
    feeds.update({"bb%d" % i: h for i, h in enumerate(heads)})
    want = run_ref(build_for(heads), feeds)
    assert want["post0"].shape == (classes, 3 * (16 + 64 + 256) // 169, 5)
    for kw in ({}, {"fp16": True}):
        got = run_hip(build_for(heads), feeds, **kw)
        check(got, want, classes)


def test_postprocess_rejects_bad_operands():
    odla = entry.load().odla
    hb = odla.HipBuilder()
    try:
        w = hb.arg("w", (1,), np.uint32)
        h = hb.arg("h", (1,), np.uint32)
        ok = [hb.arg("a%d" % i, (1, 255, d, d)) for i, d in enumerate((13, 26, 52))]
        two = hb.arg("two", (2, 255, 13, 13))
        odd = hb.arg("odd", (1, 254, 13, 13))
        fw = hb.arg("fw", (1,))
        with pytest.raises(odla.OdlaError):
            hb.yolo_postprocess(w, h, two, ok[1], ok[2])        # one image at a time
        with pytest.raises(odla.OdlaError):
            hb.yolo_postprocess(w, h, odd, ok[1], ok[2])        # channels differ / not 3 * (5 + classes)
        with pytest.raises(odla.OdlaError):
            hb.yolo_postprocess(fw, h, ok[0], ok[1], ok[2])     # the image size is an integer
    finally:
        hb.destroy()
