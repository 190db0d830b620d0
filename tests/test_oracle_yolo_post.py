"""Pins of the oracle's YOLOv3 post-processor (yolo_decode, yolo_class_walk,
yolo_postprocess) without a GPU: closed forms of the decode, the same boxes from the
sigmoid / exp graph of models_yolo (a separate formulation of the same decode),
and hand-worked cases of the per-class walk that tell "compare with the box kept
last" (models/vision/detection/yolo/yolov3_postproc.cc:142-150 of the reference
tree) from the usual greedy suppression.
"""
import numpy as np
import pytest

import __graft_entry__ as entry


@pytest.fixture(scope="module")
def ref():
    return entry.load_oracle()


def sigmoid64(v):
    return 1.0 / (1.0 + np.exp(-np.asarray(v, np.float64)))


def test_decode_closed_form_square_image(ref):
    r = np.random.default_rng(0)
    C, dim = 4, 5
    head = r.standard_normal((1, 3 * (5 + C), dim, dim)).astype(np.float32)
    rows = ref.yolo_decode(416, 416, head, (3, 4, 5))
    assert rows.shape == (dim * dim * 3, 5 + C)
    t = head[0].astype(np.float64).reshape(3, 5 + C, dim, dim)
    anchors = [(30, 61), (62, 45), (59, 119)]
    for gy in range(dim):
        for gx in range(dim):
            for a in range(3):
                v = t[a, :, gy, gx]
                cx = (sigmoid64(v[0]) + gx) / dim * 416
                cy = (sigmoid64(v[1]) + gy) / dim * 416
                w = np.exp(v[2]) * anchors[a][0]
                h = np.exp(v[3]) * anchors[a][1]
                want = [cy - h / 2, cx - w / 2, cy + h / 2, cx + w / 2, sigmoid64(v[4])]
                want += list(sigmoid64(v[5:]) * sigmoid64(v[4]))
                got = rows[(gy * dim + gx) * 3 + a]
                assert np.allclose(got, want, rtol=2e-5, atol=2e-4), (gy, gx, a)


def test_decode_letterbox(ref):
    # a 832 x 416 source image fills the network input's width and half of its
    # height: x scales by 2 per network pixel, y by 2 after removing the 104-pixel bar
    C, dim = 1, 2
    head = np.zeros((1, 3 * (5 + C), dim, dim), np.float32)      # sigmoid 0.5, exp 1
    rows = ref.yolo_decode(832, 416, head, (0, 1, 2))
    # cell (0,0), anchor 0 = (10, 13): centre (0.25, 0.25) of the network input
    cx = 0.25 * 832
    cy = (0.25 - 0.25) * 2 * 416            # offset_h = (416 - 208) / 2 / 416 = 0.25, scale_h = 2
    w = 10 / 416 * 832
    h = 13 / 416 * 2 * 416
    assert np.allclose(rows[0, :4], [cy - h / 2, cx - w / 2, cy + h / 2, cx + w / 2], rtol=1e-6, atol=1e-4)
    assert np.allclose(rows[0, 4:], [0.5, 0.25])


def test_decode_agrees_with_the_graph_formulation(ref):
    """models_yolo builds the decode from Sigmoid / Exp / Mul / Add nodes (boxes as
    fractions of the network input, anchors outermost); on a 416 x 416 image both
    must give the same boxes and scores."""
    my = entry.load().models_yolo
    r = np.random.default_rng(1)
    classes, hw = 3, 64
    heads = [r.standard_normal((1, 3 * (5 + classes), hw // s, hw // s)).astype(np.float32) for s in (32, 16, 8)]
    rb = ref.RefBuilder({"head%d" % i: h for i, h in enumerate(heads)})
    my.build_yolo_postprocess(rb, 1, hw, classes, max_out=5)
    boxes, scores = rb.outputs["boxes"][0], rb.outputs["scores"][0]      # [nb,4] fractions, [C,nb]
    first = 0
    for h, mask in zip(heads, ref.YOLO_ANCHOR_MASKS):
        g = h.shape[2]
        # the anchors are given in pixels of a 416 network input; the graph divides them by its own input size
        rows = ref.yolo_decode(416, 416, h, mask).reshape(g * g, 3, 5 + classes)
        for a in range(3):
            sl = slice(first + a * g * g, first + (a + 1) * g * g)
            centre_w = (boxes[sl][:, [1, 3]].sum(axis=1) / 2) * 416
            centre_r = rows[:, a, [1, 3]].sum(axis=1) / 2
            assert np.allclose(centre_r, centre_w, rtol=1e-5, atol=1e-3)
            centre_w = (boxes[sl][:, [0, 2]].sum(axis=1) / 2) * 416
            centre_r = rows[:, a, [0, 2]].sum(axis=1) / 2
            assert np.allclose(centre_r, centre_w, rtol=1e-5, atol=1e-3)
            # sizes: the graph's anchors are fractions of hw, the reference's of 416
            size_w = (boxes[sl][:, 3] - boxes[sl][:, 1]) * hw
            size_r = rows[:, a, 3] - rows[:, a, 1]
            assert np.allclose(size_r, size_w, rtol=1e-4, atol=1e-3)
            assert np.allclose(rows[:, a, 5:].T, scores[:, sl], rtol=1e-5, atol=1e-6)
        first += 3 * g * g


def rows_of(boxes, scores):
    rows = np.zeros((len(boxes), 6), np.float32)
    rows[:, :4] = boxes
    rows[:, 5] = scores
    return rows


def test_walk_compares_with_the_box_kept_last_only(ref):
    A = [0, 0, 10, 10]
    B = [0, 20, 10, 30]        # clear of A
    Cb = [0, 2, 10, 12]        # IoU with A = 80 / 120, with B = 0
    rows = rows_of([A, B, Cb], [0.9, 0.8, 0.7])
    # greedy suppression would drop the third box (it overlaps the first); the
    # reference compares it with the second, which was kept last, and keeps it
    assert ref.yolo_class_walk(rows, 0) == [0, 1, 2]
    # in the order A, C, B the third box meets A first and goes
    rows = rows_of([A, B, Cb], [0.9, 0.7, 0.8])
    assert ref.yolo_class_walk(rows, 0) == [0, 1]


def test_walk_thresholds(ref):
    A = [0, 0, 10, 10]
    half = [0, 5, 10, 15]      # IoU 50 / 150 = 1/3: below 0.45, kept
    most = [0, 2, 10, 12]      # IoU 2/3: suppressed
    assert ref.yolo_class_walk(rows_of([A, half], [0.9, 0.8]), 0) == [0, 1]
    assert ref.yolo_class_walk(rows_of([A, most], [0.9, 0.8]), 0) == [0]
    # the score threshold is inclusive, and nothing below it takes part
    assert ref.yolo_class_walk(rows_of([A, [50, 50, 60, 60], [80, 80, 90, 90]], [0.9, 0.3, 0.29999]), 0) == [0, 1]
    # equal scores: by rising row
    got = ref.yolo_class_walk(rows_of([[50, 50, 60, 60], A, [70, 70, 80, 80]], [0.5, 0.9, 0.5]), 0)
    assert got == [1, 0, 2]
    # degenerate box (zero area) against itself: 0 / 0 is not above the threshold
    assert ref.yolo_class_walk(rows_of([[5, 5, 5, 5], [5, 5, 5, 5]], [0.9, 0.8]), 0) == [0, 1]


def test_postprocess_shapes_padding_and_capacity(ref):
    r = np.random.default_rng(2)
    classes = 2
    heads = [(r.standard_normal((1, 3 * (5 + classes), d, d)) * 0.5).astype(np.float32) for d in (13, 26, 52)]
    for h in heads:
        h[:, 4::5 + classes] += 3.0    # objectness
        h[:, 5::5 + classes] += 2.0    # class 0 passes often, class 1 rarely
        h[:, 6::5 + classes] -= 2.0
    info, num = ref.yolo_postprocess(640, 480, *heads)
    N = 3 * (13 * 13 + 26 * 26 + 52 * 52)
    assert info.shape == (classes, N // 169, 5) and num.shape == (classes,) and num.dtype == np.uint32
    assert num[0] == N // 169                   # far more candidates than rows: the class stops at its capacity
    for c in range(classes):
        k = int(num[c])
        assert np.all(info[c, k:] == 0)
        s = info[c, :k, 4]
        assert np.all(s >= np.float32(0.3)) and np.all(np.diff(s) <= 0)
        for i in range(1, k):                   # neighbours in the result never overlap above the threshold
            assert not ref.yolo_overlapping(info[c, i - 1, :4], info[c, i, :4], 0.45)
