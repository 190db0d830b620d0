"""C3: YOLOv3 (Darknet-53 backbone, FPN with nearest 2x up-sampling and channel
concat, three 255-channel heads) and its post-processing (sigmoid/exp decode +
batched NMS) as ODLA call sequences.  BatchNorm is folded into the
convolutions; weights are He-normal, synthetic.

Decode follows the reference's post-processor
(models/vision/detection/yolo/yolov3_postproc.cc:34-88 of the reference tree):
centre = (sigmoid(t_xy) + grid) / grid_size, size = exp(t_wh) * anchor / input,
score = sigmoid(obj) * sigmoid(class); boxes are handed to odla_NMS as
(y1, x1, y2, x2) corners, scores as [N, classes, boxes].
"""
import numpy as np

ANCHORS = [(10, 13), (16, 30), (33, 23), (30, 61), (62, 45), (59, 119), (116, 90), (156, 198), (373, 326)]
MASKS = [(6, 7, 8), (3, 4, 5), (0, 1, 2)]   # head at stride 32, 16, 8
NUM_CLASSES = 80
LEAKY = 0.1


def _c(v, width):
    return max(8, int(v * width) // 8 * 8)


def yolov3_conv_specs(width=1.0, classes=NUM_CLASSES):
    """[(name, cout, cin, k, stride, leaky)] in execution order; 75 convolutions."""
    specs = []
    c = lambda v: _c(v, width)
    nout = 3 * (5 + classes)

    def add(name, cout, cin, k, s=1, act=True):
        specs.append((name, cout, cin, k, s, act))

    add("d0", c(32), 3, 3)
    cin = c(32)
    for si, (ch, blocks) in enumerate([(64, 1), (128, 2), (256, 8), (512, 8), (1024, 4)]):
        add("d%d.down" % (si + 1), c(ch), cin, 3, 2)
        cin = c(ch)
        for bi in range(blocks):
            add("d%d.b%d.c1" % (si + 1, bi), c(ch // 2), cin, 1)
            add("d%d.b%d.c2" % (si + 1, bi), cin, c(ch // 2), 3)
    route_c = {1: c(1024), 2: c(512), 3: c(256)}
    prev_branch = None
    for hi, ch in enumerate([512, 256, 128], start=1):
        if hi == 1:
            cin = route_c[1]
        else:
            add("h%d.lat" % hi, c(ch), prev_branch, 1)
            cin = c(ch) + route_c[hi]
        for j in range(5):
            cout = c(ch) if j % 2 == 0 else c(ch * 2)
            add("h%d.c%d" % (hi, j), cout, cin, 1 if j % 2 == 0 else 3)
            cin = cout
        prev_branch = cin
        add("h%d.c5" % hi, c(ch * 2), cin, 3)
        add("h%d.out" % hi, nout, c(ch * 2), 1, 1, False)
    return specs


RESIDUAL_GAMMA = 0.5   # folded BatchNorm gain of the second conv of every residual block


def yolov3_weights(width=1.0, classes=NUM_CLASSES, seed=42, head_bias=0.0, head_scale=(1.0, 1.0, 1.0)):
    """He-normal weights (gain for LeakyReLU 0.1) with the BatchNorm of every
    convolution folded in: gamma 1 (RESIDUAL_GAMMA on the last conv of a residual
    block, which keeps the activations of the 23 un-normalised residual sums
    inside the fp16 range), beta 0, mean 0, var 1.  `head_scale` rescales the three
    detection convolutions (so that their logits are O(1)); `head_bias` is added
    to the objectness and class logits."""
    rng = np.random.default_rng(seed)
    w = {}
    hi = 0
    for name, cout, cin, k, s, act in yolov3_conv_specs(width, classes):
        std = np.sqrt(2.0 / ((1 + LEAKY ** 2) * cin * k * k)) if act else np.sqrt(1.0 / (cin * k * k))
        if name.startswith("d") and name.endswith(".c2"):
            std *= RESIDUAL_GAMMA
        if not act:
            std *= head_scale[hi]
        w[name + ".w"] = (rng.standard_normal((cout, cin, k, k)) * std).astype(np.float32)
        w[name + ".b"] = np.zeros(cout, np.float32)
        if not act:
            b = w[name + ".b"].reshape(3, 5 + classes)
            b[:, 4:] = head_bias      # objectness and class logits
            hi += 1
    return w


def calibrate_heads(head_logits, classes=NUM_CLASSES, target=0.01, thr=0.3):
    """From the head outputs of a run with head_scale 1 / head_bias 0: the scales
    that bring each head's logits to unit standard deviation and the bias that
    lets about `target` of the (box, class) scores pass `thr`."""
    scales = tuple(float(1.0 / max(np.std(h), 1e-12)) for h in head_logits)
    bias = choose_head_bias([h * s for h, s in zip(head_logits, scales)], classes, target, thr)
    return scales, bias


def yolov3_input(batch, hw=416, seed=1234):
    rng = np.random.default_rng(seed)
    return {"input": rng.random((batch, 3, hw, hw), dtype=np.float32)}


def build_yolov3(b, w, batch, hw=416, width=1.0, classes=NUM_CLASSES, postprocess=True, max_out=100,
                 iou_thr=0.45, score_thr=0.3):
    spec = {s[0]: s for s in yolov3_conv_specs(width, classes)}

    def conv(x, name):
        _, cout, cin, k, s, act = spec[name]
        p = k // 2
        y = b.conv(x, b.const(name + ".w", w[name + ".w"]), b.const(name + ".b", w[name + ".b"]), (s, s),
                   (p, p, p, p), name=name)
        return b.leaky_relu(y, LEAKY, name=name + ".act") if act else y

    x = b.arg("input", (batch, 3, hw, hw))
    x = conv(x, "d0")
    routes = {}
    for si, blocks in enumerate([1, 2, 8, 8, 4]):
        x = conv(x, "d%d.down" % (si + 1))
        for bi in range(blocks):
            y = conv(conv(x, "d%d.b%d.c1" % (si + 1, bi)), "d%d.b%d.c2" % (si + 1, bi))
            x = b.add(y, x, name="d%d.b%d.add" % (si + 1, bi))
        routes[si + 1] = x
    route = {1: routes[5], 2: routes[4], 3: routes[3]}
    heads = []
    grid = hw // 32
    branch = None
    for hi in (1, 2, 3):
        if hi == 1:
            x = route[1]
        else:
            lat = conv(branch, "h%d.lat" % hi)
            grid *= 2
            up = b.resize_nearest(lat, (grid, grid), name="h%d.up" % hi)
            x = b.concat([up, route[hi]], 1, name="h%d.cat" % hi)
        for j in range(5):
            x = conv(x, "h%d.c%d" % (hi, j))
        branch = x
        heads.append(conv(conv(x, "h%d.c5" % hi), "h%d.out" % hi))
    for i, h in enumerate(heads):
        b.output(h, "head%d" % i)
    if postprocess:
        det = yolo_postprocess(b, heads, batch, hw, classes, max_out, iou_thr, score_thr)
        b.output(det, "detections")


def build_yolo_postprocess(b, batch, hw=416, classes=NUM_CLASSES, max_out=100, iou_thr=0.45, score_thr=0.3):
    """Post-processing alone: the three head tensors are arguments."""
    nout = 3 * (5 + classes)
    heads = [b.arg("head%d" % i, (batch, nout, hw // s, hw // s)) for i, s in enumerate((32, 16, 8))]
    det = yolo_postprocess(b, heads, batch, hw, classes, max_out, iou_thr, score_thr)
    b.output(det, "detections")


def yolo_postprocess(b, heads, batch, hw, classes, max_out, iou_thr, score_thr):
    all_boxes, all_scores = [], []
    for i, (h, stride) in enumerate(zip(heads, (32, 16, 8))):
        g = hw // stride
        nb = 3 * g * g
        pfx = "pp%d." % i
        t = b.reshape(h, (batch, 3, 5 + classes, g * g), name=pfx + "r0")
        t = b.transpose(t, (0, 1, 3, 2), name=pfx + "t0")                     # [N,3,gg,5+C]
        t = b.reshape(t, (batch, nb, 5 + classes), name=pfx + "r1")
        gy, gx = np.meshgrid(np.arange(g, dtype=np.float32), np.arange(g, dtype=np.float32), indexing="ij")
        grid_x = np.tile(gx.reshape(-1), 3).reshape(1, nb, 1)
        grid_y = np.tile(gy.reshape(-1), 3).reshape(1, nb, 1)
        anc = np.array([ANCHORS[m] for m in MASKS[i]], np.float32)             # [3,2] (w,h) in pixels
        anc_w = np.repeat(anc[:, 0], g * g).reshape(1, nb, 1) / np.float32(hw)
        anc_h = np.repeat(anc[:, 1], g * g).reshape(1, nb, 1) / np.float32(hw)
        inv_g = np.full((1,), 1.0 / g, np.float32)

        def comp(k0, k1, nm):
            return b.slice(t, (0, 0, k0), (batch, nb, k1), name=pfx + nm)

        cx = b.mul(b.add(b.sigmoid(comp(0, 1, "tx"), name=pfx + "sx"), b.const(pfx + "gx", grid_x), name=pfx + "ax"),
                   b.const(pfx + "ig", inv_g), name=pfx + "cx")
        cy = b.mul(b.add(b.sigmoid(comp(1, 2, "ty"), name=pfx + "sy"), b.const(pfx + "gy", grid_y), name=pfx + "ay"),
                   b.const(pfx + "ig2", inv_g), name=pfx + "cy")
        bw = b.mul(b.exp(comp(2, 3, "tw"), name=pfx + "ew"), b.const(pfx + "aw", anc_w.astype(np.float32)), name=pfx + "bw")
        bh = b.mul(b.exp(comp(3, 4, "th"), name=pfx + "eh"), b.const(pfx + "ah", anc_h.astype(np.float32)), name=pfx + "bh")
        half = b.const(pfx + "half", np.full((1,), 0.5, np.float32))
        hw_ = b.mul(bw, half, name=pfx + "hw")
        hh_ = b.mul(bh, half, name=pfx + "hh")
        box = b.concat([b.sub(cy, hh_, name=pfx + "y1"), b.sub(cx, hw_, name=pfx + "x1"),
                        b.add(cy, hh_, name=pfx + "y2"), b.add(cx, hw_, name=pfx + "x2")], 2, name=pfx + "box")
        obj = b.sigmoid(comp(4, 5, "to"), name=pfx + "obj")
        cls = b.sigmoid(comp(5, 5 + classes, "tc"), name=pfx + "cls")
        sc = b.mul(cls, obj, name=pfx + "score")                                # [N,nb,C]
        all_boxes.append(box)
        all_scores.append(b.transpose(sc, (0, 2, 1), name=pfx + "score_t"))     # [N,C,nb]
    boxes = b.concat(all_boxes, 1, name="boxes")
    scores = b.concat(all_scores, 2, name="scores")
    b.output(boxes, "boxes")
    b.output(scores, "scores")
    return b.nms(boxes, scores, max_out, iou_thr, score_thr, name="detections")


def choose_head_bias(head_logits, classes=NUM_CLASSES, target=0.01, thr=0.3):
    """Bias added to objectness and class logits so that about `target` of the
    (box, class) scores pass `thr`.  head_logits: list of [N,3*(5+C),g,g] arrays
    computed with zero bias."""
    objs, clss = [], []
    for h in head_logits:
        n, _, g, _ = h.shape
        t = h.reshape(n, 3, 5 + classes, g * g)
        objs.append(t[:, :, 4:5].reshape(-1, 1, g * g))
        clss.append(t[:, :, 5:].reshape(-1, classes, g * g))
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))
    lo, hi = -10.0, 10.0
    for _ in range(40):
        mid = 0.5 * (lo + hi)
        passed = total = 0
        for o, c in zip(objs, clss):
            s = sig(o.astype(np.float64) + mid) * sig(c.astype(np.float64) + mid)
            passed += int((s > thr).sum())
            total += s.size
        if passed / total > target:
            hi = mid
        else:
            lo = mid
    return 0.5 * (lo + hi)
