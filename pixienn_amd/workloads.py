"""Layer shapes of the benchmark configurations and seeded synthetic inputs.

Shapes follow the reference's model files (resources/models/yolov3.yml, yolov3-tiny.yml) and
the synthetic shapes the baseline names.  Inputs come from numpy's counter-based Philox
generator, so the same seed gives the same bits on every host.
"""
import numpy as np

# (channels, height == width) of every BN'd conv output
YOLOV3_TINY_CONV_SHAPES = [(16, 416), (32, 208), (64, 104), (128, 52), (256, 26), (512, 13), (1024, 13)]
TINY_ANCHORS = [10, 14, 23, 27, 37, 58, 81, 82, 135, 169, 344, 319]
TINY_MASKS = [[3, 4, 5], [0, 1, 2]]

# YOLOv3 @608: distinct BN'd conv-output shapes (channels, size) and how many conv layers have each
YOLOV3_BN_SHAPES = [(32, 608), (64, 304), (32, 304), (128, 152), (64, 152), (256, 76), (128, 76),
                    (512, 38), (256, 38), (128, 38), (1024, 19), (512, 19), (256, 19)]
# number of conv layers of yolov3.yml with each of those output shapes (72 BN'd convs in all)
YOLOV3_BN_COUNTS = [1, 2, 1, 3, 2, 12, 11, 12, 11, 1, 8, 7, 1]
# the three linear (bias only) 255-channel convs in front of the heads
YOLOV3_HEAD_CONV_SHAPES = [(255, 19), (255, 38), (255, 76)]
YOLOV3_SHORTCUT_SHAPES = [(64, 304, 1), (128, 152, 2), (256, 76, 8), (512, 38, 8), (1024, 19, 4)]
YOLOV3_MAXPOOL_SHAPES = [(64, 304), (128, 152), (256, 76), (512, 38)]
YOLOV3_UPSAMPLE_SHAPES = [(256, 19), (128, 38)]
YOLOV3_HEAD_SIZES = [19, 38, 76]
YOLOV3_ANCHORS = [10, 13, 16, 30, 33, 23, 30, 61, 62, 45, 59, 119, 116, 90, 156, 198, 373, 326]
YOLOV3_MASKS = {19: [6, 7, 8], 38: [3, 4, 5], 76: [0, 1, 2]}
YOLOV3_PARAMS = 61949149   # conv weights + biases + BN scales


def rng(seed):
    return np.random.Generator(np.random.Philox(key=int(seed)))


def normal(seed, shape, mean=0.0, std=1.0):
    return (rng(seed).standard_normal(shape, dtype=np.float32) * np.float32(std) + np.float32(mean)).astype(np.float32)


def uniform(seed, shape, lo=0.0, hi=1.0):
    return rng(seed).uniform(lo, hi, shape).astype(np.float32)


def bn_params(seed, channels):
    """gamma = 1, beta ~ N(0, 0.1), running mean ~ N(0, 0.1), running var ~ U(0.5, 1.5)."""
    g = rng(seed)
    scale = np.ones(channels, np.float32)
    bias = (0.1 * g.standard_normal(channels)).astype(np.float32)
    mean = (0.1 * g.standard_normal(channels)).astype(np.float32)
    var = g.uniform(0.5, 1.5, channels).astype(np.float32)
    return scale, bias, mean, var


def yolo_truths(seed, batch, max_boxes=20, classes=80):
    """1..max_boxes boxes per image: centres U(0,1), w/h log-uniform in [0.02, 0.9], class uniform.
    Returns (truths[batch, max_boxes, 5], counts[batch])."""
    g = rng(seed)
    counts = g.integers(1, max_boxes + 1, batch).astype(np.int32)
    truths = np.zeros((batch, max_boxes, 5), np.float32)
    for b in range(batch):
        k = int(counts[b])
        truths[b, :k, 0:2] = g.uniform(0.0, 1.0, (k, 2))
        truths[b, :k, 2:4] = np.exp(g.uniform(np.log(0.02), np.log(0.9), (k, 2)))
        truths[b, :k, 4] = g.integers(0, classes, k)
    return truths, counts


def yolo_assign_targets(truths, counts, masks, anchors, width, height, net_width, net_height):
    """Host-side positive assignment for the decoded-input loss entry point, as the reference's
    target builder does it (src/YoloTargetBuilder.cpp:21-62): every truth goes to the anchor whose
    origin-centred box overlaps its own best; if this head owns that anchor, the slot at the
    truth's cell takes its class, anchor and box (a later truth overwrites an earlier one).
    Returns (classes[slots], anchors[slots], boxes[slots, 4]) with slots = batch * masks * area."""
    batch = truths.shape[0]
    area = width * height
    slots = batch * len(masks) * area
    cls = np.full(slots, -1, np.int32)
    anc = np.full(slots, -1, np.int32)
    box = np.zeros((slots, 4), np.float32)
    aw = np.asarray(anchors[0::2], np.float32) / np.float32(net_width)
    ah = np.asarray(anchors[1::2], np.float32) / np.float32(net_height)
    for b in range(batch):
        for t in range(int(counts[b])):
            x, y, w, h, c = truths[b, t]
            if w <= 0 or h <= 0:
                continue
            inter = np.minimum(aw, w) * np.minimum(ah, h)
            iou = inter / (aw * ah + w * h - inter)
            best = int(np.argmax(iou))
            if best not in masks:
                continue
            n = list(masks).index(best)
            i = min(width - 1, max(0, int(x * width)))
            j = min(height - 1, max(0, int(y * height)))
            s = (b * len(masks) + n) * area + j * width + i
            cls[s] = int(c)
            anc[s] = best
            box[s] = (x, y, w, h)
    return cls, anc, box


# one detection record of the C ABI (struct pxh_detection): left, top, width, height, probability,
# image, class, position in the reference's emission order
DETECTION_DTYPE = np.dtype([("x", "f4"), ("y", "f4"), ("w", "f4"), ("h", "f4"), ("prob", "f4"), ("batch", "i4"),
                            ("class_index", "i4"), ("order", "u4")])


def detection_clusters(seed, n, batch, classes, clusters, spread=6.0):
    """n detection records scattered around a few centres per image, so that many overlap, with
    probabilities rounded to two decimals (plenty of ties) -- input for non-maximum suppression."""
    g = rng(seed)
    rec = np.zeros(n, DETECTION_DTYPE)
    centre = g.uniform(50, 400, (batch, clusters, 2))
    size = g.uniform(20, 120, (batch, clusters, 2))
    b = g.integers(0, batch, n)
    k = g.integers(0, clusters, n)
    rec["batch"] = b
    rec["class_index"] = g.integers(0, classes, n)
    jitter = g.normal(0, spread, (n, 4)).astype(np.float32)
    rec["w"] = np.maximum(1, size[b, k, 0] + jitter[:, 2])
    rec["h"] = np.maximum(1, size[b, k, 1] + jitter[:, 3])
    rec["x"] = centre[b, k, 0] + jitter[:, 0] - rec["w"] / 2
    rec["y"] = centre[b, k, 1] + jitter[:, 1] - rec["h"] / 2
    rec["prob"] = np.round(g.uniform(0.05, 1.0, n), 2).astype(np.float32)
    rec["order"] = np.arange(n)
    return rec


def yolov3_layers(size=608):
    """The 107 layers of the reference's resources/models/yolov3.yml as dictionaries with the output
    shape filled in: conv (filters, stride, bn, kernel), shortcut (from), route (layers), upsample, yolo (mask).
    Keys: type, c, s (output channels and height == width), plus the type's own (conv: bn, k = kernel
    size, in_c = input channels)."""
    layers = []

    def conv(filters, stride=1, bn=True, k=3):
        prev = layers[-1] if layers else dict(c=3, s=size)
        layers.append(dict(type="conv", c=filters, s=prev["s"] // stride, bn=bn, k=k, in_c=prev["c"]))

    def shortcut():
        layers.append(dict(type="shortcut", c=layers[-1]["c"], s=layers[-1]["s"], frm=len(layers) - 3))

    def residual(narrow, wide, times):
        for _ in range(times):
            conv(narrow, k=1)
            conv(wide)
            shortcut()

    conv(32)
    conv(64, 2); residual(32, 64, 1)
    conv(128, 2); residual(64, 128, 2)
    conv(256, 2); residual(128, 256, 8)
    conv(512, 2); residual(256, 512, 8)
    conv(1024, 2); residual(512, 1024, 4)
    for head, (narrow, wide, mask, joins) in enumerate([(512, 1024, [6, 7, 8], None), (256, 512, [3, 4, 5], 61),
                                                        (128, 256, [0, 1, 2], 36)]):
        if joins is not None:
            src = len(layers) - 4
            layers.append(dict(type="route", c=layers[src]["c"], s=layers[src]["s"], sources=[src]))
            conv(narrow, k=1)
            layers.append(dict(type="upsample", c=narrow, s=2 * layers[-1]["s"]))
            up = len(layers) - 1
            layers.append(dict(type="route", c=narrow + layers[joins]["c"], s=layers[up]["s"], sources=[up, joins]))
        for _ in range(3):
            conv(narrow, k=1)
            conv(wide)
        conv(255, bn=False, k=1)
        layers.append(dict(type="yolo", c=255, s=layers[-1]["s"], mask=mask))
    return layers


def yolov3_tiny_layers(size=416):
    """The 24 layers of resources/models/yolov3-tiny.yml of the reference at a size x size input, in
    model order, as dicts like yolov3_layers': conv (c, s, bn, act), maxpool (c, s = input size, stride),
    upsample, route (sources), yolo (mask)."""
    layers = []
    s = size
    for c in (16, 32, 64, 128, 256, 512):
        layers.append(dict(type="conv", c=c, s=s, bn=True, act="leaky"))
        stride = 1 if c == 512 else 2
        layers.append(dict(type="maxpool", c=c, s=s, stride=stride))
        s = s if stride == 1 else s // 2
    layers.append(dict(type="conv", c=1024, s=s, bn=True, act="leaky"))          # 12
    layers.append(dict(type="conv", c=256, s=s, bn=True, act="leaky"))           # 13
    layers.append(dict(type="conv", c=512, s=s, bn=True, act="leaky"))           # 14
    layers.append(dict(type="conv", c=255, s=s, bn=False, act="linear"))         # 15
    layers.append(dict(type="yolo", c=255, s=s, mask=TINY_MASKS[0]))             # 16
    layers.append(dict(type="route", c=256, s=s, sources=[13]))                  # 17
    layers.append(dict(type="conv", c=128, s=s, bn=True, act="leaky"))           # 18
    layers.append(dict(type="upsample", c=128, s=2 * s))                         # 19
    layers.append(dict(type="route", c=384, s=2 * s, sources=[19, 8]))           # 20
    layers.append(dict(type="conv", c=256, s=2 * s, bn=True, act="leaky"))       # 21
    layers.append(dict(type="conv", c=255, s=2 * s, bn=False, act="linear"))     # 22
    layers.append(dict(type="yolo", c=255, s=2 * s, mask=TINY_MASKS[1]))         # 23
    return layers


def yolov3_parameter_tensors(size=608):
    """(elements, takes_weight_decay) of every parameter tensor of YOLOv3 in layer order, as the engine
    holds them: per convolution the weights (filters x input channels x k x k, decayed), the biases and,
    with batch norm, the scales (include/ConvLayer.h:96-115 of the reference).  222 tensors, YOLOV3_PARAMS
    elements in all."""
    tensors = []
    for l in yolov3_layers(size):
        if l["type"] != "conv":
            continue
        tensors.append((l["c"] * l["in_c"] * l["k"] * l["k"], True))
        tensors.append((l["c"], False))
        if l["bn"]:
            tensors.append((l["c"], False))
    return tensors
