"""GPU parity: all heads of a model in one pass (pxh_yolo_forward_train_heads) against the CPU checker's
YoloLayer forward (include/YoloLayer.h:164-239, 450-547 of the reference) run head by head on the same
seeded inputs, and against pxh_yolo_forward_train on each head: outputs and deltas to the bit."""
import numpy as np
import pytest

from pixienn_amd import workloads as wl
from test_gpu_yolo_adam import compare_head, oracle_head
from util import F, assert_bit_exact, gpu, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from pixienn_amd import ops as o
    return o


def run_heads(ops, xs, truths, counts, sizes, K, masks, anchors, net, kws, forced_workers=0):
    """The heads in one call; returns per head (out, delta, cost, stats)."""
    import torch
    from pixienn_amd import capi
    N = xs[0].shape[0]
    heads, keep = [], []
    for x, W, mask, kw in zip(xs, sizes, masks, kws):
        t = dict(input=gpu(x), output=torch.full(x.shape, 7.0, device="cuda"),
                 delta=torch.full(x.shape, 7.0, device="cuda"), masks=mask, width=W, height=W,
                 stats=torch.full((12,), 5.0, device="cuda"), cost=torch.full((1,), 5.0, device="cuda"), **kw)
        heads.append(t)
    capi.load().pxh_debug_yolo_tuning(0, 0, forced_workers)
    try:
        ops.yolo_forward_train_heads(heads, gpu(truths), gpu(counts), truths.shape[1], anchors, N, K, net, net)
    finally:
        capi.load().pxh_debug_yolo_tuning(0, 0, 0)
    return [(host(h["output"]), host(h["delta"]), float(host(h["cost"])[0]), host(h["stats"])) for h in heads]


def single_head(ops, x, truths, counts, W, K, mask, anchors, net, kw):
    import torch
    N = x.shape[0]
    out = torch.full(x.shape, 7.0, device="cuda"); delta = torch.full(x.shape, 7.0, device="cuda")
    stats = torch.zeros(12, device="cuda"); cost = torch.zeros(1, device="cuda")
    ops.yolo_forward_train(gpu(x), out, delta, gpu(truths), gpu(counts), truths.shape[1], mask, anchors, stats, cost, N,
                           K, W, W, net, net, kw["ignore_thresh"], kw["truth_thresh"], kw["coord_scale"],
                           kw["object_scale"], kw["noobject_scale"], kw["class_scale"])
    return host(out), host(delta), float(host(cost)[0]), host(stats)


@pytest.mark.parametrize("forced_workers", [0, 1, 7])
def test_three_heads_of_yolov3_in_one_pass(ops, oracle, forced_workers):
    N, K = 4, 80
    sizes = [19, 38, 76]
    masks = [wl.YOLOV3_MASKS[s] for s in sizes]
    xs = [wl.normal(2700 + W, (N, 3 * (K + 5), W, W), std=2.0) for W in sizes]
    truths, counts = wl.yolo_truths(2750, N)
    kw = dict(ignore_thresh=0.7, truth_thresh=1.0, coord_scale=1.0, object_scale=2.0, noobject_scale=0.1,
              class_scale=1.0)
    got = run_heads(ops, xs, truths, counts, sizes, K, masks, wl.YOLOV3_ANCHORS, 608, [kw] * 3, forced_workers)
    positives = 0
    for x, W, mask, g in zip(xs, sizes, masks, got):
        want = oracle_head(oracle, x, truths, counts, W, W, K, mask, wl.YOLOV3_ANCHORS, 608, **kw)
        compare_head(g, want, "head %d of three" % W, 3, kw)
        positives += want[3][6]
        one = single_head(ops, x, truths, counts, W, K, mask, wl.YOLOV3_ANCHORS, 608, kw)
        assert_bit_exact(g[0], one[0], "head %d: output against the single-head call" % W)
        assert_bit_exact(g[1], one[1], "head %d: delta against the single-head call" % W)
        assert g[3][6] == one[3][6] and g[3][1] == one[3][1]
    # every truth claims one slot, on the head that holds its best anchor
    assert positives == counts.sum()


def test_heads_with_settings_of_their_own_unaligned_planes_and_one_head(ops, oracle):
    """Two heads of YOLOv3-tiny shape (13 x 13 and 26 x 26: planes of 169 floats are not a multiple of 4) with
    different thresholds and scales per head, more truths than a tile of 256 on one image, an image without
    truths; then a call with a single head."""
    N, K = 3, 5
    anchors = [10, 14, 23, 27, 37, 58, 81, 82, 135, 169, 344, 319]
    sizes = [13, 26]
    masks = [[3, 4, 5], [0, 1, 2]]
    xs = [wl.normal(2800 + W, (N, 3 * (K + 5), W, W), std=1.5) for W in sizes]
    truths, counts = wl.yolo_truths(2801, N, max_boxes=300, classes=K)
    counts[:] = [300, 0, 17]
    kws = [dict(ignore_thresh=0.5, truth_thresh=1.0, coord_scale=1.3, object_scale=1.7, noobject_scale=0.4,
                class_scale=0.8),
           dict(ignore_thresh=0.7, truth_thresh=0.3, coord_scale=1.0, object_scale=2.0, noobject_scale=0.1,
                class_scale=1.0)]
    got = run_heads(ops, xs, truths, counts, sizes, K, masks, anchors, 416, kws)
    for x, W, mask, kw, g in zip(xs, sizes, masks, kws, got):
        want = oracle_head(oracle, x, truths, counts, W, W, K, mask, anchors, 416, **kw)
        compare_head(g, want, "tiny head %d" % W, 3, kw)
    got = run_heads(ops, xs[:1], truths, counts, sizes[:1], K, masks[:1], anchors, 416, kws[:1])
    want = oracle_head(oracle, xs[0], truths, counts, 13, 13, K, masks[0], anchors, 416, **kws[0])
    compare_head(got[0], want, "one head through the many-head call", 3, kws[0])


def test_heads_call_rejects_bad_arguments(ops):
    import ctypes
    from pixienn_amd import capi
    lib = capi.load()
    table = (capi.YoloHead * 5)()
    a = np.array(wl.YOLOV3_ANCHORS, np.int32)
    assert lib.pxh_yolo_heads_workspace_bytes(0, ctypes.addressof(table), 4) == 0
    assert lib.pxh_yolo_heads_workspace_bytes(5, ctypes.addressof(table), 4) == 0
    counts = gpu(np.zeros(4, np.int32))
    rc = capi.call_raw("pxh_yolo_forward_train_heads", 5, ctypes.addressof(table), None, counts.data_ptr(), 0,
                       a.ctypes.data, 9, 4, 80, 608, 608, None, 0, None)
    assert rc == -2 and "heads per call" in capi.last_error()
    rc = capi.call_raw("pxh_yolo_forward_train_heads", 1, ctypes.addressof(table), None, counts.data_ptr(), 0,
                       a.ctypes.data, 9, 4, 80, 608, 608, None, 0, None)
    assert rc == -1 and "null pointer in head 0" in capi.last_error()
