"""GPU parity: non-maximum suppression on device-resident records against the CPU checker
(src/Box.cpp:56-147), through the C ABI.  Decisions are comparisons of float32 quantities computed
with the same operations, so the surviving records must be byte-identical and in the same order."""
import numpy as np
import pytest

from pixienn_amd import workloads as wl
from util import detection_records as _records, gpu, random_detections

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from pixienn_amd import ops as o
    return o


def run(ops, rec, batch, classes, threshold, capacity=None):
    records, count = ops.records_to_device(rec, capacity)
    kept, kept_count = ops.nms(records, count, batch, classes, threshold)
    return ops.nms_to_host(kept, kept_count)


def same(got, want, what):
    assert len(got) == len(want), "%s: %d kept, checker keeps %d" % (what, len(got), len(want))
    assert list(got["order"]) == list(want["order"]), what
    assert got.tobytes() == want.tobytes(), what


# A capacity of at most 512 takes the one-workgroup kernel, a larger one the sorting path.
PATHS = pytest.mark.parametrize("capacity", [None, 3000], ids=["one-workgroup", "sorted"])


@PATHS
def test_nms_reference_kats(ops, oracle, kats, capacity):
    """tests/src/box.cpp:25-101 on the device."""
    for case in kats["nms"]["cases"]:
        rec = _records(oracle, case["detections"])
        got = run(ops, rec, 2, 17, case["threshold"], capacity)
        if "expected_boxes" in case:
            boxes = [[float(r["x"]), float(r["y"]), float(r["w"]), float(r["h"])] for r in got]
            assert boxes == [[float(v) for v in b] for b in case["expected_boxes"]], case["name"]
        if "expected_count" in case:
            assert len(got) == case["expected_count"], case["name"]
        if "expected_classes" in case:
            assert list(got["class_index"]) == case["expected_classes"], case["name"]
        same(got, oracle.nms(rec, case["threshold"]), case["name"])


@PATHS
def test_nms_hand_worked_scenarios(ops, oracle, capacity):
    X = [0, 0, 100, 100]
    Y = [0, 0, 100, 70]
    A1 = [0, 0, 100, 95]; A2 = [0, 0, 100, 89]
    Z = [5, 5, 0, 0]
    cases = {
        "dropped duplicate does not suppress": ([X + [0, 1, 0.9], X + [0, 2, 0.8], Y + [0, 2, 0.7]], 0.5, 2),
        "dropped duplicate does not drop": ([X + [0, 1, 0.9], A1 + [0, 2, 0.8], A2 + [0, 3, 0.7]], 0.5, 2),
        "ties keep input order": ([X + [0, 1, 0.5], X + [0, 1, 0.5]], 0.5, 1),
        "sorted across images": ([X + [1, 1, 0.2], X + [0, 1, 0.9], X + [2, 1, 0.5]], 0.5, 3),
        "negative extents": ([X + [0, 1, 0.9], [100, 100, -100, -100, 0, 1, 0.8]], 0.5, 1),
        "empty boxes": ([Z + [0, 1, 0.9], Z + [0, 1, 0.8]], 0.0, 2),
        "at the threshold": ([[0, 0, 100, 100, 0, 1, 0.9], [0, 0, 100, 50, 0, 1, 0.8]], 0.5, 2),
        "past 1024 in a group": ([X + [0, 1, 1.0 - i * 1e-4] for i in range(1100)], 0.5, 77),
        "dropped members use up places": ([X + [0, 2, 1.0]] + [X + [0, 1, 0.9 - i * 1e-4] for i in range(1100)],
                                          0.5, 1),
    }
    for name, (rows, thr, expect) in cases.items():
        rec = _records(oracle, rows)
        got = run(ops, rec, 3, 4, thr, capacity)
        assert len(got) == expect, name
        same(got, oracle.nms(rec, thr), name)


def test_nms_empty_and_capacity(ops, oracle):
    import torch
    got = run(ops, _records(oracle, []), 1, 1, 0.5, capacity=16)
    assert len(got) == 0
    # a counter above the capacity (a detection pass that overflowed) means "capacity records"
    rec = random_detections(oracle, 11, 300, 2, 3, 2)
    records, count = ops.records_to_device(rec, 300)
    count.fill_(100000)
    kept, kept_count = ops.nms(records, count, 2, 3, 0.45)
    same(ops.nms_to_host(kept, kept_count), oracle.nms(rec, 0.45), "overflowed counter")
    # capacity far above the live count, a caller-owned workspace, a negative counter
    need = ops.capi.load().pxh_nms_workspace_bytes(5000)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    records, count = ops.records_to_device(rec, 5000)
    kept, kept_count = ops.nms(records, count, 2, 3, 0.45, workspace=ws)
    same(ops.nms_to_host(kept, kept_count), oracle.nms(rec, 0.45), "capacity above count")
    count.fill_(-5)
    kept, kept_count = ops.nms(records, count, 2, 3, 0.45, workspace=ws)
    assert len(ops.nms_to_host(kept, kept_count)) == 0
    with pytest.raises(ops.capi.PxError):
        ops.nms(records, count, 2, 3, -0.1)
    with pytest.raises(ops.capi.PxError):
        ops.nms(records, count, 2, 3, 0.45, workspace=ws[:1024])


@pytest.mark.parametrize("seed,n,batch,classes,clusters,thr", [
    (21, 300, 2, 3, 3, 0.45), (22, 5000, 1, 2, 2, 0.3), (23, 4097, 3, 5, 1, 0.6), (24, 20000, 8, 80, 6, 0.4),
    (25, 12000, 1, 300, 4, 0.5), (26, 9000, 300, 2, 1, 0.5), (27, 4096, 1, 1, 3, 0.45), (28, 30000, 2, 1, 2, 0.7),
    (29, 495, 2, 5, 2, 0.4), (30, 320, 1, 80, 3, 0.45), (31, 64, 3, 2, 1, 0.0), (32, 1, 1, 1, 1, 0.5),
])
def test_nms_random_clusters_match_the_checker(ops, oracle, seed, n, batch, classes, clusters, thr):
    rec = random_detections(oracle, seed, n, batch, classes, clusters)
    rec["order"] = np.random.Generator(np.random.Philox(key=seed)).permutation(n)   # orders need not be sorted
    want = oracle.nms(rec[np.argsort(rec["order"])], thr)          # the checker takes the input sequence
    got = run(ops, rec, batch, classes, thr, capacity=n + 17)
    assert 0 < len(want) and (len(want) < n or n == 1)
    same(got, want, "seed %d" % seed)


def chain(oracle, length, ratio, classes):
    """Boxes shrinking by `ratio` per step: each overlaps its neighbour by `ratio` and the one after
    that by ratio^2, so every decision hangs on the one before it."""
    rows = []
    for k in range(length):
        rows.append([0, 0, 100, 100 * ratio ** k, 0, k % classes, 0.99 - 0.01 * k])
    return _records(oracle, rows)


@PATHS
@pytest.mark.parametrize("sweeps", [1, 3])
def test_nms_long_dependency_chains(ops, oracle, sweeps, capacity):
    """Chains as long as the list: alternating classes exercise the duplicate step's repeated sweeps
    and its per-image loop, one class the greedy step's loop."""
    lib = ops.capi.load()
    before = lib.pxh_debug_nms_sweeps(sweeps)
    try:
        rec = chain(oracle, 40, 0.92, 2)               # 0.92 > 0.9 > 0.92^2: duplicate chain
        want = oracle.nms(rec, 0.95)
        assert list(want["order"]) == list(range(0, 40, 2))
        same(run(ops, rec, 1, 2, 0.95, capacity), want, "duplicate chain")
        rec = chain(oracle, 60, 0.7, 1)                # 0.7 > 0.5 > 0.49: greedy chain
        want = oracle.nms(rec, 0.5)
        assert list(want["order"]) == list(range(0, 60, 2))
        same(run(ops, rec, 1, 1, 0.5, capacity), want, "greedy chain")
        # many chains in many images at once, longer than the number of sweeps
        parts = []
        for b in range(5):
            c = chain(oracle, 30 + b, 0.92, 3)
            c["batch"] = b
            parts.append(c)
        rec = np.concatenate(parts)
        rec["order"] = np.arange(len(rec))
        same(run(ops, rec, 5, 3, 0.95, capacity), oracle.nms(rec, 0.95), "chains in five images")
    finally:
        lib.pxh_debug_nms_sweeps(before)


def test_detections_of_two_heads_then_nms(ops, oracle):
    """Two heads append into one record array with continuing orders, as Model::detections walks the
    YOLO layers; nms runs on the array without it leaving the device."""
    import torch
    N, K, thr = 2, 6, 0.35
    heads = [(13, [3, 4, 5]), (26, [0, 1, 2])]
    cap = 1 << 16
    records = torch.zeros((cap, 8), dtype=torch.int32, device="cuda")
    count = torch.zeros(1, dtype=torch.int32, device="cuda")
    want_parts = []
    base = 0
    for W, mask in heads:
        logits = wl.normal(3700 + W, (N, len(mask) * (K + 5), W, W), std=1.5)
        cfg, keep = oracle.yolo_cfg(N, W, W, K, mask, wl.TINY_ANCHORS, 416, 416)
        decoded = np.zeros_like(logits)
        oracle.yolo_decode(cfg, logits, decoded)
        part, found = oracle.yolo_detections(cfg, decoded, thr, cap, image_width=640, image_height=480)
        part = part.copy()
        part["order"] += base
        want_parts.append(part)
        ops.yolo_detections_append(gpu(decoded), N, mask, wl.TINY_ANCHORS, K, W, W, 416, 416, thr, base, records,
                                   count, image_width=640, image_height=480)
        base += N * len(mask) * W * W * K
    all_want = np.concatenate(want_parts)
    torch.cuda.synchronize()
    found = int(count.item())
    assert found == len(all_want) and 100 < found < cap
    got_all = records[:found].cpu().numpy().view(oracle.DETECTION_DTYPE).reshape(-1)
    got_all = got_all[np.argsort(got_all["order"])]
    assert np.array_equal(got_all["order"], all_want["order"])
    # the device's own records (pixel boxes may differ from the checker's by a truncation) are the input
    kept, kept_count = ops.nms(records, count, N, K, 0.45)
    same(ops.nms_to_host(kept, kept_count), oracle.nms(got_all, 0.45), "two heads")
