"""Seeded random geometries for the index-work kernels, bit for bit against the CPU checker:
whatever kernel, stride, padding, size, channel mismatch or pointer alignment a model file can
ask for has to give the CPU layer's result, not only the shapes of the shipped networks."""
import numpy as np
import pytest

from pixienn_amd import workloads as wl
from util import F, assert_bit_exact, gpu, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from pixienn_amd import ops as o
    return o


def test_maxpool_random_geometries(ops, oracle):
    import torch
    r = np.random.default_rng(101)
    done = 0
    while done < 60:
        k = int(r.integers(1, 5)); s = int(r.integers(1, 4)); p = int(r.integers(0, k + 1))
        H = int(r.integers(1, 24)); W = int(r.integers(1, 24)); N = int(r.integers(1, 4)); C = int(r.integers(1, 6))
        oh = oracle.maxpool_out_dim(H, k, s, p); ow = oracle.maxpool_out_dim(W, k, s, p)
        if oh <= 0 or ow <= 0:
            continue
        done += 1
        x = wl.normal(5000 + done, (N, C, H, W))
        if done % 5 == 0:
            x = np.round(x)            # ties: the first maximum in window order must win
        want = np.empty((N, C, oh, ow), F); widx = np.empty((N, C, oh, ow), np.int32)
        oracle.maxpool_forward(x, want, widx, N, C, H, W, oh, ow, k, s, p)
        out = torch.full((N, C, oh, ow), 9.0, device="cuda")
        idx = torch.full((N, C, oh, ow), -9, device="cuda", dtype=torch.int32)
        ops.maxpool_forward(gpu(x), out, idx, k, s, p)
        what = "maxpool %s k%d s%d p%d" % ((N, C, H, W), k, s, p)
        assert_bit_exact(host(out), want, what + " values")
        assert_bit_exact(host(idx), widx, what + " indexes")
        delta = wl.normal(5100 + done, want.shape); grad0 = wl.normal(5200 + done, x.shape)
        gw = grad0.copy()
        oracle.maxpool_backward(delta, widx, gw)
        gg = gpu(grad0)
        ops.maxpool_backward(gpu(delta), idx, gg, k, s, p)
        assert_bit_exact(host(gg), gw, what + " backward")


def test_upsample_random_geometries(ops, oracle):
    import torch
    r = np.random.default_rng(102)
    for case in range(40):
        stride = int(r.integers(1, 5)); H = int(r.integers(1, 20)); W = int(r.integers(1, 20))
        N = int(r.integers(1, 4)); C = int(r.integers(1, 6)); scale = float(r.choice([1.0, 0.5, 2.0, -1.25]))
        x = wl.normal(5300 + case, (N, C, H, W))
        want = np.empty((N, C, H * stride, W * stride), F)
        oracle.upsample(x, W, H, C, N, stride, True, scale, None, want)
        out = torch.full(want.shape, 7.0, device="cuda")
        ops.upsample_forward(gpu(x), out, stride, scale)
        what = "upsample %s stride %d scale %g" % ((N, C, H, W), stride, scale)
        assert_bit_exact(host(out), want, what)
        d = wl.normal(5400 + case, want.shape); acc0 = wl.normal(5500 + case, x.shape)
        aw = acc0.copy()
        oracle.upsample(None, W, H, C, N, stride, False, scale, aw, d.copy())
        ga = gpu(acc0)
        ops.upsample_backward(gpu(d), ga, stride, scale)
        assert_bit_exact(host(ga), aw, what + " backward")


def test_shortcut_random_shape_pairs(ops, oracle):
    """shortcutGpu's index map: integer stride (out smaller than add's source) or sample (larger)."""
    r = np.random.default_rng(103)
    done = 0
    while done < 40:
        N = int(r.integers(1, 3)); h2 = int(r.integers(1, 7)); w2 = int(r.integers(1, 7))
        f = int(r.integers(1, 4)); grow = bool(r.integers(0, 2))
        w1, h1 = (w2 * f, h2 * f) if grow else (w2, h2)
        w2, h2 = (w2, h2) if grow else (w2 * f, h2 * f)
        c1 = int(r.integers(1, 6)); c2 = int(r.integers(1, 6))
        add = wl.normal(5600 + done, (N, c1, h1, w1)); out0 = wl.normal(5700 + done, (N, c2, h2, w2))
        want = out0.copy()
        if oracle.shortcut(N, w1, h1, c1, add, w2, h2, c2, 0.75, 1.5, want) != 0:
            continue
        done += 1
        g = gpu(out0)
        ops.shortcut(N, w1, h1, c1, gpu(add), w2, h2, c2, 0.75, 1.5, g)
        assert_bit_exact(host(g), want, "shortcut %s into %s" % ((N, c1, h1, w1), (N, c2, h2, w2)))


def test_streaming_kernels_with_unaligned_views(ops, oracle):
    """Pointers 4, 8 and 12 bytes off a 16-byte boundary take the scalar kernels: same bits."""
    import torch
    n = 4099
    for off in (1, 2, 3):
        a = wl.normal(5800 + off, n + off); b = wl.normal(5810 + off, n + off)
        ga = gpu(a)[off:]; gb = gpu(b)[off:]
        out = torch.zeros(n + off, device="cuda")[off:]
        ops.shortcut_forward(ga.view(1, 1, 1, n), gb.view(1, 1, 1, n), out.view(1, 1, 1, n), "leaky")
        want = np.empty(n, F); pre = np.empty(n, F)
        oracle.shortcut_forward("leaky", 1, n, 1, 1, a[off:].copy(), b[off:].copy(), 1.0, 1.0, want, pre)
        assert_bit_exact(host(out), want, "shortcut forward at offset %d" % off)
        w = a[off:].copy(); d = b[off:].copy()
        oracle.sgd_update(w, d, 4, 1e-2, 0.9, 1e-3, True)
        gw = gpu(a)[off:]; gd = gpu(b)[off:]
        ops.sgd_update(gw, gd, 4, 1e-2, 0.9, 1e-3, True)
        assert np.allclose(host(gw), w, rtol=1e-6, atol=1e-7) and np.allclose(host(gd), d, rtol=1e-6, atol=1e-7)
        route = torch.full((2, 3 * n), -1.0, device="cuda")
        src = gpu(np.stack([a[off:], b[off:]]))
        ops.route_forward(src, route, n + 1)           # an odd offset inside the concatenation
        assert torch.equal(route[:, n + 1:2 * n + 1], src) and float(route[:, :n + 1].max()) == -1.0


def test_yolo_training_pass_random_heads(ops, oracle):
    """Rectangular heads, 1 to 200 classes, any subset of the anchors as mask, truth tables with
    empty rows, truths outside the image, empty or inverted boxes and labels outside the class
    range: delta support, cost and statistics must follow the CPU layer."""
    from test_gpu_yolo_adam import YOLO_SHAPES, compare_head, gpu_head, oracle_head
    from pixienn_amd import capi
    lib = capi.load()
    r = np.random.default_rng(107)
    for case in range(40):
        W = int(r.integers(1, 30)); H = int(r.integers(1, 30)); K = int(r.choice([1, 2, 3, 7, 20, 64, 80, 129, 200]))
        total_anchors = int(r.integers(1, 10)); masks = int(r.integers(1, min(total_anchors, 5) + 1))
        mask = sorted(r.choice(total_anchors, masks, replace=False).tolist())
        anchors = [int(v) for v in r.integers(2, 300, 2 * total_anchors)]
        N = int(r.integers(1, 5)); net = int(r.choice([32, 96, 416, 608]))
        max_truth = int(r.choice([1, 3, 20, 90]))
        x = wl.normal(7000 + case, (N, masks * (K + 5), H, W), std=float(r.choice([0.5, 2.0, 4.0])))
        truths = np.zeros((N, max_truth, 5), F)
        truths[..., 0:2] = r.uniform(-0.1, 1.1, (N, max_truth, 2))
        truths[..., 2:4] = np.exp(r.uniform(np.log(0.01), np.log(1.2), (N, max_truth, 2)))
        truths[..., 4] = r.integers(0, K, (N, max_truth))
        for _ in range(int(r.integers(0, 4))):
            b = int(r.integers(0, N)); t = int(r.integers(0, max_truth))
            kind = int(r.integers(0, 4))
            if kind == 0:
                truths[b, t, 2] = 0.0
            elif kind == 1:
                truths[b, t, 3] = -0.2
            elif kind == 2:
                truths[b, t, 0:2] = [1.0, 0.0]
            else:
                truths[b, t, 4] = K + 3
        counts = r.integers(0, max_truth + 1, N).astype(np.int32)
        kw = dict(ignore_thresh=float(r.choice([0.3, 0.5, 0.7])), truth_thresh=float(r.choice([1.0, 1.0, 0.4])),
                  coord_scale=float(r.choice([1.0, 1.5])), object_scale=float(r.choice([1.0, 2.0])),
                  noobject_scale=float(r.choice([1.0, 0.1])), class_scale=float(r.choice([1.0, 0.7])))
        what = "case %d: N%d %dx%d K%d mask %s of %d net %d counts %s" % (case, N, W, H, K, mask, total_anchors, net,
                                                                           counts.tolist())
        want = oracle_head(oracle, x, truths, counts, W, H, K, mask, anchors, net, **kw)
        # the library's own choice of form and lanes per slot, and one forced shape per case in turn
        for form, lanes in ((0, 0), YOLO_SHAPES[1 + case % 4]):
            lib.pxh_debug_yolo_tuning(form, lanes, 0)
            try:
                got = gpu_head(ops, x, truths, counts, W, H, K, mask, anchors, net, **kw)
            finally:
                lib.pxh_debug_yolo_tuning(0, 0, 0)
            compare_head(got, want, what + " form %d lanes %d" % (form, lanes), masks, kw, sum_rtol=5e-5)


def test_yolo_detections_random_heads(ops, oracle):
    """Detection extraction on rectangular heads and class counts on either side of the kernel's
    32- and 128-class steps: the same records, in the same emission order, as the CPU layer."""
    r = np.random.default_rng(108)
    for case in range(24):
        W = int(r.integers(1, 40)); H = int(r.integers(1, 40))
        K = int(r.choice([1, 2, 31, 32, 33, 80, 127, 128, 129, 300]))
        total_anchors = int(r.integers(1, 8)); masks = int(r.integers(1, min(total_anchors, 4) + 1))
        mask = sorted(r.choice(total_anchors, masks, replace=False).tolist())
        anchors = [int(v) for v in r.integers(2, 300, 2 * total_anchors)]
        N = int(r.integers(1, 4)); net = (int(r.choice([96, 416, 608])), int(r.choice([96, 416, 608])))
        thr = float(r.choice([0.05, 0.3, 0.6]))
        image = [(0, 0), (640, 480), (333, 500), (100, 1000)][case % 4]
        logits = wl.normal(8000 + case, (N, masks * (K + 5), H, W), std=2.0)
        cfg, keep = oracle.yolo_cfg(N, W, H, K, mask, anchors, net[0], net[1])
        decoded = np.zeros_like(logits)
        oracle.yolo_decode(cfg, logits, decoded)
        cap = 1 << 21
        want, found_w = oracle.yolo_detections(cfg, decoded, thr, cap, image_width=image[0], image_height=image[1])
        got, found_g = ops.yolo_detections(gpu(decoded), N, mask, anchors, K, W, H, net[0], net[1], thr, cap,
                                           image_width=image[0], image_height=image[1])
        what = "case %d: N%d %dx%d K%d mask %s net %s thr %g image %s" % (case, N, W, H, K, mask, net, thr, image)
        assert found_g == found_w <= cap, what
        for k in ("order", "batch", "class_index"):
            assert np.array_equal(got[k], want[k]), (what, k)
        assert_bit_exact(got["prob"], want["prob"], what + " probabilities")
        for k in "xywh":
            d = np.abs(got[k].astype(np.float64) - want[k])
            # pixel boxes: a last-place difference in exp may move a truncation by one pixel; relative boxes:
            # left/top are differences of the centre and half the size
            bound = 1.0 if image[0] else 1e-5 * np.maximum(1.0, np.abs(want[k]) + np.abs(want["w"]) + np.abs(want["h"]))
            assert np.all(d <= bound), (what, k, float(d.max()))
