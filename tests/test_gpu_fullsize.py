"""GPU parity at the baseline's full shapes.

The CPU checker is run on whole tensors where it finishes in seconds and on image / range slices
otherwise (every kernel here is independent per image or per element, so a slice of the output is
the output of the slice); on top of that each case checks properties that do not depend on a
second implementation: conservation of sums, copies that must be bit copies, invariants of batch
norm, the cost being the checksum of the delta, bit-identical repeats.
"""
import numpy as np
import pytest

from pixienn_amd import workloads as wl
from util import F, assert_bit_exact, assert_close, gpu, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from pixienn_amd import ops as o
    return o


def device_normal(shape, seed, std=1.0):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return torch.randn(shape, device="cuda", generator=g) * std


@pytest.mark.parametrize("act", ["leaky", "mish", "logistic"])
def test_epilogue_largest_sweep_shape(ops, oracle, act):
    """64 x 16 x 416^2 (709 MB): images 0, 31 and 63 against the checker, in place == out of place."""
    import torch
    N, C, S = 64, 16, 416
    x = device_normal((N, C, S, S), 11)
    scale, bias, mean, var = wl.bn_params(2000, C)
    y = torch.empty_like(x)
    folded = ops.bn_fold(gpu(mean), gpu(var), gpu(scale), gpu(bias))
    ops.bn_folded_act_forward(x, y, folded, act)
    for n in (0, 31, 63):
        want = host(x[n:n + 1]).copy()
        oracle.conv_epilogue_forward(True, False, act, 1, C, S, S, want, None, np.zeros(C, F), np.zeros(C, F),
                                     mean.copy(), var.copy(), scale, bias, None, None)
        assert_close(host(y[n:n + 1]), want, 1e-5, 1e-3, "%s image %d" % (act, n))
    y2 = torch.empty_like(x)
    ops.bn_infer_act_forward(x, y2, gpu(mean), gpu(var), gpu(scale), gpu(bias), act)
    assert torch.equal(y, y2), "folded and two-launch entry points differ"
    ops.bn_folded_act_forward(x, x, folded, act)
    assert torch.equal(x, y), "in place differs from out of place"


def test_bn_training_largest_shape(ops, oracle):
    """16 x 32 x 608^2 (757 MB): statistics against fp64, batch-norm invariants forward and backward."""
    import torch
    N, C, S = 16, 32, 608
    x = device_normal((N, C, S, S), 12) * 1.7 + 0.3
    scale, bias, rmean, rvar = (gpu(a) for a in wl.bn_params(2001, C))
    mean = torch.zeros(C, device="cuda"); var = torch.zeros(C, device="cuda")
    y = torch.empty_like(x)
    ops.bn_train_act_forward(x, y, mean, var, rmean, rvar, scale, bias, "linear")
    x64 = x.double()
    m64 = x64.mean(dim=(0, 2, 3)); v64 = x64.var(dim=(0, 2, 3), unbiased=False)
    assert_close(host(mean), host(m64), 1e-6, 0.1, "batch mean vs fp64")
    assert_close(host(var), host(v64), 1e-6, 1.0, "batch variance vs fp64")
    # y = x_hat * scale + bias: per channel, mean(y) = bias and var(y) = (scale * sigma / (sigma + 1e-5))^2
    y64 = y.double()
    sig = v64.sqrt()
    assert_close(host(y64.mean(dim=(0, 2, 3))), host(bias.double()), 1e-5, 1.0, "mean of the normalised output")
    want_var = (scale.double() * sig / (sig + 1e-5)) ** 2
    assert_close(host(y64.var(dim=(0, 2, 3), unbiased=False)), host(want_var), 1e-5, 1.0, "variance of the output")
    # one image against the checker, given the batch statistics
    n = 7
    want = host(x[n:n + 1]).copy()
    hm, hv = host(mean), host(var)
    oracle.normalize(want, hm, hv, 1, C, S * S)
    oracle.scale_bias(want, host(scale), 1, C, S * S)
    oracle.add_bias(want, host(bias), 1, C, S * S)
    assert_close(host(y[n:n + 1]), want, 1e-5, 2.0, "image 7 given the statistics")
    del x64, y64
    # backward: dx is orthogonal to 1 and to x_hat within each channel
    d = device_normal((N, C, S, S), 13)
    su = torch.zeros(C, device="cuda"); bu = torch.zeros(C, device="cuda")
    d_in = d.clone()
    ops.bn_act_backward(d, x, mean, var, scale, bias, su, bu, "linear")
    assert_close(host(bu), host(d_in.double().sum(dim=(0, 2, 3))), 1e-5, 100.0, "bias updates vs fp64")
    xhat = (x.double() - m64.view(1, C, 1, 1)) / (sig + 1e-5).view(1, C, 1, 1)
    assert_close(host(su), host((d_in.double() * xhat).sum(dim=(0, 2, 3))), 1e-5, 100.0, "scale updates vs fp64")
    dx = d.double()
    norm = float(dx.abs().sum(dim=(0, 2, 3)).max())
    assert float(dx.sum(dim=(0, 2, 3)).abs().max()) <= 1e-5 * norm, "sum of dx per channel must vanish"
    assert float((dx * xhat).sum(dim=(0, 2, 3)).abs().max()) <= 2e-5 * norm, "dx must be orthogonal to x_hat"


@pytest.mark.parametrize("shape", [(16, 32, 608), (16, 256, 76), (16, 1024, 19)])
def test_bn_backward_clipped_at_training_shapes(ops, shape):
    """The rescale + clip folded into the backward at configs[4] shapes -- three launches with 11 552 norm partials,
    the one-launch form with part of the slice in LDS, the scalar one-launch form at 1024 channels -- against the
    two-call sequence it replaces (pxh_rescale_clip, then pxh_bn_act_backward; each held to the checker elsewhere):
    to the bit when nothing changes, within 1e-5 when the delta is rescaled or clamped."""
    import torch
    N, C, S = shape
    x = device_normal((N, C, S, S), 21) * 1.3 + 0.2
    scale, bias, rmean, rvar = (gpu(a) for a in wl.bn_params(2101, C))
    mean = torch.zeros(C, device="cuda"); var = torch.zeros(C, device="cuda")
    y = torch.empty_like(x)
    ops.bn_train_act_forward(x, y, mean, var, rmean, rvar, scale, bias, "leaky")
    del y
    delta = device_normal((N, C, S, S), 22)
    spiky = delta.clone()
    spiky[:, 0] *= 20.0
    norm = float(torch.linalg.vector_norm(delta.double()))
    spiky_norm = float(torch.linalg.vector_norm(spiky.double()))
    peak = float(delta.abs().max())
    cases = [("nothing changes", delta, 2.0 * norm, 2.0 * peak), ("rescale only", delta, 0.37 * norm, 0.0),
             ("rescale and clamp", delta, 0.5 * norm, 0.3),
             ("clamp in one channel only", spiky, 2.0 * spiky_norm, 1.5 * peak)]
    for name, d0, threshold, clip in cases:
        want = d0.clone(); su_w = torch.zeros(C, device="cuda"); bu_w = torch.zeros(C, device="cuda")
        norm_w = torch.zeros(1, device="cuda")
        ops.rescale_clip(want, threshold, clip, norm_out=norm_w)
        size = float(want.double().pow(2).mean().sqrt())
        ops.bn_act_backward(want, x, mean, var, scale, bias, su_w, bu_w, "leaky")
        got = d0.clone(); su = torch.zeros(C, device="cuda"); bu = torch.zeros(C, device="cuda")
        norm_g = torch.zeros(1, device="cuda")
        ops.bn_act_backward_clipped(got, x, mean, var, scale, bias, su, bu, "leaky", threshold, clip, norm_out=norm_g)
        what = "%s %s" % (shape, name)
        assert_close(host(norm_g), host(norm_w), 1e-6, 1e-30, what + " norm")
        if name == "nothing changes":
            assert torch.equal(got, want) and torch.equal(su, su_w) and torch.equal(bu, bu_w), what
        else:
            sums = float(np.sqrt(N * S * S)) * size
            assert_close(host(su), host(su_w), 1e-5, sums, what + " scale updates")
            assert_close(host(bu), host(bu_w), 1e-5, sums, what + " bias updates")
            worst = float(((got - want).abs() / want.abs().clamp_min(0.1 * size)).max())
            assert worst <= 1e-5, (what, worst)
        del want, got


@pytest.mark.parametrize("shape", [(16, 64, 304), (16, 256, 76), (16, 512, 38), (16, 1024, 19)])
def test_epilogue_with_shortcut_at_training_shapes(ops, shape):
    """A residual block's shortcut taken into the epilogue of the convolution in front of it, at the shapes of
    YOLOv3's blocks at batch 16 -- three launches, the one-launch form with part of the slice in LDS, the 128-bit
    and the scalar one-launch forms -- against the two calls it replaces (each held to the checker elsewhere)."""
    import torch
    N, C, S = shape
    x = device_normal((N, C, S, S), 31) * 1.3 + 0.2
    frm = device_normal((N, C, S, S), 32)
    scale, bias, rmean, rvar = (gpu(a) for a in wl.bn_params(3101, C))
    m0, v0, m1, v1 = (torch.zeros(C, device="cuda") for _ in range(4))
    rm0, rv0, rm1, rv1 = rmean.clone(), rvar.clone(), rmean.clone(), rvar.clone()
    y = torch.empty_like(x); want = torch.empty_like(x)
    ops.bn_train_act_forward(x, y, m0, v0, rm0, rv0, scale, bias, "leaky")
    ops.shortcut_forward(y, frm, want, "linear")
    del y
    got = torch.empty_like(x)
    ops.bn_train_act_shortcut_forward(x, got, m1, v1, rm1, rv1, scale, bias, "leaky", frm)
    if S % 2 == 0 or C < 512:
        assert torch.equal(got, want) and torch.equal(m1, m0) and torch.equal(v1, v0) and torch.equal(rm1, rm0), shape
    else:
        # 1024 scalar slices: alone, the layer adds its statistics up with workgroups of half the size
        assert_close(host(m1), host(m0), 2e-6, 1.0, "mean")
        assert_close(host(v1), host(v0), 2e-6, 1.0, "var")
        worst = float(((got - want).abs() / (want.abs() + frm.abs()).clamp_min(1.0)).max())
        assert worst <= 2e-6, (shape, worst)


def test_maxpool_largest_shape(ops, oracle):
    """16 x 64 x 304^2: whole tensor against the checker and against an independent routine."""
    import torch
    N, C, S = 16, 64, 304
    x = device_normal((N, C, S, S), 14)
    out = torch.empty((N, C, S // 2, S // 2), device="cuda")
    idx = torch.empty((N, C, S // 2, S // 2), device="cuda", dtype=torch.int32)
    ops.maxpool_forward(x, out, idx, 2, 2, 1)
    hx = host(x)
    want = np.empty(out.shape, F); widx = np.empty(out.shape, np.int32)
    oracle.maxpool_forward(hx, want, widx, N, C, S, S, S // 2, S // 2, 2, 2, 1)
    assert_bit_exact(host(out), want, "max-pool values")
    assert_bit_exact(host(idx), widx, "max-pool indexes")
    ref, ref_idx = torch.nn.functional.max_pool2d(x, 2, 2, return_indices=True)
    assert torch.equal(ref, out), "values differ from torch max_pool2d"
    assert torch.equal(x.flatten()[idx.flatten().long()], out.flatten()), "indexes do not point at the maxima"
    # backward: windows do not overlap, so every grad cell receives at most one delta
    delta = device_normal(out.shape, 15)
    grad0 = device_normal(x.shape, 16)
    grad = grad0.clone()
    ops.maxpool_backward(delta, idx, grad, 2, 2, 1)
    expect = grad0.flatten().index_put((idx.flatten().long(),), delta.flatten(), accumulate=True).view_as(grad0)
    assert torch.equal(grad, expect), "backward differs from a scatter-add"
    assert abs(float((grad.double() - grad0.double()).sum()) - float(delta.double().sum())) < 1e-6 * delta.numel()


def test_upsample_and_route_full_shapes(ops, oracle):
    import torch
    N = 16
    for c, s in wl.YOLOV3_UPSAMPLE_SHAPES:
        x = device_normal((N, c, s, s), 17)
        out = torch.empty((N, c, 2 * s, 2 * s), device="cuda")
        ops.upsample_forward(x, out, 2, 1.0)
        for dy in (0, 1):
            for dx in (0, 1):
                assert torch.equal(out[:, :, dy::2, dx::2], x), "upsample replica (%d,%d)" % (dy, dx)
        want = np.empty(out.shape, F)
        oracle.upsample(host(x), s, s, c, N, 2, True, 1.0, None, want)
        assert_bit_exact(host(out), want, "upsample forward %dx%d" % (c, s))
        acc0 = device_normal(x.shape, 18)
        acc = acc0.clone()
        ops.upsample_backward(out, acc, 2, 1.0)
        expect = (((acc0 + out[:, :, 0::2, 0::2]) + out[:, :, 0::2, 1::2]) + out[:, :, 1::2, 0::2]) + out[:, :, 1::2, 1::2]
        assert torch.equal(acc, expect), "upsample backward raster-order sum"
        # concat with the skip connection of twice the channels, as YOLOv3 does
        skip = device_normal((N, 2 * c, 2 * s, 2 * s), 19)
        route = torch.empty((N, 3 * c, 2 * s, 2 * s), device="cuda")
        ops.route_forward(out, route, 0)
        ops.route_forward(skip, route, c * 4 * s * s)
        assert torch.equal(route, torch.cat([out, skip], dim=1)), "route forward is a concatenation"
        d_up = device_normal(out.shape, 20); d_skip = device_normal(skip.shape, 21)
        e_up = d_up + route[:, :c]; e_skip = d_skip + route[:, c:]
        ops.route_backward(route, d_up, 0)
        ops.route_backward(route, d_skip, c * 4 * s * s)
        assert torch.equal(d_up, e_up) and torch.equal(d_skip, e_skip), "route backward adds the slices"


def test_shortcut_largest_shape(ops, oracle):
    import torch
    N, C, S = 16, 64, 304
    a = device_normal((N, C, S, S), 22); b = device_normal((N, C, S, S), 23)
    out = torch.empty_like(a)
    ops.shortcut_forward(a, b, out, "linear")
    assert torch.equal(out, a + b), "shortcut forward is one rounded add"
    want = np.empty((1, C, S, S), F); pre = np.empty((1, C, S, S), F)
    oracle.shortcut_forward("linear", 1, S, S, C, host(a[3:4]), host(b[3:4]), 1.0, 1.0, want, pre)
    assert_bit_exact(host(out[3:4]), want, "image 3 against the checker")
    delta = device_normal(a.shape, 24)
    from_delta0 = device_normal(a.shape, 25); grad0 = device_normal(a.shape, 26)
    from_delta = from_delta0.clone(); grad = grad0.clone()
    ops.shortcut_backward(delta, from_delta, grad, "linear")
    assert torch.equal(from_delta, from_delta0 + delta) and torch.equal(grad, grad0 + delta)


def test_yolo_largest_head(ops, oracle):
    """64 x 255 x 76^2: the whole head against the checker, cost == checksum of delta, bit-identical repeat."""
    from test_gpu_yolo_adam import compare_head, gpu_head, oracle_head
    N, K, W = 64, 80, 76
    x = wl.normal(5076, (N, 3 * (K + 5), W, W), std=2.0)
    truths, counts = wl.yolo_truths(5100, N)
    kw = dict(ignore_thresh=0.7, truth_thresh=1.0, coord_scale=1.0, object_scale=2.0, noobject_scale=0.1,
              class_scale=1.0)
    mask = wl.YOLOV3_MASKS[W]
    got = gpu_head(ops, x, truths, counts, W, W, K, mask, wl.YOLOV3_ANCHORS, 608, **kw)
    want = oracle_head(oracle, x, truths, counts, W, W, K, mask, wl.YOLOV3_ANCHORS, 608, **kw)
    # The CPU layer forms its statistics as running fp32 sums over 1.1 M slots; addends below half
    # an ulp of the running sum are lost, which biases those sums low by up to ~1e-3 relative.  So
    # they are compared with the CPU's to 2e-3 only, and with fp64 sums of the kernel's own output
    # and delta to 1e-6.
    compare_head(got, want, "head 76 at batch 64", 3, kw, sum_rtol=2e-3)
    out, delta, cost, stats = got
    o4 = out.reshape(N, 3, K + 5, W * W).astype(np.float64)
    d4 = delta.reshape(N, 3, K + 5, W * W).astype(np.float64)
    dobj = d4[:, :, 4]
    exact = {5: o4[:, :, 4].sum(), 8: np.square(d4[:, :, :4]).sum(), 9: np.square(dobj[dobj >= 0]).sum(),
             10: np.square(dobj[dobj < 0]).sum(), 11: np.square(d4[:, :, 5:]).sum()}
    for k, v in exact.items():
        assert abs(stats[k] - v) <= 1e-6 * max(v, 1.0), ("statistic %d vs fp64" % k, stats[k], v)
    checksum = float(np.square(delta.astype(np.float64)).sum())
    assert abs(cost - checksum) <= 1e-5 * checksum, (cost, checksum)
    v = out.reshape(N, 3, K + 5, W * W); xi = x.reshape(N, 3, K + 5, W * W)
    assert_bit_exact(v[:, :, 2:4], xi[:, :, 2:4], "raw w/h entries are copies")
    again = gpu_head(ops, x, truths, counts, W, W, K, mask, wl.YOLOV3_ANCHORS, 608, **kw)
    assert_bit_exact(again[1], delta, "delta of a second run")
    assert again[2] == cost and np.array_equal(again[3], stats), "cost and statistics must not depend on timing"


def test_yolo_three_heads_at_full_batch_in_one_pass(ops, oracle):
    """64 x 255 x {19, 38, 76}^2 through pxh_yolo_forward_train_heads: every head against the checker run head by
    head on the same logits and truths; every truth claims exactly one slot on the head that holds its best
    anchor; each head's cost is the checksum of its delta."""
    from test_gpu_yolo_adam import compare_head, oracle_head
    from test_gpu_yolo_heads import run_heads
    N, K = 64, 80
    sizes = [19, 38, 76]
    masks = [wl.YOLOV3_MASKS[s] for s in sizes]
    xs = [wl.normal(5000 + W, (N, 3 * (K + 5), W, W), std=2.0) for W in sizes]
    truths, counts = wl.yolo_truths(5100, N)
    kw = dict(ignore_thresh=0.7, truth_thresh=1.0, coord_scale=1.0, object_scale=2.0, noobject_scale=0.1,
              class_scale=1.0)
    got = run_heads(ops, xs, truths, counts, sizes, K, masks, wl.YOLOV3_ANCHORS, 608, [kw] * 3)
    positives = 0
    for x, W, mask, g in zip(xs, sizes, masks, got):
        want = oracle_head(oracle, x, truths, counts, W, W, K, mask, wl.YOLOV3_ANCHORS, 608, **kw)
        # the CPU layer's statistics are running fp32 sums over up to 1.1 M slots (see test_yolo_largest_head)
        compare_head(g, want, "head %d of three at batch 64" % W, 3, kw, sum_rtol=2e-3)
        positives += want[3][6]
        checksum = float(np.square(g[1].astype(np.float64)).sum())
        assert abs(g[2] - checksum) <= 1e-5 * checksum, (W, g[2], checksum)
    assert positives == counts.sum()


def test_yolo_one_launch_sums_do_not_depend_on_arrival_order(ops, oracle):
    """64 x 255 x 19^2 in the one-launch form, where whichever head workgroup finishes last adds up the
    sums of all of them: cost, statistics and every delta are bit-identical from run to run, for each
    number of lanes per slot, and the runs of different lane counts agree to the checker's tolerance."""
    from test_gpu_yolo_adam import compare_head, gpu_head, oracle_head
    from pixienn_amd import capi
    lib = capi.load()
    N, K, W = 64, 80, 19
    x = wl.normal(5019, (N, 3 * (K + 5), W, W), std=2.0)
    truths, counts = wl.yolo_truths(5101, N)
    kw = dict(ignore_thresh=0.7, truth_thresh=1.0, coord_scale=1.0, object_scale=2.0, noobject_scale=0.1,
              class_scale=1.0)
    mask = wl.YOLOV3_MASKS[W]
    want = oracle_head(oracle, x, truths, counts, W, W, K, mask, wl.YOLOV3_ANCHORS, 608, **kw)
    try:
        for lanes in (1, 2, 4):
            lib.pxh_debug_yolo_tuning(1, lanes, 0)
            first = gpu_head(ops, x, truths, counts, W, W, K, mask, wl.YOLOV3_ANCHORS, 608, **kw)
            compare_head(first, want, "19^2 at batch 64, %d lanes per slot" % lanes, 3, kw, sum_rtol=2e-4)
            for _ in range(3):
                again = gpu_head(ops, x, truths, counts, W, W, K, mask, wl.YOLOV3_ANCHORS, 608, **kw)
                assert_bit_exact(again[1], first[1], "delta of a repeated run")
                assert again[2] == first[2] and np.array_equal(again[3], first[3]), "sums must not depend on timing"
    finally:
        lib.pxh_debug_yolo_tuning(0, 0, 0)


@pytest.mark.parametrize("decay_form", [1, 2])
def test_adam_full_parameter_buffer(ops, oracle, decay_form):
    """61.9 M parameters, 10 steps: the first, a middle and the last million against the checker, with the
    reference's L2 term (1) and with the decoupled decay the baseline's configuration names (2)."""
    import torch
    P = wl.YOLOV3_PARAMS
    w = device_normal((P,), 27, 0.02); g = device_normal((P,), 28, 1e-3)
    m = torch.zeros(P, device="cuda"); v = torch.zeros(P, device="cuda")
    d = torch.empty(P, device="cuda")
    spans = [(0, 1 << 20), (P // 2 - 3, P // 2 - 3 + (1 << 20)), (P - (1 << 20) - 1, P)]
    hw = [host(w[a:b]).copy() for a, b in spans]
    hg = [host(g[a:b]).copy() for a, b in spans]
    hm = [np.zeros(b - a, F) for a, b in spans]; hv = [np.zeros(b - a, F) for a, b in spans]
    for t in range(1, 11):
        d.copy_(g)
        ops.adam_update(w, d, m, v, 16, t, 1e-3, 0.9, 0.999, 1e-8, 5e-4, decay_form)
        for k in range(len(spans)):
            hd = hg[k].copy()
            oracle.adam_update(hw[k], hd, hm[k], hv[k], 16, t, 1e-3, 0.9, 0.999, 1e-8, 5e-4, decay_form)
    assert float(d.abs().max()) == 0.0, "the update buffer must be zero after a step"
    for k, (a, b) in enumerate(spans):
        assert_close(host(w[a:b]), hw[k], 1e-6, 1e-3, "weights of span %d" % k)
        assert_close(host(m[a:b]), hm[k], 1e-6, 1e-6, "first moment of span %d" % k)
        assert_close(host(v[a:b]), hv[k], 1e-6, 1e-12, "second moment of span %d" % k)
    assert bool(torch.isfinite(w).all())
