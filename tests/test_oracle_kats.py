"""Pins the CPU checker (oracle/) against the known-answer vectors the reference's own
unit tests hold (tests/golden/reference_kats.json) and against the reference's own
Activation.h compiled as oracle/_ref.  No GPU."""
import math
import os

import numpy as np
import pytest

from util import detection_records, random_detections

F = np.float32


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def float_eq(a, b):
    """gtest's EXPECT_FLOAT_EQ: within 4 ULPs."""
    a = np.float32(a)
    b = np.float32(b)
    if a == b:
        return True
    ia = int(np.array(a, np.float32).view(np.int32))
    ib = int(np.array(b, np.float32).view(np.int32))
    # map sign-magnitude to a monotone integer line
    ia = ia if ia >= 0 else -(ia & 0x7FFFFFFF)
    ib = ib if ib >= 0 else -(ib & 0x7FFFFFFF)
    return abs(ia - ib) <= 4


# ---------------------------------------------------------------- activations
def test_activation_kats(oracle, kats):
    for case in kats["activations"]["cases"]:
        x = f32(case["input"])
        if case["apply"] is not None:
            y = oracle.activate(case["name"], x.copy())
            for got, want in zip(y, case["apply"]):
                assert float_eq(got, want), (case["name"], got, want)
        d = oracle.gradient(case["name"], x, f32(case["delta"]))
        for got, want in zip(d, case["gradient"]):
            if "gradient_tol" in case:
                assert abs(float(got) - want) <= case["gradient_tol"], (case["name"], got, want)
            else:
                assert float_eq(got, want), (case["name"], got, want)


def test_activation_matches_compiled_reference(oracle):
    """Bit-for-bit against the reference's Activation.h (oracle/_ref), all 9 activations,
    over a dense sweep that crosses the softplus thresholds at +-20."""
    if oracle.ref_lib() is None:
        pytest.skip("oracle/_ref was not built (reference tree absent at build time)")
    rng = np.random.default_rng(7)
    x = np.concatenate([
        np.linspace(-30, 30, 24001, dtype=np.float32),
        rng.standard_normal(20000).astype(np.float32) * 3,
        f32([0.0, -0.0, 20.0, -20.0, 20.000002, -20.000002, 1e-30, -1e-30, 88.0, -88.0, 100.0, -104.0]),
    ]).astype(np.float32)
    d = rng.standard_normal(x.size).astype(np.float32)
    for name in oracle.ACTIVATIONS:
        a = oracle.activate(name, x.copy())
        b = oracle.ref_activate(name, x.copy())
        assert np.array_equal(a.view(np.int32), b.view(np.int32)), name
        ga = oracle.gradient(name, x, d.copy())
        gb = oracle.ref_gradient(name, x, d.copy())
        assert np.array_equal(ga.view(np.int32), gb.view(np.int32)), name


def test_activation_closed_forms(oracle):
    x = np.linspace(-8, 8, 1001, dtype=np.float32)
    xd = x.astype(np.float64)
    sig = 1 / (1 + np.exp(-xd))
    sp = np.log1p(np.exp(xd))
    want = {"logistic": sig, "swish": xd * sig, "mish": xd * np.tanh(sp), "leaky": np.where(xd > 0, xd, 0.1 * xd),
            "tanh": np.tanh(xd), "relu": np.maximum(xd, 0), "softplus": sp, "loggy": 2 * sig - 1}
    for name, w in want.items():
        got = oracle.activate(name, x.copy()).astype(np.float64)
        assert np.max(np.abs(got - w)) < 2e-6, name
    # derivative by central differences of the closed form
    h = 1e-4
    fns = {"logistic": lambda t: 1 / (1 + np.exp(-t)), "swish": lambda t: t / (1 + np.exp(-t)),
           "mish": lambda t: t * np.tanh(np.log1p(np.exp(t))), "tanh": np.tanh,
           "softplus": lambda t: np.log1p(np.exp(t))}
    ones = np.ones_like(x)
    for name, fn in fns.items():
        got = oracle.gradient(name, x, ones.copy()).astype(np.float64)
        fd = (fn(xd + h) - fn(xd - h)) / (2 * h)
        assert np.max(np.abs(got - fd)) < 2e-5, name


# ---------------------------------------------------------------- BN primitives
def test_blas_kats(oracle, kats):
    k = kats["blas"]
    assert float_eq(oracle.mag_array(f32(k["mag_array"]["input"])), math.sqrt(k["mag_array"]["expected_sq"]))
    assert float_eq(oracle.sum_array(f32(k["sum_array"]["input"])), k["sum_array"]["expected"])

    for key in ("backward_bias", "backward_bias_gpu"):
        c = k[key]
        bu = f32(c["bias_updates"])
        oracle.backward_bias(bu, f32(c["delta"]), c["batch"], c["n"], c["size"])
        assert bu.tolist() == c["expected"]

    c = k["add_bias"]
    out = np.full(c["batch"] * c["n"] * c["size"], c["fill"], F)
    oracle.add_bias(out, np.full(c["n"], c["bias_fill"], F), c["batch"], c["n"], c["size"])
    assert all(float_eq(v, c["expected_each"]) for v in out)

    c = k["scale_bias"]
    out = np.full(c["batch"] * c["n"] * c["size"], c["fill"], F)
    oracle.scale_bias(out, np.full(c["n"], c["scale_fill"], F), c["batch"], c["n"], c["size"])
    assert all(float_eq(v, c["expected_each"]) for v in out)

    c = k["backward_scale"]
    su = np.zeros(c["n"], F)
    oracle.backward_scale(f32(c["xnorm"]), np.full(len(c["xnorm"]), c["delta_fill"], F), c["batch"], c["n"],
                          c["size"], su)
    assert su.tolist() == c["expected"]

    c = k["mean"]
    m = np.zeros(c["filters"], F)
    oracle.mean(f32(c["input"]), c["batch"], c["filters"], c["spatial"], m)
    assert all(float_eq(v, w) for v, w in zip(m, c["expected"]))

    c = k["variance"]
    v = np.zeros(c["filters"], F)
    oracle.variance(f32(c["input"]), f32(c["mean"]), c["batch"], c["filters"], c["spatial"], v)
    assert np.allclose(v, c["expected"], atol=c["tol"], rtol=0)

    for key in ("mean_delta", "mean_delta_signs"):
        c = k[key]
        md = np.zeros(c["filters"], F)
        oracle.mean_delta(f32(c["delta"]), f32(c["variance"]), c["batch"], c["filters"], c["spatial"], md)
        assert np.allclose(md, c["expected"], atol=c["tol"], rtol=0), key

    c = k["variance_delta"]
    vd = np.zeros(c["filters"], F)
    oracle.variance_delta(f32(c["x"]), f32(c["delta"]), f32(c["mean"]), f32(c["variance"]), c["batch"],
                          c["filters"], c["spatial"], vd)
    assert np.allclose(vd, c["expected"], atol=c["tol"], rtol=0)

    c = k["normalize_delta"]
    d = np.full(len(c["x"]), c["delta_fill"], F)
    oracle.normalize_delta(f32(c["x"]), f32(c["mean"]), f32(c["variance"]), f32(c["mean_delta"]),
                           f32(c["variance_delta"]), c["batch"], c["filters"], c["spatial"], d)
    assert np.allclose(d, c["expected"], atol=c["tol"], rtol=0)


def _bn_buffers(rng, N, C, H, W):
    x = rng.standard_normal((N, C, H, W)).astype(F) * 1.7 + 0.3
    scales = (1 + 0.2 * rng.standard_normal(C)).astype(F)
    biases = (0.1 * rng.standard_normal(C)).astype(F)
    rmean = (0.1 * rng.standard_normal(C)).astype(F)
    rvar = rng.uniform(0.5, 1.5, C).astype(F)
    return x, scales, biases, rmean, rvar


def test_bn_inference_closed_form(oracle):
    """y = (x - rmean) / (sqrt(rvar) + 1e-5) * scale + bias, the eps OUTSIDE the root."""
    rng = np.random.default_rng(11)
    N, C, H, W = 3, 5, 7, 6
    x, scales, biases, rmean, rvar = _bn_buffers(rng, N, C, H, W)
    out = np.empty_like(x)
    mean = np.zeros(C, F); var = np.zeros(C, F)
    rm, rv = rmean.copy(), rvar.copy()
    oracle.batchnorm_forward(False, N, C, H, W, x, out, mean, var, rm, rv, scales, biases, None, None)
    sh = (1, C, 1, 1)
    want = (x.astype(np.float64) - rmean.reshape(sh)) / (np.sqrt(rvar.astype(np.float64)).reshape(sh) + 1e-5) \
        * scales.reshape(sh) + biases.reshape(sh)
    assert np.max(np.abs(out - want)) < 2e-6
    # the textbook sqrt(var + eps) convention must NOT be what is computed
    text = (x.astype(np.float64) - rmean.reshape(sh)) / np.sqrt(rvar.astype(np.float64) + 1e-5).reshape(sh) \
        * scales.reshape(sh) + biases.reshape(sh)
    assert np.max(np.abs(out - want)) < 0.2 * np.max(np.abs(text - want))
    assert np.array_equal(rm, rmean) and np.array_equal(rv, rvar)


def test_bn_training_forward_invariants(oracle):
    rng = np.random.default_rng(12)
    N, C, H, W = 4, 6, 9, 5
    x, scales, biases, rmean, rvar = _bn_buffers(rng, N, C, H, W)
    out = np.empty_like(x); xs = np.empty_like(x); xn = np.empty_like(x)
    mean = np.zeros(C, F); var = np.zeros(C, F)
    rm, rv = rmean.copy(), rvar.copy()
    oracle.batchnorm_forward(True, N, C, H, W, x, out, mean, var, rm, rv, scales, biases, xs, xn)
    x64 = x.astype(np.float64)
    mu = x64.mean(axis=(0, 2, 3)); va = x64.var(axis=(0, 2, 3))          # population variance
    assert np.allclose(mean, mu, atol=2e-6) and np.allclose(var, va, rtol=2e-6)
    assert np.array_equal(xs, x)
    assert np.allclose(rm, 0.99 * rmean + 0.01 * mu, atol=1e-6)
    assert np.allclose(rv, 0.99 * rvar + 0.01 * va, atol=1e-6)
    # x-hat: zero mean and (nearly) unit second moment per channel
    assert np.max(np.abs(xn.astype(np.float64).mean(axis=(0, 2, 3)))) < 1e-6
    assert np.allclose((xn.astype(np.float64) ** 2).mean(axis=(0, 2, 3)), 1.0, atol=1e-4)
    sh = (1, C, 1, 1)
    assert np.allclose(out, xn * scales.reshape(sh) + biases.reshape(sh), atol=1e-6)
    # wide variant agrees closely at this size
    out2 = np.empty_like(x); mean2 = np.zeros(C, F); var2 = np.zeros(C, F)
    oracle.batchnorm_forward(True, N, C, H, W, x, out2, mean2, var2, rmean.copy(), rvar.copy(), scales, biases,
                             np.empty_like(x), np.empty_like(x), wide=True)
    assert np.allclose(out, out2, atol=1e-5)


def test_bn_backward_matches_autograd_up_to_eps_convention(oracle):
    """dx of the restated backward against torch autograd of textbook BN in fp64.  The
    two differ only through the epsilon placement (forward sqrt(var)+eps, backward
    sqrt(var+eps)), an O(1e-5) relative effect."""
    import torch
    rng = np.random.default_rng(13)
    N, C, H, W = 3, 4, 5, 6
    x, scales, biases, rmean, rvar = _bn_buffers(rng, N, C, H, W)
    delta = rng.standard_normal(x.shape).astype(F)
    out = np.empty_like(x); xs = np.empty_like(x); xn = np.empty_like(x)
    mean = np.zeros(C, F); var = np.zeros(C, F)
    oracle.batchnorm_forward(True, N, C, H, W, x, out, mean, var, rmean.copy(), rvar.copy(), scales, biases, xs, xn)
    d = delta.copy()
    md = np.zeros(C, F); vd = np.zeros(C, F); su = np.full(C, 0.5, F); bu = np.full(C, -0.25, F)
    oracle.batchnorm_backward(N, C, H, W, d, mean, var, md, vd, scales, su, bu, xs, xn)

    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    g = torch.tensor(scales, dtype=torch.float64, requires_grad=True)
    b = torch.tensor(biases, dtype=torch.float64, requires_grad=True)
    y = torch.nn.functional.batch_norm(xt, None, None, g, b, training=True, eps=1e-5)
    y.backward(torch.tensor(delta, dtype=torch.float64))
    assert np.max(np.abs(d - xt.grad.numpy())) < 5e-5
    # updates ACCUMULATE onto what was there
    assert np.allclose(bu + 0.25, b.grad.numpy(), atol=2e-5)
    assert np.allclose(su - 0.5, g.grad.numpy(), atol=1e-4)


def test_conv_epilogue_order(oracle):
    """bias / BN first, then the pre-activation copy, then the activation."""
    rng = np.random.default_rng(14)
    N, C, H, W = 2, 3, 4, 4
    x, scales, biases, rmean, rvar = _bn_buffers(rng, N, C, H, W)
    out = x.copy(); pre = np.empty_like(x)
    oracle.conv_epilogue_forward(False, False, "leaky", N, C, H, W, out, pre, None, None, None, None, None,
                                 biases, None, None)
    want_pre = x + biases.reshape(1, C, 1, 1)
    assert np.array_equal(pre, want_pre)
    assert np.array_equal(out, np.where(want_pre > 0, want_pre, F(0.1) * want_pre))
    d = rng.standard_normal(x.shape).astype(F); d0 = d.copy()
    bu = np.zeros(C, F)
    oracle.conv_epilogue_backward(False, "leaky", N, C, H, W, d, pre, None, None, None, None, None, None, bu,
                                  None, None)
    assert np.array_equal(d, d0 * np.where(pre > 0, F(1), F(0.1)))
    assert np.allclose(bu, d.sum(axis=(0, 2, 3)), atol=1e-5)


# ---------------------------------------------------------------- max-pool
def test_maxpool_kat(oracle, kats):
    c = kats["maxpool"]
    n = c["oh"] * c["ow"]
    out = np.zeros(n, F); idx = np.full(n, -7, np.int32)
    oracle.maxpool_forward(f32(c["input"]), out, idx, c["batch"], c["channels"], c["ih"], c["iw"], c["oh"],
                           c["ow"], c["kernel"], c["stride"], c["padding"])
    assert out.tolist() == c["expected_out"]
    grad = np.full(c["ih"] * c["iw"], c["grad_fill"], F)
    oracle.maxpool_backward(np.full(n, c["delta_fill"], F), idx, grad)
    assert grad.tolist() == c["expected_grad"]
    assert oracle.maxpool_out_dim(3, 2, 1, 1) == 3
    assert oracle.maxpool_out_dim(416, 2, 2, 1) == 208
    assert oracle.maxpool_out_dim(13, 2, 1, 1) == 13


def test_maxpool_vs_torch_and_ties(oracle):
    import torch
    rng = np.random.default_rng(21)
    N, C, H, W = 2, 3, 8, 10
    # few distinct values -> many ties; torch keeps the first maximum as well
    x = rng.integers(-2, 3, (N, C, H, W)).astype(F)
    oh, ow = oracle.maxpool_out_dim(H, 2, 2, 1), oracle.maxpool_out_dim(W, 2, 2, 1)
    out = np.zeros((N, C, oh, ow), F); idx = np.zeros((N, C, oh, ow), np.int32)
    oracle.maxpool_forward(x, out, idx, N, C, H, W, oh, ow, 2, 2, 1)
    tv, ti = torch.nn.functional.max_pool2d(torch.tensor(x), 2, 2, return_indices=True)
    assert np.array_equal(out, tv.numpy())
    plane = (np.arange(N * C).reshape(N, C, 1, 1) * H * W)
    assert np.array_equal(idx, ti.numpy() + plane)
    # -0.0 does not replace +0.0 (strict >), NaN first is sticky
    z = f32([0.0, -0.0, -0.0, 0.0]).reshape(1, 1, 2, 2)
    o1 = np.zeros(1, F); i1 = np.zeros(1, np.int32)
    oracle.maxpool_forward(z, o1, i1, 1, 1, 2, 2, 1, 1, 2, 2, 1)
    assert i1[0] == 0
    z = f32([np.nan, 5.0, 6.0, 7.0]).reshape(1, 1, 2, 2)
    oracle.maxpool_forward(z, o1, i1, 1, 1, 2, 2, 1, 1, 2, 2, 1)
    assert i1[0] == 0 and np.isnan(o1[0])
    z = f32([1.0, np.nan, 6.0, 7.0]).reshape(1, 1, 2, 2)
    oracle.maxpool_forward(z, o1, i1, 1, 1, 2, 2, 1, 1, 2, 2, 1)
    assert i1[0] == 3 and o1[0] == 7.0


# ---------------------------------------------------------------- upsample / shortcut
def test_upsample_closed_form(oracle):
    import torch
    rng = np.random.default_rng(31)
    N, C, H, W = 2, 3, 4, 5
    x = rng.standard_normal((N, C, H, W)).astype(F)
    out = np.zeros((N, C, 2 * H, 2 * W), F)
    oracle.upsample(x, W, H, C, N, 2, True, 1.0, None, out)
    assert np.array_equal(out, np.repeat(np.repeat(x, 2, axis=2), 2, axis=3))
    assert np.array_equal(out, torch.nn.functional.interpolate(torch.tensor(x), scale_factor=2, mode="nearest").numpy())
    # backward: raster-order accumulation ((g + a) + b) + c) + d, scale applied per term
    d = rng.standard_normal(out.shape).astype(F)
    g0 = rng.standard_normal(x.shape).astype(F)
    g = g0.copy()
    s = F(0.75)
    oracle.upsample(None, W, H, C, N, 2, False, float(s), g, d)
    want = g0.copy()
    for dy in (0, 1):
        for dx in (0, 1):
            want = want + s * d[:, :, dy::2, dx::2]
    assert np.array_equal(g, want)


def test_shortcut_closed_form(oracle):
    rng = np.random.default_rng(32)
    N, C, H, W = 2, 3, 4, 5
    a = rng.standard_normal((N, C, H, W)).astype(F)
    b = rng.standard_normal((N, C, H, W)).astype(F)
    out = np.empty_like(a); pre = np.empty_like(a)
    oracle.shortcut_forward("linear", N, W, H, C, a, b, 1.0, 1.0, out, pre)
    assert np.array_equal(out, a + b) and np.array_equal(pre, out)
    al, be = F(0.5), F(1.25)
    oracle.shortcut_forward("leaky", N, W, H, C, a, b, float(al), float(be), out, pre)
    want = al * a + be * b
    assert np.array_equal(pre, want)
    assert np.array_equal(out, np.where(want > 0, want, F(0.1) * want))
    d0 = rng.standard_normal(a.shape).astype(F)
    fd0 = rng.standard_normal(a.shape).astype(F)
    g0 = rng.standard_normal(a.shape).astype(F)
    d, fd, g = d0.copy(), fd0.copy(), g0.copy()
    oracle.shortcut_backward("leaky", N, W, H, C, d, pre, fd, g, float(al), float(be))
    dd = d0 * np.where(pre > 0, F(1), F(0.1))
    assert np.array_equal(d, dd)
    assert np.array_equal(fd, F(1.0) * fd0 + be * dd)
    assert np.array_equal(g, g0 + al * dd)
    # mismatched spatial ratios are an error in the reference
    assert oracle.shortcut(1, 4, 4, 1, a, 2, 4, 1, 1.0, 1.0, out) != 0


def test_route_is_channel_concat_and_slice_add(oracle):
    """Route has no reference test: forward is np.concatenate over channels (include/RouteLayer.h:91-113),
    backward adds each source's channel slice of the route's delta to that source's delta (115-137)."""
    rng = np.random.default_rng(33)
    N, H, W = 3, 4, 5
    a = rng.standard_normal((N, 2, H, W)).astype(F)
    b = rng.standard_normal((N, 5, H, W)).astype(F)
    c = rng.standard_normal((N, 1, H, W)).astype(F)
    out = np.full((N, 8, H, W), np.nan, F)
    at = 0
    for src in (a, b, c):
        oracle.route_forward(src, out, at)
        at += src[0].size
    assert np.array_equal(out, np.concatenate([a, b, c], axis=1))
    d = rng.standard_normal(out.shape).astype(F)
    da0, db0, dc0 = (rng.standard_normal(t.shape).astype(F) for t in (a, b, c))
    da, db, dc = da0.copy(), db0.copy(), dc0.copy()
    at = 0
    for dst in (da, db, dc):
        oracle.route_backward(d, dst, at)
        at += dst[0].size
    assert np.array_equal(da, da0 + d[:, 0:2]) and np.array_equal(db, db0 + d[:, 2:7])
    assert np.array_equal(dc, dc0 + d[:, 7:8])
    # a transposed or batch-strided mistake would show with N > 1 and unequal source sizes; so would "=" for "+="
    assert not np.array_equal(db, d[:, 2:7])


# ---------------------------------------------------------------- boxes
def test_darkbox_kats(oracle, kats):
    c = kats["darkbox"]
    assert float_eq(oracle.box_intersection(c["box1"], c["box2"]), c["intersection"])
    assert float_eq(oracle.box_union(c["box1"], c["box2"]), c["union"])
    assert float_eq(oracle.box_iou(c["box1"], c["box2"]), c["iou"])


def test_iou_brute_force(oracle):
    rng = np.random.default_rng(41)
    for _ in range(2000):
        a = rng.uniform(-0.5, 1.5, 2).tolist() + rng.uniform(0.01, 1.0, 2).tolist()
        b = rng.uniform(-0.5, 1.5, 2).tolist() + rng.uniform(0.01, 1.0, 2).tolist()
        iw = max(0.0, min(a[0] + a[2] / 2, b[0] + b[2] / 2) - max(a[0] - a[2] / 2, b[0] - b[2] / 2))
        ih = max(0.0, min(a[1] + a[3] / 2, b[1] + b[3] / 2) - max(a[1] - a[3] / 2, b[1] - b[3] / 2))
        inter = iw * ih
        union = a[2] * a[3] + b[2] * b[3] - inter
        assert abs(oracle.box_iou(a, b) - inter / union) < 1e-5
    assert oracle.box_iou([0.5, 0.5, 0.0, 0.3], [0.5, 0.5, 0.2, 0.2]) == 0.0   # empty operand
    assert oracle.box_iou([0.5, 0.5, 0.0, 0.0], [0.5, 0.5, 0.0, 0.0]) == 0.0   # zero union
    assert oracle.box_iou([0.2, 0.2, 0.1, 0.1], [0.8, 0.8, 0.1, 0.1]) == 0.0   # disjoint


# ---------------------------------------------------------------- YOLO
def _truth_arrays(truth_lists, max_truth=None):
    n = len(truth_lists)
    mt = max(1, max(len(t) for t in truth_lists)) if max_truth is None else max_truth
    tr = np.zeros((n, mt, 5), F)
    cnt = np.zeros(n, np.int32)
    for b, tl in enumerate(truth_lists):
        cnt[b] = len(tl)
        for t, row in enumerate(tl):
            tr[b, t] = row
    return tr, cnt, mt


def test_yolo_target_builder_kats(oracle, kats):
    c = kats["yolo_target_builder"]["collision"]
    cfg, keep = oracle.yolo_cfg(1, c["width"], c["height"], 1, c["mask"], c["anchors"], *c["net"])
    slots = len(c["mask"]) * c["width"] * c["height"]
    cls = np.zeros(slots, np.int32); anc = np.zeros(slots, np.int32); box = np.zeros(slots * 4, F)
    tr = f32(c["truths"])
    assert oracle.yolo_build_targets(cfg, tr, len(c["truths"]), cls, anc, box) == c["assigned"]
    cell = c["cell"]
    assert cls[cell] == c["class_at_cell"] and anc[cell] == c["anchor_at_cell"]
    assert cls[16 + cell] == -1 and anc[16 + cell] == -1
    assert np.allclose(box[4 * cell:4 * cell + 4], c["truths"][1][:4])
    c = kats["yolo_target_builder"]["other_head"]
    cfg, keep = oracle.yolo_cfg(1, c["width"], c["height"], 1, c["mask"], c["anchors"], *c["net"])
    slots = len(c["mask"]) * c["width"] * c["height"]
    cls = np.zeros(slots, np.int32); anc = np.zeros(slots, np.int32); box = np.zeros(slots * 4, F)
    assert oracle.yolo_build_targets(cfg, f32(c["truths"]), 1, cls, anc, box) == 0
    assert np.all(cls == -1)


def test_yolo_cpu_truth_thresh_kat(oracle, kats):
    c = kats["yolo_cpu_truth_thresh"]
    cfg, keep = oracle.yolo_cfg(1, 1, 1, c["classes"], c["mask"], c["anchors"], *c["net"],
                                ignore_thresh=c["ignore_thresh"], truth_thresh=c["truth_thresh"],
                                object_scale=c["object_scale"], noobject_scale=c["noobject_scale"])
    tr, cnt, mt = _truth_arrays([c["truths"]])
    out = np.zeros(6, F); delta = np.full(6, 9.0, F)
    oracle.yolo_forward(cfg, f32(c["input"]), tr, cnt, mt, out, delta)
    assert float_eq(delta[4], c["expected_delta4"])


def test_yolo_decode_kat(oracle, kats):
    c = kats["yolo_decode"]
    cfg, keep = oracle.yolo_cfg(1, 1, 1, 1, [0], [1, 1], 1, 1)
    x = f32(c["input"]); out = np.zeros(6, F)
    oracle.yolo_decode(cfg, x, out)
    sig = lambda v: 1 / (1 + math.exp(-v))
    want = [sig(0.2), sig(-0.4), 0.1, -0.2, sig(2.0), sig(1.5)]
    assert np.max(np.abs(out - want)) < c["tol"]
    assert out[2] == x[2] and out[3] == x[3]


def _run_kernel_kat(oracle, c, unassign=False):
    """The kernel-level vectors drive one 1x1 cell.  'unassigned' vectors (no positive
    slot) are reproduced on the CPU path by adding a second anchor that matches the
    truth exactly and is outside this head's mask."""
    anchors = list(c["anchors"]); truths = [list(t) for t in c["truths"]]
    if unassign:
        t = truths[0]
        anchors += [int(round(t[2] * c["net"][0])), int(round(t[3] * c["net"][1]))]
    cfg, keep = oracle.yolo_cfg(1, c["width"], c["height"], c["classes"], c["mask"], anchors, *c["net"],
                                ignore_thresh=c["ignore"], truth_thresh=c["truth"], coord_scale=c["coord"],
                                object_scale=c["object"], noobject_scale=c["noobject"], class_scale=c["class"])
    tr, cnt, mt = _truth_arrays([truths])
    n = 5 + c["classes"]
    out = np.zeros(n, F); delta = np.full(n, 7.0, F)
    cost, stats = oracle.yolo_forward(cfg, f32(c["raw"]), tr, cnt, mt, out, delta)
    return out, delta, cost, stats


def test_yolo_kernel_level_kats(oracle, kats):
    k = kats["yolo_kernel_kats"]
    c = k["assigned_target"]
    out, delta, cost, stats = _run_kernel_kat(oracle, c)
    s1, sm1 = 1 / (1 + math.exp(-1.0)), 1 / (1 + math.exp(1.0))
    assert all(float_eq(a, b) for a, b in zip(out[:5], c["expected_output_head"]))
    assert abs(out[5] - sm1) < 1e-6 and abs(out[6] - s1) < 1e-6
    assert all(float_eq(a, b) for a, b in zip(delta[:5], c["expected_delta_head"]))
    assert abs(delta[5] + 3 * sm1) < 1e-6 and abs(delta[6] - 3 * (1 - s1)) < 1e-6
    assert abs(cost - float(np.sum(delta.astype(np.float64) ** 2))) < 1e-5
    for key, want in c["expected_stats"].items():
        assert abs(stats[int(key)] - want) < 1e-6, key
    assert abs(stats[3] - s1) < 1e-6

    c = k["sparse_background"]
    out, delta, cost, stats = _run_kernel_kat(oracle, c)
    assert all(float_eq(a, b) for a, b in zip(delta, c["expected_delta"]))

    c = k["truth_thresh_override"]
    out, delta, cost, stats = _run_kernel_kat(oracle, c, unassign=True)
    assert stats[6] == 0 and float_eq(delta[4], c["expected_delta4"])

    c = k["ignore_only_iou"]
    out, delta, cost, stats = _run_kernel_kat(oracle, c, unassign=True)
    assert stats[6] == 0 and out[5] < c["output5_below"] and float_eq(delta[4], c["expected_delta4"])

    c = k["class_scale"]
    out, delta, cost, stats = _run_kernel_kat(oracle, c)
    assert all(float_eq(a, b) for a, b in zip(delta[5:8], c["expected_delta_classes"]))


def test_yolo_training_2x2_consistency(oracle, kats):
    """The reference only checks CPU against CUDA on this vector; here the restated CPU
    path is checked for the structure the two must share."""
    c = kats["yolo_training_2x2"]
    cfg, keep = oracle.yolo_cfg(c["batch"], c["width"], c["height"], c["classes"], c["mask"], c["anchors"],
                                *c["net"], ignore_thresh=c["ignore_thresh"], truth_thresh=c["truth_thresh"],
                                coord_scale=c["coord_scale"], object_scale=c["object_scale"],
                                noobject_scale=c["noobject_scale"], class_scale=c["class_scale"])
    x = f32([((i % 13) - 6) * np.float32(0.11) for i in range(56)])
    tr, cnt, mt = _truth_arrays([c["truths"]])
    out = np.zeros(56, F); delta = np.zeros(56, F)
    cost, stats = oracle.yolo_forward(cfg, x, tr, cnt, mt, out, delta)
    assert abs(cost - float(np.sum(delta.astype(np.float64) ** 2))) < c["tol_cost"]
    assert abs(stats[8] + stats[9] + stats[10] + stats[11] - cost) < 1e-4
    assert 1 <= stats[6] <= 3
    o = out.reshape(2, 7, 4); xi = x.reshape(2, 7, 4)
    assert np.array_equal(o[:, 2:4], xi[:, 2:4])
    assert np.allclose(o[:, [0, 1, 4, 5, 6]], 1 / (1 + np.exp(-xi[:, [0, 1, 4, 5, 6]].astype(np.float64))), atol=1e-6)


# ---------------------------------------------------------------- Adam
def test_adam_t1_closed_form(oracle):
    """From zero moments at t=1: m-hat = g, v-hat = g*g, so the step is lr*g/(|g|+eps)."""
    rng = np.random.default_rng(51)
    n = 4096
    w0 = (0.02 * rng.standard_normal(n)).astype(F)
    g0 = (1e-3 * rng.standard_normal(n)).astype(F)
    w, d, m, v = w0.copy(), g0.copy(), np.zeros(n, F), np.zeros(n, F)
    oracle.adam_update(w, d, m, v, 1, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, False)
    g = g0.astype(np.float64)
    want = w0 + 1e-3 * g / (np.abs(g) + 1e-8)
    assert np.max(np.abs(w - want) / np.maximum(np.abs(want), 1e-3)) < 1e-5
    assert np.all(d == 0)
    assert np.allclose(m, 0.1 * g, rtol=1e-6) and np.allclose(v, 0.001 * g * g, rtol=1e-5)


def test_adam_10_steps_vs_fp64_l2(oracle):
    """L2 decay folded into the update before the moments (not decoupled), step ADDED."""
    rng = np.random.default_rng(52)
    n = 2048
    lr, b1, b2, eps, decay, batch = 1e-3, 0.9, 0.999, 1e-8, 5e-4, 16
    w = (0.02 * rng.standard_normal(n)).astype(F)
    m = np.zeros(n, F); v = np.zeros(n, F)
    w64 = w.astype(np.float64); m64 = np.zeros(n); v64 = np.zeros(n)
    for t in range(1, 11):
        g = (1e-3 * rng.standard_normal(n)).astype(F)
        d = g.copy()
        oracle.adam_update(w, d, m, v, batch, t, lr, b1, b2, eps, decay, True)
        g64 = g.astype(np.float64) / batch - decay * w64
        m64 = b1 * m64 + (1 - b1) * g64
        v64 = b2 * v64 + (1 - b2) * g64 * g64
        w64 = w64 + lr * (m64 / (1 - b1 ** t)) / (np.sqrt(v64 / (1 - b2 ** t)) + eps)
    assert np.max(np.abs(w - w64) / np.maximum(np.abs(w64), 1e-2)) < 1e-5
    # a decoupled-decay (AdamW) recurrence is measurably different: the restatement is not that
    assert np.max(np.abs(w - w64)) < 1e-6


def test_adam_decoupled_decay_closed_form_and_fp64_recurrence(oracle):
    """apply_decay = 2 (no counterpart in the reference): from zero moments at t = 1 the weight is
    w0 + lr*g/(|g|+eps) - lr*decay*w0; ten steps against the AdamW recurrence carried in fp64, which the
    L2 form (apply_decay = 1) measurably is not."""
    rng = np.random.default_rng(53)
    n = 2048
    lr, b1, b2, eps, decay, batch = 1e-3, 0.9, 0.999, 1e-8, 5e-4, 16
    w0 = (0.02 * rng.standard_normal(n)).astype(F)
    g0 = (1e-3 * rng.standard_normal(n)).astype(F)
    w, d, m, v = w0.copy(), g0.copy(), np.zeros(n, F), np.zeros(n, F)
    oracle.adam_update(w, d, m, v, 1, 1, lr, b1, b2, eps, 0.5, 2)          # a decay large enough to see
    g = g0.astype(np.float64)
    want = w0 + lr * g / (np.abs(g) + eps) - lr * 0.5 * w0.astype(np.float64)
    assert np.max(np.abs(w - want) / np.maximum(np.abs(want), 1e-3)) < 1e-5
    assert np.allclose(m, 0.1 * g, rtol=1e-6) and np.all(d == 0)           # the moments do not see the decay
    w = w0.copy(); m = np.zeros(n, F); v = np.zeros(n, F)
    l2 = w0.copy(); m2 = np.zeros(n, F); v2 = np.zeros(n, F)
    w64 = w.astype(np.float64); m64 = np.zeros(n); v64 = np.zeros(n)
    for t in range(1, 11):
        g = (1e-3 * rng.standard_normal(n)).astype(F)
        oracle.adam_update(w, g.copy(), m, v, batch, t, lr, b1, b2, eps, decay, 2)
        oracle.adam_update(l2, g.copy(), m2, v2, batch, t, lr, b1, b2, eps, decay, 1)
        g64 = g.astype(np.float64) / batch
        m64 = b1 * m64 + (1 - b1) * g64
        v64 = b2 * v64 + (1 - b2) * g64 * g64
        w64 = w64 + lr * (m64 / (1 - b1 ** t)) / (np.sqrt(v64 / (1 - b2 ** t)) + eps) - lr * decay * w64
    assert np.max(np.abs(w - w64) / np.maximum(np.abs(w64), 1e-2)) < 1e-6
    assert np.max(np.abs(l2 - w64) / np.maximum(np.abs(w64), 1e-2)) > 1e-3


def test_sgd_closed_form_and_fp64_recurrence(oracle):
    """The reference holds no numeric test of ConvLayer::update: one step against its closed form,
    ten steps against the same recurrence carried in fp64."""
    rng = np.random.default_rng(11)
    n = 4096
    w0 = rng.normal(0, 0.02, n).astype(F); g = rng.normal(0, 0.5, (10, n)).astype(F)
    lr, mom, decay, batch = 1e-3, 0.9, 5e-4, 16
    w = w0.copy(); d = g[0].copy()
    oracle.sgd_update(w, d, batch, lr, mom, decay, True)
    d_eff = g[0].astype(np.float64) - decay * batch * w0.astype(np.float64)
    assert np.allclose(w, w0 + lr / batch * d_eff, rtol=1e-6, atol=1e-9)
    assert np.allclose(d, mom * d_eff, rtol=1e-6, atol=1e-9)
    # without decay the weights do not enter the update
    w2 = w0.copy(); d2 = g[0].copy()
    oracle.sgd_update(w2, d2, batch, lr, mom, decay, False)
    assert np.allclose(w2, w0 + lr / batch * g[0].astype(np.float64), rtol=1e-6, atol=1e-9)
    assert np.allclose(d2, mom * g[0].astype(np.float64), rtol=1e-6, atol=1e-9)
    # ten steps
    w = w0.copy(); d = np.zeros(n, F)
    w64 = w0.astype(np.float64); d64 = np.zeros(n)
    for t in range(10):
        d += g[t]; d64 += g[t]
        oracle.sgd_update(w, d, batch, lr, mom, decay, True)
        d64 = d64 - decay * batch * w64
        w64 = w64 + lr / batch * d64
        d64 = mom * d64
    assert np.allclose(w, w64, rtol=1e-5, atol=1e-8)
    assert np.allclose(d, d64, rtol=1e-5, atol=2e-6)      # sums of O(1) terms rounded to fp32 ten times


def test_rescale_clip_invariants(oracle):
    rng = np.random.default_rng(12)
    x0 = rng.normal(0, 1.0, 10000).astype(F)
    norm = np.sqrt(np.square(x0.astype(np.float64)).sum())
    # above the threshold: the result has the threshold as its norm and the direction of x
    x = x0.copy()
    got = oracle.rescale_clip(x, 0.5 * norm, 0.0)
    assert abs(got - norm) <= 1e-6 * norm
    assert abs(np.sqrt(np.square(x.astype(np.float64)).sum()) - 0.5 * norm) <= 1e-6 * norm
    assert np.allclose(x, 0.5 * x0, rtol=1e-6)
    # below the threshold, or no threshold: untouched
    for thr in (2.0 * norm, 0.0):
        x = x0.copy()
        oracle.rescale_clip(x, thr, 0.0)
        assert np.array_equal(x, x0)
    # clip only: clamp
    x = x0.copy()
    oracle.rescale_clip(x, 0.0, 0.7)
    assert np.array_equal(x, np.clip(x0, -0.7, 0.7))
    # both: rescale first, then clamp (the order of Layer::backward)
    x = x0.copy()
    oracle.rescale_clip(x, 0.5 * norm, 0.3)
    assert np.allclose(x, np.clip(0.5 * x0, -0.3, 0.3), rtol=1e-6)
    # zero tensor: the norm test keeps it untouched
    z = np.zeros(8, F)
    assert oracle.rescale_clip(z, 1.0, 0.0) == 0.0 and not z.any()


def test_detections_hand_computed(oracle):
    """addDetects on a 2x2 head with one anchor and two classes, values worked out by hand."""
    W = H = 2; K = 2
    cfg, keep = oracle.yolo_cfg(1, W, H, K, [0], [16, 16], 64, 64)
    p = np.zeros((1, K + 5, H, W), F)
    # cell (row 0, col 1): centre offsets 0.5, log-sizes 0, objectness 0.9, class probabilities 0.8 / 0.5
    p[0, 0, 0, 1] = 0.5; p[0, 1, 0, 1] = 0.5; p[0, 4, 0, 1] = 0.9; p[0, 5, 0, 1] = 0.8; p[0, 6, 0, 1] = 0.5
    # cell (row 1, col 0): objectness below the threshold; cell (1, 1): objectness passes, no class does
    p[0, 4, 1, 0] = 0.49; p[0, 5, 1, 0] = 1.0
    p[0, 4, 1, 1] = 0.6; p[0, 5, 1, 1] = 0.8
    rec, found = oracle.yolo_detections(cfg, p, 0.5, 16)
    assert found == 1 and len(rec) == 1
    r = rec[0]
    # x = (1 + .5)/2 = .75, y = (0 + .5)/2 = .25, w = h = exp(0)*16/64 = .25 -> left .625, top .125
    assert (r["x"], r["y"], r["w"], r["h"]) == (0.625, 0.125, 0.25, 0.25)
    assert r["class_index"] == 0 and r["batch"] == 0 and abs(r["prob"] - 0.72) < 1e-7
    assert r["order"] == (0 * 4 + 1) * 1 * K + 0
    # a 128 x 64 image letterboxed into 64 x 64: newW 64, newH 32; x stays .75, y -> (.25 - .25)/.5 = 0,
    # w .25, h .25 * 2 = .5 -> left int(.625*128) = 80, right int(.875*128) = 112, top max(0, int(-.25*64)) = 0,
    # bottom int(.25*64) = 16
    rec, found = oracle.yolo_detections(cfg, p, 0.5, 16, image_width=128, image_height=64)
    assert found == 1
    r = rec[0]
    assert (r["x"], r["y"], r["w"], r["h"]) == (80.0, 0.0, 32.0, 16.0)
    # a lower threshold lets the other class and the other cells in, in cell / mask / class order
    rec, found = oracle.yolo_detections(cfg, p, 0.4, 16)
    assert found == 4
    assert list(rec["order"]) == [2, 3, 4, 6] and list(rec["class_index"]) == [0, 1, 0, 0]
    # capacity smaller than the number found: the count still says how many there are
    rec, found = oracle.yolo_detections(cfg, p, 0.4, 2)
    assert found == 4 and len(rec) == 2


def test_nms_kats(oracle, kats):
    """tests/src/box.cpp:25-101."""
    for case in kats["nms"]["cases"]:
        out = oracle.nms(detection_records(oracle, case["detections"]), case["threshold"])
        if "expected_boxes" in case:
            got = [[float(r["x"]), float(r["y"]), float(r["w"]), float(r["h"])] for r in out]
            assert got == [[float(v) for v in b] for b in case["expected_boxes"]], case["name"]
        if "expected_count" in case:
            assert len(out) == case["expected_count"], case["name"]
        if "expected_classes" in case:
            assert list(out["class_index"]) == case["expected_classes"], case["name"]
        if "expected_probs" in case:
            assert np.allclose(out["prob"], case["expected_probs"], rtol=1e-7), case["name"]


def test_nms_hand_worked_scenarios(oracle):
    """Cases whose answer follows from src/Box.cpp:56-147 by hand."""
    X = [0, 0, 100, 100]
    Y = [0, 0, 100, 70]          # overlap ratio with X: 0.7
    # a box discarded as a cross-class duplicate never suppresses a weaker box of its own class
    out = oracle.nms(detection_records(oracle, [X + [0, 1, 0.9], X + [0, 2, 0.8], Y + [0, 2, 0.7]]), 0.5)
    assert [(int(r["class_index"]), float(r["h"])) for r in out] == [(1, 100.0), (2, 70.0)]
    # ... and does not discard a near-identical box of a third class either (it is skipped, 76-79)
    A = [0, 0, 100, 100]; A1 = [0, 0, 100, 95]; A2 = [0, 0, 100, 89]      # A/A1 .95, A1/A2 .937, A/A2 .89
    out = oracle.nms(detection_records(oracle, [A + [0, 1, 0.9], A1 + [0, 2, 0.8], A2 + [0, 3, 0.7]]), 0.5)
    assert list(out["class_index"]) == [1, 3]
    # equal probabilities keep their input order (stable sort): the first of two twins survives
    out = oracle.nms(detection_records(oracle, [X + [0, 1, 0.5], X + [0, 1, 0.5]]), 0.5)
    assert len(out) == 1 and out[0]["order"] == 0
    # the output is sorted by probability whatever the input order, across images
    out = oracle.nms(detection_records(oracle, [X + [1, 1, 0.2], X + [0, 1, 0.9], X + [2, 1, 0.5]]), 0.5)
    assert list(out["batch"]) == [0, 2, 1]
    # negative extents are normalised (47-54): (100,100,-100,-100) is X
    out = oracle.nms(detection_records(oracle, [X + [0, 1, 0.9], [100, 100, -100, -100, 0, 1, 0.8]]), 0.5)
    assert len(out) == 1
    # empty boxes have no overlap ratio (0/0 counts as none): both stay
    Z = [5, 5, 0, 0]
    out = oracle.nms(detection_records(oracle, [Z + [0, 1, 0.9], Z + [0, 1, 0.8]]), 0.0)
    assert len(out) == 2
    # exactly at the threshold is not above it
    out = oracle.nms(detection_records(oracle, [[0, 0, 100, 100, 0, 1, 0.9], [0, 0, 100, 50, 0, 1, 0.8]]), 0.5)
    assert len(out) == 2
    # only the first 1024 members of a group are visited; the rest stay whatever they overlap
    rows = [X + [0, 1, 1.0 - i * 1e-4] for i in range(1100)]
    out = oracle.nms(detection_records(oracle, rows), 0.5)
    assert len(out) == 1 + (1100 - 1024)
    assert list(out["order"]) == [0] + list(range(1024, 1100))
    # members that the duplicate pass discarded still use up places among the 1024
    rows = [X + [0, 2, 1.0]] + [X + [0, 1, 0.9 - i * 1e-4] for i in range(1100)]
    out = oracle.nms(detection_records(oracle, rows), 0.5)        # all of class 1 are duplicates of the class-2 box
    assert len(out) == 1 and out[0]["class_index"] == 2
    assert len(oracle.nms(detection_records(oracle, []), 0.5)) == 0


def nms_by_the_book(rec, threshold):
    """src/Box.cpp:56-147 restated with Python containers and numpy float32 arithmetic, written
    independently of the C checker (dictionary groups, lists of kept boxes)."""
    f = np.float32

    def norm(r):
        x, y, w, h = f(r["x"]), f(r["y"]), f(r["w"]), f(r["h"])
        x1, y1 = min(x, f(x + w)), min(y, f(y + h))
        x2, y2 = max(x, f(x + w)), max(y, f(y + h))
        return x1, y1, max(f(0), f(x2 - x1)), max(f(0), f(y2 - y1))

    def iou(a, b):
        if a[2] <= 0 or a[3] <= 0 or b[2] <= 0 or b[3] <= 0:
            inter = f(0)
        else:
            xl, xh = (a, b) if a[0] < b[0] else (b, a)
            yl, yh = (a, b) if a[1] < b[1] else (b, a)
            if (xl[0] < 0 and f(xl[0] + xl[2]) < xh[0]) or (yl[1] < 0 and f(yl[1] + yl[3]) < yh[1]):
                inter = f(0)
            else:
                iw = min(f(xl[2] - f(xh[0] - xl[0])), xh[2])
                ih = min(f(yl[3] - f(yh[1] - yl[1])), yh[3])
                inter = f(iw * ih) if iw > 0 and ih > 0 else f(0)
        uni = max(f(0), f(f(f(a[2] * a[3]) + f(b[2] * b[3])) - inter))
        with np.errstate(divide="ignore", invalid="ignore"):
            q = inter / uni
        return f(0) if not np.isfinite(q) else q

    order = sorted(range(len(rec)), key=lambda i: -float(rec[i]["prob"]))      # sorted() is stable
    boxes = [norm(rec[i]) for i in order]
    discard = [False] * len(order)
    for i in range(len(order)):
        for j in range(i):
            a, b = rec[order[i]], rec[order[j]]
            if discard[j] or a["batch"] != b["batch"] or a["class_index"] == b["class_index"]:
                continue
            if iou(boxes[i], boxes[j]) > f(0.9):
                discard[i] = True
                break
    groups = {}
    for i in range(len(order)):
        groups.setdefault((int(rec[order[i]]["batch"]), int(rec[order[i]]["class_index"])), []).append(i)
    for members in groups.values():
        kept = []
        for i in members[:1024]:
            if discard[i]:
                continue
            if any(iou(boxes[i], boxes[j]) > f(threshold) for j in kept):
                discard[i] = True
            else:
                kept.append(i)
    return rec[[order[i] for i in range(len(order)) if not discard[i]]]


@pytest.mark.parametrize("seed,n,batch,classes,clusters,thr", [(1, 300, 2, 3, 3, 0.45), (2, 500, 1, 2, 2, 0.3),
                                                               (3, 400, 3, 5, 1, 0.6), (4, 64, 1, 1, 1, 0.0)])
def test_nms_matches_the_book_on_random_clusters(oracle, seed, n, batch, classes, clusters, thr):
    rec = random_detections(oracle, seed, n, batch, classes, clusters, spread=3.0 if seed == 3 else 6.0)
    want = nms_by_the_book(rec, thr)
    got = oracle.nms(rec, thr)
    assert len(got) == len(want) and 0 < len(got) < n
    assert list(got["order"]) == list(want["order"])
    assert got.tobytes() == want.tobytes()
