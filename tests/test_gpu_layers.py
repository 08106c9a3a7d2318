"""GPU parity: max-pool, upsample and shortcut, forward and backward, bit-exact against the CPU
checker (values, int32 indices and accumulation order), through the C ABI."""
import numpy as np
import pytest

from pixienn_amd import workloads as wl
from util import F, assert_bit_exact, gpu, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from pixienn_amd import ops as o
    return o


def run_maxpool(ops, oracle, x, kernel, stride, padding, seed):
    import torch
    N, C, H, W = x.shape
    oh = oracle.maxpool_out_dim(H, kernel, stride, padding)
    ow = oracle.maxpool_out_dim(W, kernel, stride, padding)
    assert oh == ops.maxpool_out_dim(H, kernel, stride, padding)
    out_w = np.zeros((N, C, oh, ow), F); idx_w = np.zeros((N, C, oh, ow), np.int32)
    oracle.maxpool_forward(x, out_w, idx_w, N, C, H, W, oh, ow, kernel, stride, padding)
    # poisoned outputs: the kernel must write every element itself
    gout = torch.full((N, C, oh, ow), 123.0, device="cuda")
    gidx = torch.full((N, C, oh, ow), -77, device="cuda", dtype=torch.int32)
    ops.maxpool_forward(gpu(x), gout, gidx, kernel, stride, padding)
    what = "maxpool %s k%d s%d p%d" % (x.shape, kernel, stride, padding)
    assert_bit_exact(host(gout), out_w, what + " values")
    assert_bit_exact(host(gidx), idx_w, what + " indexes")
    delta = wl.normal(seed, out_w.shape)
    grad0 = wl.normal(seed + 1, x.shape)
    grad_w = grad0.copy()
    oracle.maxpool_backward(delta, idx_w, grad_w)
    ggrad = gpu(grad0)
    ops.maxpool_backward(gpu(delta), gidx, ggrad, kernel, stride, padding)
    assert_bit_exact(host(ggrad), grad_w, what + " backward")
    return idx_w, delta, grad0, grad_w


def test_maxpool_reference_kat(ops, kats):
    import torch
    c = kats["maxpool"]
    x = gpu(np.array(c["input"], F).reshape(1, 1, 3, 3))
    out = torch.zeros(1, 1, 3, 3, device="cuda"); idx = torch.full((1, 1, 3, 3), -1, device="cuda", dtype=torch.int32)
    ops.maxpool_forward(x, out, idx, c["kernel"], c["stride"], c["padding"])
    assert host(out).ravel().tolist() == c["expected_out"]
    grad = torch.full((1, 1, 3, 3), c["grad_fill"], device="cuda")
    ops.maxpool_backward(torch.full((1, 1, 3, 3), c["delta_fill"], device="cuda"), idx, grad, c["kernel"], c["stride"],
                         c["padding"])
    assert host(grad).ravel().tolist() == c["expected_grad"]


@pytest.mark.parametrize("shape", [(2, 3, 304, 304), (2, 4, 76, 76), (2, 5, 38, 38), (3, 4, 26, 26),
                                   (1, 2, 416, 416), (2, 3, 6, 10), (2, 2, 20, 12), (1, 1, 6, 4), (1, 3, 2, 12)])
def test_maxpool_2x2_stride2(ops, oracle, shape):
    x = wl.normal(1000 + shape[2], shape)
    run_maxpool(ops, oracle, x, 2, 2, 1, 1100)
    run_maxpool(ops, oracle, x, 2, 2, 0, 1101)
    # heavy ties: the first maximum in window order must win
    xt = np.round(x).astype(F)
    run_maxpool(ops, oracle, xt, 2, 2, 1, 1102)


@pytest.mark.parametrize("geom", [(13, 13, 2, 1, 1), (13, 13, 3, 1, 2), (9, 11, 3, 2, 2), (7, 7, 2, 2, 1),
                                  (8, 8, 3, 3, 0), (5, 9, 2, 1, 0), (6, 6, 4, 2, 3), (4, 4, 1, 1, 0), (5, 5, 2, 3, 1)])
def test_maxpool_general_geometry(ops, oracle, geom):
    H, W, k, s, p = geom
    x = wl.normal(1200 + H * W + k, (2, 3, H, W))
    run_maxpool(ops, oracle, x, k, s, p, 1300)
    run_maxpool(ops, oracle, np.round(x).astype(F), k, s, p, 1301)


def test_maxpool_special_values(ops, oracle):
    x = wl.normal(1400, (1, 2, 8, 8))
    x[0, 0, 0, 0] = np.nan          # first tap NaN: sticky
    x[0, 0, 2, 3] = np.nan          # later tap NaN: never taken
    x[0, 1, 4:6, 4:6] = [[0.0, -0.0], [-0.0, 0.0]]
    x[0, 1, 0:2, 0:2] = -np.inf
    x[0, 1, 6:8, 6:8] = np.finfo(np.float32).min
    run_maxpool(ops, oracle, x, 2, 2, 1, 1401)
    run_maxpool(ops, oracle, x, 2, 1, 1, 1402)


def test_maxpool_scatter_signature(ops, oracle):
    x = wl.normal(1500, (2, 3, 12, 12))
    idx_w, delta, grad0, grad_w = run_maxpool(ops, oracle, x, 2, 2, 1, 1501)
    g = gpu(grad0)
    ops.maxpool_backward_scatter(gpu(delta), gpu(idx_w), g)
    assert_bit_exact(host(g), grad_w, "scatter (unique indexes)")


@pytest.mark.parametrize("shape,stride", [((2, 3, 19, 19), 2), ((2, 4, 38, 38), 2), ((2, 3, 13, 13), 2),
                                          ((1, 2, 8, 12), 2), ((2, 2, 5, 6), 2), ((2, 2, 5, 7), 3), ((1, 3, 4, 4), 1),
                                          ((2, 2, 6, 10), 4)])
def test_upsample_forward_backward(ops, oracle, shape, stride):
    import torch
    N, C, H, W = shape
    x = wl.normal(1600 + H, shape)
    for scale in (1.0, 0.75):
        out_w = np.zeros((N, C, H * stride, W * stride), F)
        oracle.upsample(x, W, H, C, N, stride, True, scale, None, out_w)
        gout = torch.full(out_w.shape, 55.0, device="cuda")     # no zero-fill needed
        ops.upsample_forward(gpu(x), gout, stride, scale)
        assert_bit_exact(host(gout), out_w, "upsample fwd %s s%d" % (shape, stride))
        delta = wl.normal(1700 + W, out_w.shape)
        grad0 = wl.normal(1701 + W, shape)
        grad_w = grad0.copy()
        oracle.upsample(None, W, H, C, N, stride, False, scale, grad_w, delta)
        gg = gpu(grad0)
        ops.upsample_backward(gpu(delta), gg, stride, scale)
        assert_bit_exact(host(gg), grad_w, "upsample bwd %s s%d scale %g" % (shape, stride, scale))


@pytest.mark.parametrize("shape,stride,other,offset", [((2, 8, 19, 19), 2, 16, 0), ((2, 8, 19, 19), 2, 16, 16),
                                                       ((3, 4, 8, 12), 2, 5, 5), ((2, 3, 5, 7), 2, 3, 0),
                                                       ((2, 3, 5, 7), 3, 2, 2), ((1, 2, 4, 4), 2, 1, 1)])
def test_upsample_into_concatenation_buffer(ops, oracle, shape, stride, other, offset):
    """The strided form writes (and, backward, reads) a channel slice of a wider tensor: the result
    equals the dense upsample followed by the route copy, and the other channels stay untouched."""
    import torch
    N, C, H, W = shape
    OH, OW = H * stride, W * stride
    x = wl.normal(1650 + H + offset, shape)
    dense = np.zeros((N, C, OH, OW), F)
    oracle.upsample(x, W, H, C, N, stride, True, 0.75, None, dense)
    buf0 = wl.normal(1651 + W, (N, C + other, OH, OW))
    expect = buf0.copy()
    expect[:, offset:offset + C] = dense
    gbuf = gpu(buf0)
    ops.upsample_forward_into(gpu(x), gbuf, offset, stride, 0.75)
    assert_bit_exact(host(gbuf), expect, "upsample into buffer %s +%d" % (shape, offset))
    delta_buf = wl.normal(1652 + W, (N, C + other, OH, OW))
    grad0 = wl.normal(1653 + W, shape)
    grad_w = grad0.copy()
    oracle.upsample(None, W, H, C, N, stride, False, 0.75, grad_w,
                    np.ascontiguousarray(delta_buf[:, offset:offset + C]))
    gg = gpu(grad0)
    gdelta = gpu(delta_buf)
    ops.upsample_backward_from(gdelta, offset, gg, stride, 0.75)
    assert_bit_exact(host(gg), grad_w, "upsample from buffer %s +%d" % (shape, offset))
    assert_bit_exact(host(gdelta), delta_buf, "delta buffer untouched")
    with pytest.raises(ValueError):
        ops.upsample_forward_into(gpu(x), gbuf, other + 1, stride, 0.75)


@pytest.mark.parametrize("act", ["linear", "leaky"])
@pytest.mark.parametrize("shape", [(2, 8, 38, 38), (3, 5, 19, 19), (1, 1, 1, 3), (4, 64, 76, 76)])
def test_shortcut_backward_as_first_writer(ops, oracle, shape, act):
    """The overwriting form gives what the CPU layer's accumulation into cleared tensors gives, and
    reads neither target: they start as NaN here."""
    import torch
    N, C, H, W = shape
    for alpha, beta in ((1.0, 1.0), (0.5, 1.25)):
        pre = wl.normal(1820 + W, shape)
        d0 = wl.normal(1821 + W, shape)
        d0[0, 0, 0, 0] = 0.0                                  # a zero delta: -0 * beta stays a zero of either sign
        d_w, fd_w, g_w = d0.copy(), np.zeros(shape, F), np.zeros(shape, F)
        oracle.shortcut_backward(act, N, W, H, C, d_w, pre, fd_w, g_w, alpha, beta)
        gd = gpu(d0)
        gfd = torch.full(shape, float("nan"), device="cuda"); gg = torch.full(shape, float("nan"), device="cuda")
        ops.shortcut_backward_first(gd, gfd, gg, act, alpha, beta, pre_activation=gpu(pre))
        what = "first-writer shortcut %s %s a=%g b=%g" % (shape, act, alpha, beta)
        assert_bit_exact(host(gd), d_w, what + " delta")
        for got, want, name in ((host(gfd), fd_w, "from delta"), (host(gg), g_w, "grad")):
            assert np.array_equal(got, want), what + " " + name                       # equal as numbers
            nonzero = want != 0
            assert_bit_exact(got[nonzero], want[nonzero], what + " " + name)         # and bit for bit off zero
        # without a grad target only from_delta is written
        gfd2 = torch.full(shape, float("nan"), device="cuda")
        ops.shortcut_backward_first(gpu(d0), gfd2, None, act, alpha, beta, pre_activation=gpu(pre))
        assert np.array_equal(host(gfd2), fd_w), what + " from delta alone"
    with pytest.raises(ops.capi.PxError):
        ops.shortcut_backward_first(gd, gfd, gfd, act, 1.0, 1.0, pre_activation=gpu(pre))


@pytest.mark.parametrize("act", ["linear", "leaky"])
@pytest.mark.parametrize("shape", [(2, 8, 38, 38), (3, 5, 19, 19), (1, 1, 1, 3), (2, 3, 64, 64)])
def test_shortcut_forward_backward(ops, oracle, shape, act):
    import torch
    N, C, H, W = shape
    a = wl.normal(1800 + W, shape); b = wl.normal(1801 + W, shape)
    for alpha, beta in ((1.0, 1.0), (0.5, 1.25)):
        out_w = np.empty_like(a); pre_w = np.empty_like(a)
        oracle.shortcut_forward(act, N, W, H, C, a, b, alpha, beta, out_w, pre_w)
        gout = torch.full(shape, 9.0, device="cuda"); gpre = torch.full(shape, 9.0, device="cuda")
        ops.shortcut_forward(gpu(a), gpu(b), gout, act, alpha, beta, pre_activation=gpre)
        what = "shortcut %s %s a=%g b=%g" % (shape, act, alpha, beta)
        assert_bit_exact(host(gout), out_w, what + " out")
        assert_bit_exact(host(gpre), pre_w, what + " pre")
        d0 = wl.normal(1810 + W, shape); fd0 = wl.normal(1811 + W, shape); g0 = wl.normal(1812 + W, shape)
        d_w, fd_w, g_w = d0.copy(), fd0.copy(), g0.copy()
        oracle.shortcut_backward(act, N, W, H, C, d_w, pre_w, fd_w, g_w, alpha, beta)
        gd, gfd, gg = gpu(d0), gpu(fd0), gpu(g0)
        ops.shortcut_backward(gd, gfd, gg, act, alpha, beta, pre_activation=gpre)
        assert_bit_exact(host(gd), d_w, what + " delta")
        assert_bit_exact(host(gfd), fd_w, what + " from delta")
        assert_bit_exact(host(gg), g_w, what + " grad")
        # first layer: grad == NULL
        gd, gfd = gpu(d0), gpu(fd0)
        ops.shortcut_backward(gd, gfd, None, act, alpha, beta, pre_activation=gpre)
        assert_bit_exact(host(gfd), fd_w, what + " from delta (no grad)")


def test_shortcut_reference_signature(ops, oracle):
    """shortcutGpu's index-mapped blend, same shape and the shapes the CPU layer accepts."""
    N, C, H, W = 2, 3, 6, 6
    add = wl.normal(1900, (N, C, H, W)); out0 = wl.normal(1901, (N, C, H, W))
    want = out0.copy()
    assert oracle.shortcut(N, W, H, C, add, W, H, C, 0.5, 2.0, want) == 0
    g = gpu(out0)
    ops.shortcut(N, W, H, C, gpu(add), W, H, C, 0.5, 2.0, g)
    assert_bit_exact(host(g), want, "shortcut same shape")
    # fewer channels on one side (min over channels), identity spatial maps
    add2 = wl.normal(1902, (N, 2, H, W))
    want = out0.copy()
    assert oracle.shortcut(N, W, H, 2, add2, W, H, C, 1.0, 1.0, want) == 0
    g = gpu(out0)
    ops.shortcut(N, W, H, 2, gpu(add2), W, H, C, 1.0, 1.0, g)
    assert_bit_exact(host(g), want, "shortcut channel mismatch")


# route: YOLOv3-tiny concatenates 128x26^2 (upsampled) with 256x26^2; odd sizes take the scalar path
@pytest.mark.parametrize("layers", [[(128, 26), (256, 26)], [(3, 5), (2, 5), (7, 5)], [(256, 38), (512, 38)], [(1, 1)]])
def test_route_forward_backward(ops, oracle, layers):
    import torch
    N = 3
    outs = [wl.normal(8100 + i, (N, c, s, s)) for i, (c, s) in enumerate(layers)]
    per_image = [o[0].size for o in outs]
    total = sum(per_image)
    want = np.full((N, total), -5.0, F)
    got = torch.full((N, total), -5.0, device="cuda")
    offset = 0
    for o, size in zip(outs, per_image):
        oracle.route_forward(o, want, offset)
        ops.route_forward(gpu(o), got, offset)
        offset += size
    assert_bit_exact(host(got), want, "route forward %s" % (layers,))
    assert not (want == -5.0).any()
    route_delta = wl.normal(8200, (N, total))
    offset = 0
    for i, (o, size) in enumerate(zip(outs, per_image)):
        d0 = wl.normal(8300 + i, o.shape)
        d_w = d0.copy()
        oracle.route_backward(route_delta, d_w, offset)
        d_g = gpu(d0)
        ops.route_backward(gpu(route_delta), d_g, offset)
        assert_bit_exact(host(d_g), d_w, "route backward %s layer %d" % (layers, i))
        offset += size


def test_route_rejects_slice_outside_route(ops):
    import torch
    from pixienn_amd import capi
    a = torch.zeros(2, 8, device="cuda")
    r = torch.zeros(2, 12, device="cuda")
    with pytest.raises(capi.PxError):
        ops.route_forward(a, r, 8)
