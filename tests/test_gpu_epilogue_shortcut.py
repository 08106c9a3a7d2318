"""GPU parity: a convolution's epilogue with the linear ShortcutLayer that follows it taken into the same
pass (pxh_bn_train_act_shortcut_forward, pxh_bn_folded_act_shortcut_forward) against the two layers one
after the other -- include/cuda/ConvLayer.h:284-307 then include/cuda/ShortcutLayer.h:23-37 of the
reference: against the CPU checker's two calls at the tolerance of the epilogue alone, and TO THE BIT
against this library's own two calls (the same operations in the same order; only the tensor in between
is gone), for every form of the forward: flat 128-bit, scalar, one launch per layer (small, large and at
more than 512 channels), three launches.
"""
import numpy as np
import pytest

from pixienn_amd import workloads as wl
from test_gpu_epilogue import SHAPES, TRAIN_SHAPES, WIDE_ABOVE, bn_case
from util import F, assert_bit_exact, assert_close, gpu, host

pytestmark = pytest.mark.gpu

FACTORS = [(1.0, 1.0), (0.75, -1.5)]


@pytest.fixture(scope="module")
def ops():
    from pixienn_amd import ops as o
    return o


@pytest.mark.parametrize("act", ["leaky", "mish", "linear", "logistic"])
def test_training_epilogue_with_shortcut_is_the_two_calls_to_the_bit(ops, act):
    # (+ a 128-bit slice of 7000 vectors: the half-size workgroups with sixteen vectors per lane)
    for si, (N, C, HW) in enumerate(TRAIN_SHAPES + [(4, 96, 7000)]):
        x, scale, bias, rmean, rvar = bn_case(3000 + si, N, C, HW, spread=1.5)
        frm = wl.normal(3050 + si, x.shape)
        alpha, beta = FACTORS[si % 2]
        gx, gfrom, gscale, gbias = gpu(x), gpu(frm), gpu(scale), gpu(bias)
        # the two layers one after the other
        y0, pre0, xs0, xn0, out0 = (gpu(np.zeros_like(x)) for _ in range(5))
        m0, v0, rm0, rv0 = gpu(np.zeros(C, F)), gpu(np.zeros(C, F)), gpu(rmean), gpu(rvar)
        ops.bn_train_act_forward(gx, y0, m0, v0, rm0, rv0, gscale, gbias, act, pre_activation=pre0, x_saved=xs0,
                                 x_norm=xn0)
        ops.shortcut_forward(y0, gfrom, out0, "linear", alpha, beta)
        # ... and as one call
        y1, pre1, xs1, xn1 = (gpu(np.full_like(x, 7.0)) for _ in range(4))
        m1, v1, rm1, rv1 = gpu(np.zeros(C, F)), gpu(np.zeros(C, F)), gpu(rmean), gpu(rvar)
        ops.bn_train_act_shortcut_forward(gx, y1, m1, v1, rm1, rv1, gscale, gbias, act, gfrom, alpha, beta,
                                          pre_activation=pre1, x_saved=xs1, x_norm=xn1)
        what = "%s %s alpha %g beta %g" % (act, (N, C, HW), alpha, beta)
        # Scalar slices of 512 channels and more: alone, the layer runs with workgroups of half the size, which
        # add up a channel's statistics in another order than the full workgroups the fused call keeps; there
        # the two agree to rounding of the sums (1e-6 of the statistics), everywhere else to the bit.
        same_order = not (HW % 4 != 0 and C >= 512)
        if same_order:
            same = assert_bit_exact
        else:
            sigma = np.sqrt(host(v0).astype(np.float64))
            fl = ((np.abs(host(m0)) + sigma) / sigma).reshape(1, C, 1, 1) * 4.0 + np.abs(frm)

            def same(got, want, what):
                assert_close(got, want, 2e-6, fl if got.ndim == 4 else 1.0, what)
        same(host(y1), host(out0), what + " output")
        for name, a, b in (("pre-activation", pre1, pre0), ("x_norm", xn1, xn0), ("mean", m1, m0),
                           ("var", v1, v0), ("rolling mean", rm1, rm0), ("rolling var", rv1, rv0)):
            same(host(a), host(b), what + " " + name)
        assert_bit_exact(host(xs1), host(xs0), what + " x_saved")
        # no extra outputs, the shortcut's source in the output tensor itself (the layer writes in place of `from`)
        y2 = gpu(frm)
        m2, v2, rm2, rv2 = gpu(np.zeros(C, F)), gpu(np.zeros(C, F)), gpu(rmean), gpu(rvar)
        ops.bn_train_act_shortcut_forward(gx, y2, m2, v2, rm2, rv2, gscale, gbias, act, y2, alpha, beta)
        same(host(y2), host(out0), what + " output, from == y")


@pytest.mark.parametrize("act", ["leaky", "mish", "linear", "swish", "relu"])
def test_inference_epilogue_with_shortcut_is_the_two_calls_to_the_bit(ops, act):
    import torch
    for si, (N, C, HW) in enumerate(SHAPES + [(2, 130, 1444)]):
        x, scale, bias, rmean, rvar = bn_case(3100 + si, N, C, HW)
        frm = wl.normal(3150 + si, x.shape)
        alpha, beta = FACTORS[(si + 1) % 2]
        folded = ops.bn_fold(gpu(rmean), gpu(rvar), gpu(scale), gpu(bias))
        gx, gfrom = gpu(x), gpu(frm)
        y0, pre0, out0 = (gpu(np.zeros_like(x)) for _ in range(3))
        ops.bn_folded_act_forward(gx, y0, folded, act, pre_activation=pre0)
        ops.shortcut_forward(y0, gfrom, out0, "linear", alpha, beta)
        y1, pre1 = gpu(np.full_like(x, 7.0)), gpu(np.full_like(x, 7.0))
        ops.bn_folded_act_shortcut_forward(gx, y1, folded, act, gfrom, alpha, beta, pre_activation=pre1)
        what = "%s %s" % (act, (N, C, HW))
        assert_bit_exact(host(y1), host(out0), what + " output")
        assert_bit_exact(host(pre1), host(pre0), what + " pre-activation")
        if N * C * HW > 8:
            # tensors that do not start on a 16-byte boundary: one element per lane
            n = N * C * HW
            bx, bf, by = (torch.zeros(n + 1, device="cuda") for _ in range(3))
            bx[1:] = gx.reshape(-1); bf[1:] = gfrom.reshape(-1)
            ops.bn_folded_act_shortcut_forward(bx[1:].view(N, C, HW, 1), by[1:].view(N, C, HW, 1), folded, act,
                                               bf[1:].view(N, C, HW, 1), alpha, beta)
            assert_bit_exact(host(by[1:]).reshape(x.shape), host(out0), what + " output, unaligned")
            assert float(by[0]) == 0.0


@pytest.mark.parametrize("act", ["leaky", "mish"])
def test_epilogue_with_shortcut_matches_the_checkers_two_layers(ops, oracle, act):
    for si, (N, C, HW) in enumerate([(3, 16, 361), (16, 128, 1444), (8, 192, 4800), (4, 8, 52 * 52), (5, 1024, 361)]):
        x, scale, bias, rmean, rvar = bn_case(3200 + si, N, C, HW, spread=1.5)
        frm = wl.normal(3250 + si, x.shape)
        alpha, beta = 1.0, 1.0
        y_w = x.copy(); pre_w = np.empty_like(x); xs_w = np.empty_like(x); xn_w = np.empty_like(x)
        mean_w = np.zeros(C, F); var_w = np.zeros(C, F)
        oracle.conv_epilogue_forward(True, True, act, N, C, HW, 1, y_w, pre_w, mean_w, var_w, rmean.copy(), rvar.copy(),
                                     scale, bias, xs_w, xn_w, wide=N * HW > WIDE_ABOVE)
        out_w = np.empty_like(x); sc_pre = np.empty_like(x)
        oracle.shortcut_forward("linear", N, HW, 1, C, y_w, frm, alpha, beta, out_w, sc_pre)
        gy = gpu(np.zeros_like(x))
        ops.bn_train_act_shortcut_forward(gpu(x), gy, gpu(np.zeros(C, F)), gpu(np.zeros(C, F)), gpu(rmean), gpu(rvar),
                                          gpu(scale), gpu(bias), act, gpu(frm), alpha, beta)
        # the epilogue's own bound (relative to the operands of x_hat * scale + bias), carried into a sum
        # with the shortcut's source
        sigma = np.sqrt(var_w.astype(np.float64))
        fl = ((np.abs(mean_w) + sigma) / sigma * np.abs(scale) + np.abs(bias)).reshape(1, C, 1, 1) + np.abs(frm)
        assert_close(host(gy), out_w, 1e-5, fl, "%s %s" % (act, (N, C, HW)))


def test_epilogue_with_shortcut_argument_checks(ops):
    from pixienn_amd import capi
    x = gpu(np.zeros((2, 4, 16, 1), F)); c = gpu(np.zeros(4, F))
    args = [x.data_ptr(), x.data_ptr(), None, None, None] + [c.data_ptr()] * 6
    rc = capi.call_raw("pxh_bn_train_act_shortcut_forward", *args, None, 1.0, 1.0, 2, 4, 16, 0, None, 0, None)
    assert rc == -1 and "from" in capi.last_error()
    pre = gpu(np.zeros((2, 4, 16, 1), F))
    args[2] = pre.data_ptr()
    rc = capi.call_raw("pxh_bn_train_act_shortcut_forward", *args, pre.data_ptr(), 1.0, 1.0, 2, 4, 16, 0, None, 0, None)
    assert rc == -1 and "alias" in capi.last_error()
    rc = capi.call_raw("pxh_bn_folded_act_shortcut_forward", x.data_ptr(), x.data_ptr(), None, None, x.data_ptr(), 1.0,
                       1.0, 2, 4, 16, 0, None)
    assert rc == -1
