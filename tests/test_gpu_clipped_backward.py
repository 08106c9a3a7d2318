"""GPU parity: Layer::backward's gradient rescale + clip folded into the conv epilogue's backward
(pxh_bn_act_backward_clipped, pxh_bias_act_backward_clipped) against the checker's composition of the
two steps, include/Layer.h:385-397 then include/ConvLayer.h:244-252 of the reference, on the same
seeded inputs: below the threshold (nothing changes), rescale only, clamp only, both, and a clamp that
bites in some channels only.

Tolerance: 1e-5 relative as for the plain backward, with its floors scaled by the size of the delta
that reaches the sums (a rescaled delta is smaller by the factor, and so is everything linear in it).
"""
import numpy as np
import pytest

from pixienn_amd import workloads as wl
from test_gpu_epilogue import TRAIN_SHAPES, WIDE_ABOVE, bn_case
from util import F, assert_bit_exact, assert_close, gpu, host

pytestmark = pytest.mark.gpu

RTOL = 1e-5


@pytest.fixture(scope="module")
def ops():
    from pixienn_amd import ops as o
    return o


def cases(delta):
    """(name, threshold, clip, delta) for one shape; thresholds are placed well away from the norm."""
    norm = float(np.sqrt(np.sum(delta.astype(np.float64) ** 2)))
    peak = float(np.abs(delta).max())
    spiky = delta.copy()
    spiky[:, 0] *= 20.0                      # one channel far above the others
    spiky_norm = float(np.sqrt(np.sum(spiky.astype(np.float64) ** 2)))
    return [
        ("nothing changes", 2.0 * norm, 2.0 * peak, delta),
        ("helpers off", 0.0, 0.0, delta),
        ("rescale only", 0.37 * norm, 0.0, delta),
        ("rescale, clamp far away", 0.37 * norm, 2.0 * peak, delta),
        ("clamp only", 2.0 * norm, 0.8, delta),
        ("rescale and clamp", 0.5 * norm, 0.3, delta),
        ("clamp bites in one channel only", 2.0 * spiky_norm, 1.5 * peak, spiky),
        ("rescale, and the clamp bites in one channel only", 0.6 * spiky_norm, 0.8 * peak, spiky),
    ]


@pytest.mark.parametrize("act", ["leaky", "linear", "mish"])
@pytest.mark.parametrize("with_pre", [True, False])
def test_bn_backward_clipped_matches_rescale_clip_then_backward(ops, oracle, act, with_pre):
    for si, (N, C, HW) in enumerate(TRAIN_SHAPES):
        x, scale, bias, rmean, rvar = bn_case(1600 + si, N, C, HW, spread=1.5)
        delta0 = wl.normal(1650 + si, x.shape)
        out = x.copy(); pre = np.empty_like(x); xs = np.empty_like(x); xn = np.empty_like(x)
        mean = np.zeros(C, F); var = np.zeros(C, F)
        wide = N * HW > WIDE_ABOVE
        oracle.conv_epilogue_forward(True, True, act, N, C, HW, 1, out, pre, mean, var, rmean.copy(), rvar.copy(),
                                     scale, bias, xs, xn, wide=wide)
        su0 = wl.normal(1660 + si, C); bu0 = wl.normal(1661 + si, C)
        gx, gpre, gmean, gvar, gscale, gbias = gpu(x), gpu(pre), gpu(mean), gpu(var), gpu(scale), gpu(bias)
        for name, threshold, clip, delta in cases(delta0):
            d_w = delta.copy()
            norm_w = oracle.rescale_clip(d_w, threshold, clip)
            size = float(np.sqrt(np.mean(d_w.astype(np.float64) ** 2)))      # of the delta that reaches the sums
            su_w = su0.copy(); bu_w = bu0.copy(); md_w = np.zeros(C, F); vd_w = np.zeros(C, F)
            oracle.conv_epilogue_backward(True, act, N, C, HW, 1, d_w, pre, mean, var, md_w, vd_w, scale, su_w, bu_w,
                                          xs, xn, wide=wide)
            gd = gpu(delta); gsu = gpu(su0); gbu = gpu(bu0); gmd = gpu(np.zeros(C, F)); gvd = gpu(np.zeros(C, F))
            gnorm = gpu(np.zeros(1, F))
            ops.bn_act_backward_clipped(gd, gx, gmean, gvar, gscale, gbias, gsu, gbu, act, threshold, clip,
                                        norm_out=gnorm, pre_activation=gpre if with_pre else None, mean_delta=gmd,
                                        var_delta=gvd)
            what = "%s pre=%s %s, %s" % (act, with_pre, (N, C, HW), name)
            assert_close(host(gnorm), np.array([norm_w], F), 1e-6, 1e-30, what + " norm")
            # a sum's floor follows the size of what was added up: the channel's own delta where it is
            # larger than the tensor's (the channel that was made to stand out)
            per_channel = np.sqrt(np.mean(d_w.astype(np.float64) ** 2, axis=(0, 2, 3)))
            sum_scale = np.sqrt(N * HW) * np.maximum(per_channel, size)
            # an accumulated update is held relative to what was added to it
            assert_close(host(gbu) - bu0, bu_w - bu0, RTOL, np.maximum(sum_scale, 1e-2 * np.abs(bu0).max()), what + " bias updates")
            assert_close(host(gsu) - su0, su_w - su0, RTOL, np.maximum(sum_scale, 1e-2 * np.abs(su0).max()), what + " scale updates")
            assert_close(host(gmd), md_w, RTOL, sum_scale, what + " mean delta")
            assert_close(host(gvd), vd_w, RTOL, sum_scale, what + " var delta")
            assert_close(host(gd), d_w, RTOL, 1e-1 * size, what + " dx")
            if name in ("nothing changes", "helpers off"):
                # ... and then it is the plain backward to the bit
                gd2 = gpu(delta); gsu2 = gpu(su0); gbu2 = gpu(bu0)
                ops.bn_act_backward(gd2, gx, gmean, gvar, gscale, gbias, gsu2, gbu2, act,
                                    pre_activation=gpre if with_pre else None)
                assert_bit_exact(host(gd), host(gd2), what + " dx against the plain backward")
                assert_bit_exact(host(gsu), host(gsu2), what + " scale updates against the plain backward")
                assert_bit_exact(host(gbu), host(gbu2), what + " bias updates against the plain backward")


@pytest.mark.parametrize("act", ["linear", "leaky", "logistic"])
def test_bias_backward_clipped_matches_rescale_clip_then_backward(ops, oracle, act):
    for si, (N, C, HW) in enumerate([(2, 255, 169), (3, 18, 361), (2, 4, 4096), (3, 5, 27), (16, 255, 361)]):
        pre = wl.normal(1700 + si, (N, C, HW, 1))
        delta0 = wl.normal(1710 + si, pre.shape)
        bu0 = wl.normal(1720 + si, C)
        for name, threshold, clip, delta in cases(delta0):
            d_w = delta.copy(); bu_w = bu0.copy()
            norm_w = oracle.rescale_clip(d_w, threshold, clip)
            size = float(np.sqrt(np.mean(d_w.astype(np.float64) ** 2)))
            oracle.conv_epilogue_backward(False, act, N, C, HW, 1, d_w, pre, None, None, None, None, None, None, bu_w,
                                          None, None)
            gd = gpu(delta); gbu = gpu(bu0); gnorm = gpu(np.zeros(1, F))
            ops.bias_act_backward_clipped(gd, gpu(pre), gbu, act, threshold, clip, norm_out=gnorm)
            what = "bias %s %s, %s" % (act, (N, C, HW), name)
            assert_close(host(gnorm), np.array([norm_w], F), 1e-6, 1e-30, what + " norm")
            if act == "logistic":
                assert_close(host(gd), d_w, RTOL, 1e-6 * size, what + " delta")
            else:
                assert_bit_exact(host(gd), d_w, what + " delta")
            assert_close(host(gbu) - bu0, bu_w - bu0, RTOL, max(np.sqrt(N * HW) * size, 1e-2 * np.abs(bu0).max()),
                         what + " bias updates")


def test_clipped_backward_argument_checks(ops):
    from pixienn_amd import capi
    assert capi.load().pxh_bn_clipped_workspace_bytes(0, 4, 4) == 0
    need = capi.load().pxh_bn_clipped_workspace_bytes(2, 4, 16)
    assert need >= capi.load().pxh_bn_workspace_bytes(2, 4, 16)
    d = gpu(np.zeros((2, 4, 16, 1), F)); c = gpu(np.zeros(4, F))
    small = gpu(np.zeros(4, F))
    rc = capi.call_raw("pxh_bn_act_backward_clipped", d.data_ptr(), d.data_ptr(), None, c.data_ptr(), c.data_ptr(),
                       c.data_ptr(), c.data_ptr(), c.data_ptr(), c.data_ptr(), None, None, 2, 4, 16, 0, 1.0, 1.0, None,
                       small.data_ptr(), 16, None)
    assert rc < 0 and "workspace" in capi.last_error()
    rc = capi.call_raw("pxh_bias_act_backward_clipped", None, None, c.data_ptr(), 2, 4, 16, 1, 1.0, 1.0, None, None, 0,
                       None)
    assert rc < 0
