"""GPU parity: a convolution's inference epilogue with the 2 x 2, stride 2 MaxPoolLayer that follows it in
the same pass (pxh_bn_folded_act_maxpool_forward) against the two layers one after the other --
include/cuda/ConvLayer.h:284-307 (inference) then include/cuda/MaxPoolLayer.h:23-37 of the reference: to the
bit against this library's own two calls (each held to the CPU checker elsewhere), and against the checker's
two layers, for the three widths of the kernel (rows of a multiple of 8, of 4, of 2 floats), with and without
the layer's own output, with NaN and infinities among the values."""
import numpy as np
import pytest

from pixienn_amd import workloads as wl
from test_gpu_epilogue import bn_case
from util import F, assert_bit_exact, assert_close, gpu, host

pytestmark = pytest.mark.gpu

# N, C, H, W: the YOLOv3-tiny planes (416 ... 26), rows of 2 and 6 floats, one window per plane
SHAPES = [(2, 16, 416, 416), (2, 32, 208, 208), (3, 8, 104, 104), (3, 8, 52, 52), (2, 5, 26, 26), (1, 3, 2, 2),
          (2, 4, 6, 10), (3, 7, 8, 6), (2, 3, 4, 12), (1, 130, 38, 38)]


@pytest.fixture(scope="module")
def ops():
    from pixienn_amd import ops as o
    return o


def two_calls(ops, gx, folded, act, N, C, H, W):
    import torch
    y = torch.zeros_like(gx)
    ops.bn_folded_act_forward(gx.view(N, C, H * W, 1), y.view(N, C, H * W, 1), folded, act)
    pooled = torch.zeros((N, C, H // 2, W // 2), device="cuda")
    idx = torch.zeros((N, C, H // 2, W // 2), dtype=torch.int32, device="cuda")
    ops.maxpool_forward(y, pooled, idx, 2, 2, 1)
    return y, pooled


@pytest.mark.parametrize("act", ["leaky", "mish", "linear", "relu", "logistic"])
def test_epilogue_with_maxpool_is_the_two_calls_to_the_bit(ops, act):
    import torch
    for si, (N, C, H, W) in enumerate(SHAPES):
        x, scale, bias, rmean, rvar = bn_case(3300 + si, N, C, H * W)
        x = x.reshape(N, C, H, W).copy()
        if x.size > 64:
            flat = x.reshape(-1)
            flat[5] = np.nan; flat[17] = np.inf; flat[33] = -np.inf
        folded = ops.bn_fold(gpu(rmean), gpu(rvar), gpu(scale), gpu(bias))
        gx = gpu(x)
        y_w, pooled_w = two_calls(ops, gx, folded, act, N, C, H, W)
        what = "%s %s" % (act, (N, C, H, W))
        pooled = torch.full((N, C, H // 2, W // 2), 7.0, device="cuda")
        ops.bn_folded_act_maxpool_forward(gx, pooled, folded, act)
        assert_bit_exact(host(pooled), host(pooled_w), what + " pooled")
        pooled = torch.full((N, C, H // 2, W // 2), 7.0, device="cuda")
        y = torch.full((N, C, H, W), 7.0, device="cuda")
        ops.bn_folded_act_maxpool_forward(gx, pooled, folded, act, y=y)
        assert_bit_exact(host(pooled), host(pooled_w), what + " pooled, with the layer's output")
        assert_bit_exact(host(y), host(y_w), what + " the layer's output")


def test_epilogue_with_maxpool_matches_the_checkers_two_layers(ops, oracle):
    for si, (N, C, H, W) in enumerate([(2, 8, 52, 52), (2, 5, 26, 26), (1, 16, 104, 104)]):
        x, scale, bias, rmean, rvar = bn_case(3400 + si, N, C, H * W)
        y_w = x.copy(); pre_w = np.empty_like(x)
        oracle.conv_epilogue_forward(True, False, "leaky", N, C, H * W, 1, y_w, pre_w, np.zeros(C, F), np.zeros(C, F),
                                     rmean.copy(), rvar.copy(), scale, bias, None, None)
        pooled_w = np.zeros((N, C, H // 2, W // 2), F); idx_w = np.zeros((N, C, H // 2, W // 2), np.int32)
        oracle.maxpool_forward(np.ascontiguousarray(y_w.reshape(N, C, H, W)), pooled_w, idx_w, N, C, H, W, H // 2, W // 2,
                               2, 2, 1)
        import torch
        folded = ops.bn_fold(gpu(rmean), gpu(rvar), gpu(scale), gpu(bias))
        pooled = torch.zeros((N, C, H // 2, W // 2), device="cuda")
        ops.bn_folded_act_maxpool_forward(gpu(x.reshape(N, C, H, W)), pooled, folded, "leaky")
        assert_close(host(pooled), pooled_w, 1e-5, 1e-3, "leaky %s" % ((N, C, H, W),))


def test_epilogue_with_maxpool_argument_checks(ops):
    import torch
    from pixienn_amd import capi
    x = torch.zeros((1, 2, 5, 4), device="cuda"); p = torch.zeros((1, 2, 2, 2), device="cuda")
    folded = ops.bn_fold(*(torch.ones(2, device="cuda") for _ in range(4)))
    rc = capi.call_raw("pxh_bn_folded_act_maxpool_forward", x.data_ptr(), None, p.data_ptr(), folded.data_ptr(), 1, 2, 5,
                       4, 0, None)
    assert rc == -2 and "two" in capi.last_error()
    rc = capi.call_raw("pxh_bn_folded_act_maxpool_forward", x.data_ptr(), None, None, folded.data_ptr(), 1, 2, 4, 4, 0,
                       None)
    assert rc == -1
    x = torch.zeros((1, 2, 4, 4), device="cuda")
    rc = capi.call_raw("pxh_bn_folded_act_maxpool_forward", x.data_ptr(), None, x.data_ptr(), folded.data_ptr(), 1, 2, 4,
                       4, 0, None)
    assert rc == -1 and "its own" in capi.last_error()
