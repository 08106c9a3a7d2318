"""GPU parity of pxh_bn_train_act_forward_static, the BN-training forward for callers that cannot
allocate: its partial sums and per-channel constants live in a buffer built into the library's
device code instead of a workspace.  It runs the same kernels as pxh_bn_train_act_forward, so every
output must be bit-identical to that entry point's on the same inputs (which the epilogue tests hold
to 1e-5 of the CPU checker) -- on two calls in a row, the second with a smaller input, so that what
the first left in the shared buffer is seen not to leak into the second.
"""
import numpy as np
import pytest
import torch

from pixienn_amd import capi, workloads as wl
from util import F, assert_bit_exact, gpu, host

pytestmark = pytest.mark.gpu

STATIC_BYTES = 1 << 20      # PXH_BN_STATIC_SCRATCH_BYTES of include/pixienn_hip.h


def run(entry, x, scale, bias, rmean, rvar, act, with_workspace):
    """One call of `entry` through the C ABI on fresh device tensors; returns every output on the host."""
    N, C, HW = x.shape[0], x.shape[1], x.shape[2] * x.shape[3]
    gx = gpu(x)
    gy, gpre, gxs, gxn = (torch.full(x.shape, 7.0, device="cuda") for _ in range(4))
    gm, gv = torch.zeros(C, device="cuda"), torch.zeros(C, device="cuda")
    grm, grv = gpu(rmean), gpu(rvar)
    gs, gb = gpu(scale), gpu(bias)
    stream = torch.cuda.current_stream().cuda_stream
    args = [gx.data_ptr(), gy.data_ptr(), gpre.data_ptr(), gxs.data_ptr(), gxn.data_ptr(), gm.data_ptr(),
            gv.data_ptr(), grm.data_ptr(), grv.data_ptr(), gs.data_ptr(), gb.data_ptr(), N, C, HW,
            capi.act_id(act)]
    if with_workspace:
        need = int(capi.load().pxh_bn_workspace_bytes(N, C, HW))
        ws = torch.zeros(need // 4 + 4, device="cuda")
        args += [ws.data_ptr(), ws.numel() * 4]
    capi.call(entry, *args, stream)
    return {k: host(t) for k, t in dict(y=gy, pre=gpre, x_saved=gxs, x_norm=gxn, mean=gm, var=gv, rolling_mean=grm,
                                        rolling_var=grv).items()}


def case(seed, N, C, H, W):
    x = wl.normal(seed, (N, C, H, W), std=1.5) + wl.normal(seed + 1, (1, C, 1, 1), std=2.0)
    scale, bias, rmean, rvar = wl.bn_params(seed + 2, C)
    return x.astype(F), scale, bias, rmean, rvar


# Two calls in a row on the shared buffer.  The first of each pair takes the three-launch form with
# many partial sums per channel; the second is smaller (fewer channels, fewer partials, then a shape
# of the one-launch form that uses no scratch at all).
PAIRS = [
    ((4, 32, 64, 64), (2, 16, 40, 40), "leaky"),
    ((3, 24, 76, 76), (2, 5, 13, 13), "mish"),
    ((16, 64, 152, 152), (3, 96, 19, 19), "leaky"),
]


@pytest.mark.parametrize("first,second,act", PAIRS)
def test_static_scratch_matches_workspace_entry_point(first, second, act):
    lib = capi.load()
    for seed, shape in ((900, first), (910, second)):
        N, C, H, W = shape
        assert lib.pxh_bn_workspace_bytes(N, C, H * W) <= STATIC_BYTES
        x, scale, bias, rmean, rvar = case(seed, N, C, H, W)
        want = run("pxh_bn_train_act_forward", x, scale, bias, rmean, rvar, act, True)
        got = run("pxh_bn_train_act_forward_static", x, scale, bias, rmean, rvar, act, False)
        for k in want:
            assert_bit_exact(got[k], want[k], "%s %s %s" % (shape, act, k))
        assert_bit_exact(got["x_saved"], x, "%s x_saved" % (shape,))


def test_static_scratch_rejects_a_shape_beyond_its_buffer():
    lib = capi.load()
    N, C, HW = 32, 2048, 128 * 128          # 1 MB of partial sums + 128 KB of constants
    assert lib.pxh_bn_workspace_bytes(N, C, HW) > STATIC_BYTES
    # rejected before anything is launched or read: one small tensor stands in for every pointer
    t = torch.zeros(64, device="cuda")
    p = t.data_ptr()
    q = torch.zeros(64, device="cuda").data_ptr()
    rc = capi.call_raw("pxh_bn_train_act_forward_static", p, q, None, None, None, q, q, q, q, q, q, N, C, HW, 0,
                       torch.cuda.current_stream().cuda_stream)
    assert rc == -3, rc                     # PXH_ERR_WORKSPACE
    msg = capi.last_error()
    assert "scratch" in msg and "pxh_bn_train_act_forward" in msg, msg
    torch.cuda.synchronize()
    assert float(t.abs().sum()) == 0.0
