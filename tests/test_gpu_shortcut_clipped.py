"""GPU parity: a ShortcutLayer's whole backward in one call (pxh_shortcut_backward_clipped) -- Layer::backward's
rescale + clip of the layer's delta, include/Layer.h:385-397 and 474-499 of the reference, then the shortcut's
own backward, include/ShortcutLayer.h:98-111 -- against the two calls it stands for (pxh_rescale_clip, then
pxh_shortcut_backward_first or pxh_shortcut_backward, each held to the CPU checker elsewhere): to the bit in the
delta, both targets and the norm, for the form that reads the delta once (first writer, linear, 128-bit) and for
every case that runs the sequence itself; and against the checker's own composition of the two steps."""
import numpy as np
import pytest

from pixienn_amd import workloads as wl
from util import F, assert_bit_exact, assert_close, gpu, host

pytestmark = pytest.mark.gpu

# values: less than one step of the walk, a few steps with a ragged last one, more steps than the capped grid
# takes at once (1024 workgroups x 8192 values), not a multiple of four
SIZES = [4, 1000, 8192, 3 * 8192 + 260, 16 * 64 * 38 * 38, 1024 * 8192 + 5 * 8192 + 12, 1003, 4 * 100000 + 2]


@pytest.fixture(scope="module")
def ops():
    from pixienn_amd import ops as o
    return o


def cases(delta):
    norm = float(np.sqrt(np.sum(delta.astype(np.float64) ** 2)))
    peak = float(np.abs(delta).max())
    return [("nothing changes", 2.0 * norm, 2.0 * peak), ("rescale only", 0.37 * norm, 0.0),
            ("clamp only", 0.0, 0.5 * peak), ("clamp only, far away", 2.0 * norm, 3.0 * peak),
            ("rescale and clamp", 0.5 * norm, 0.2 * peak), ("norm only", 0.0, 0.0)]


def place(a, offset):
    """On the device; optionally `offset` floats past a 16-byte boundary."""
    import torch
    if a is None:
        return None
    buf = torch.empty(a.size + 4, device="cuda")
    view = buf[offset:offset + a.size]
    view.copy_(torch.from_numpy(np.ascontiguousarray(a).reshape(-1)))
    return view


def two_calls(ops, delta, frm, grad, first, act, pre, alpha, beta, threshold, clip, offset=0):
    import torch
    d, f, g, p = place(delta, offset), place(frm, offset), place(grad, offset), place(pre, offset)
    norm = torch.full((1,), -1.0, device="cuda")
    ops.rescale_clip(d, threshold, clip, norm_out=norm)
    if first:
        ops.shortcut_backward_first(d, f, g, act, alpha, beta, pre_activation=p)
    else:
        ops.shortcut_backward(d, f, g, act, alpha, beta, pre_activation=p)
    return host(d), host(f), None if g is None else host(g), float(host(norm)[0])


def one_call(ops, delta, frm, grad, first, act, pre, alpha, beta, threshold, clip, offset=0):
    import torch
    d, f, g, p = place(delta, offset), place(frm, offset), place(grad, offset), place(pre, offset)
    norm = torch.full((1,), -1.0, device="cuda")
    ops.shortcut_backward_clipped(d, f, g, act, alpha, beta, pre_activation=p, first=first, threshold=threshold,
                                  clip=clip, norm_out=norm)
    return host(d), host(f), None if g is None else host(g), float(host(norm)[0])


def same(got, want, what):
    assert_bit_exact(got[0], want[0].reshape(-1), what + " delta")
    assert_bit_exact(got[1], want[1].reshape(-1), what + " from_delta")
    if want[2] is not None:
        assert_bit_exact(got[2], want[2].reshape(-1), what + " grad")
    assert got[3] == want[3], (what, "norm", got[3], want[3])


@pytest.mark.parametrize("with_grad", [True, False])
def test_first_writer_form_is_the_two_calls_to_the_bit(ops, with_grad):
    for si, n in enumerate(SIZES):
        delta = wl.normal(8100 + si, n)
        frm = wl.normal(8150 + si, n); grad = wl.normal(8170 + si, n) if with_grad else None
        alpha, beta = [(1.0, 1.0), (0.75, -1.5)][si % 2]
        for name, threshold, clip in cases(delta):
            what = "n %d %s alpha %g beta %g" % (n, name, alpha, beta)
            want = two_calls(ops, delta, frm, grad, True, "linear", None, alpha, beta, threshold, clip)
            got = one_call(ops, delta, frm, grad, True, "linear", None, alpha, beta, threshold, clip)
            same(got, want, what)
            if name == "nothing changes":
                assert_bit_exact(got[0], delta.reshape(-1), what + ": the delta is left alone")
        # tensors that do not start on a 16-byte boundary run the sequence itself
        name, threshold, clip = cases(delta)[4]
        want = two_calls(ops, delta, frm, grad, True, "linear", None, alpha, beta, threshold, clip, offset=1)
        got = one_call(ops, delta, frm, grad, True, "linear", None, alpha, beta, threshold, clip, offset=1)
        same(got, want, "n %d unaligned %s" % (n, name))


@pytest.mark.parametrize("act", ["linear", "leaky", "mish"])
def test_accumulating_and_non_linear_forms_run_the_sequence(ops, act):
    for si, n in enumerate([1000, 3 * 8192 + 260, 1003]):
        delta = wl.normal(8200 + si, n); pre = wl.normal(8210 + si, n)
        frm = wl.normal(8250 + si, n); grad = wl.normal(8270 + si, n)
        for first in (False, True):
            if first and act == "linear":
                continue
            for name, threshold, clip in cases(delta):
                what = "%s n %d first %s %s" % (act, n, first, name)
                p = None if act == "linear" else pre
                want = two_calls(ops, delta, frm, grad, first, act, p, 1.0, 1.0, threshold, clip)
                got = one_call(ops, delta, frm, grad, first, act, p, 1.0, 1.0, threshold, clip)
                same(got, want, what)


def test_matches_the_checkers_two_steps(ops, oracle):
    """rescale + clip, then ShortcutLayer::backward into cleared targets, on the CPU checker."""
    N, C, S = 2, 6, 20
    n = N * C * S * S
    delta = wl.normal(8300, n)
    for name, threshold, clip in cases(delta):
        d_w = delta.copy()
        oracle.rescale_clip(d_w, threshold, clip)
        f_w = np.zeros(n, F); g_w = np.zeros(n, F)
        oracle.shortcut_backward("linear", N, S, S, C, d_w, d_w.copy(), f_w, g_w, 1.0, 1.0)
        got = one_call(ops, delta, np.full(n, 7.0, F), np.full(n, 7.0, F), True, "linear", None, 1.0, 1.0, threshold,
                       clip)
        size = float(np.abs(d_w).max())
        assert_close(got[0], d_w, 1e-6, size, name + " delta")
        assert_close(got[1], f_w, 1e-6, size, name + " from_delta")
        assert_close(got[2], g_w, 1e-6, size, name + " grad")


def test_without_helpers_it_is_the_backward_alone_and_bad_arguments_are_rejected(ops):
    import torch
    from pixienn_amd import capi
    n = 4096
    delta = wl.normal(8400, n); frm = wl.normal(8401, n); grad = wl.normal(8402, n)
    d, f, g = gpu(delta), gpu(frm), gpu(grad)
    ops.shortcut_backward_clipped(d, f, g, "linear", 1.0, 1.0, first=True)
    assert_bit_exact(host(d), delta, "delta"); assert_bit_exact(host(f), delta, "from_delta")
    assert_bit_exact(host(g), delta, "grad")
    args = (n, 1.0, 1.0, 1, 1, 1.0, 1.0, None, None, 0, None)
    rc = capi.call_raw("pxh_shortcut_backward_clipped", d.data_ptr(), None, d.data_ptr(), g.data_ptr(), *args)
    assert rc == -1 and "of its own" in capi.last_error()
    rc = capi.call_raw("pxh_shortcut_backward_clipped", d.data_ptr(), None, f.data_ptr(), f.data_ptr(), *args)
    assert rc == -1 and "distinct" in capi.last_error()
    rc = capi.call_raw("pxh_shortcut_backward_clipped", d.data_ptr(), None, None, g.data_ptr(), *args)
    assert rc == -1
    rc = capi.call_raw("pxh_shortcut_backward_clipped", d.data_ptr(), None, f.data_ptr(), g.data_ptr(), n, 1.0, 1.0, 0, 1,
                       1.0, 1.0, None, None, 0, None)
    assert rc == -1 and "pre_activation" in capi.last_error()
    small = torch.empty(8, device="cuda")
    rc = capi.call_raw("pxh_shortcut_backward_clipped", d.data_ptr(), None, f.data_ptr(), g.data_ptr(), n, 1.0, 1.0, 1, 1,
                       1.0, 1.0, None, small.data_ptr(), 32, None)
    assert rc == -3
