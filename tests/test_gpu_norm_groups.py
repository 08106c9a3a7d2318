"""GPU parity of the norm + peak that a kernel leaves behind when it writes a delta
(pxh_norm_groups, pxh_axpy_norm, pxh_shortcut_backward_norm, pxh_rescale_clip_from_groups).

Layer::backward opens with the gradient rescale + clip of the layer's own delta
(include/Layer.h:385-397 of the reference); pxh_rescale_clip, which the other tests hold to the CPU
checker, reads the tensor once for the norm.  The entry points here spare that read, and must leave
the norm, the verdict (nothing to do / rewrite) and the rewritten tensor as pxh_rescale_clip does on
the same data, bit for bit -- for lengths on every side of the group (256), step (8192) and grid
(1024 steps) boundaries, for tensors without group sums (unaligned, length not a multiple of 4), and
with NaN and infinity among the values.  The producers must also leave their own tensors exactly as
the plain entry points do."""
import numpy as np
import pytest
import torch

from pixienn_amd import workloads as wl
from util import assert_bit_exact, gpu, host

pytestmark = pytest.mark.gpu

# groups of 256, steps of 8192 values, 1024 workgroups: one step each up to 8 388 608 values
SIZES = [4, 252, 256, 260, 1020, 8188, 8192, 8196, 3 * 8192 + 512, 1000 * 8192 + 36, 1024 * 8192, 1024 * 8192 + 4,
         2 * 1024 * 8192 + 8192 + 260, 5 * 1024 * 8192 + 77 * 256]
NO_GROUPS = [1, 3, 255, 8190, 100001]          # lengths that are not a multiple of 4


@pytest.fixture(scope="module")
def ops():
    from pixienn_amd import ops as o
    return o


def settings(norm):
    return [("below", 2.0 * norm, 0.0), ("rescale", 0.5 * norm, 0.0), ("clip", 0.0, 0.7), ("both", 0.25 * norm, 0.05),
            ("clip above the peak", 0.0, 1e6)]


def poisoned(ops, x):
    """A group buffer whose stale contents would show: NaN everywhere."""
    g = ops.norm_groups_like(x)
    g.fill_(float("nan"))
    return g


def copy_of(x):
    """A copy at the same offset from a 16-byte boundary (clone() would align it)."""
    off = x.data_ptr() % 16 // 4
    buf = torch.empty(x.numel() + 4, dtype=x.dtype, device=x.device)
    out = buf[off:off + x.numel()]
    out.copy_(x)
    assert out.data_ptr() % 16 == x.data_ptr() % 16
    return out


def both_ways(ops, x, groups, threshold, clip, what):
    """rescale + clip of copies of x through the tensor's own read and through the group sums."""
    a, b = copy_of(x), copy_of(x)
    na = torch.full((1,), -1.0, device=x.device)
    nb = torch.full((1,), -2.0, device=x.device)
    ops.rescale_clip(a, threshold, clip, na)
    ops.rescale_clip_from_groups(b, groups, threshold, clip, nb)
    assert_bit_exact(host(nb), host(na), "norm, " + what)
    assert_bit_exact(host(b), host(a), "tensor, " + what)
    return float(na)


@pytest.mark.parametrize("n", SIZES)
def test_group_sums_of_a_tensor_give_what_the_read_gives(ops, n):
    x = gpu(wl.normal(9100 + n % 97, n, std=0.3))
    groups = poisoned(ops, x)
    ops.norm_groups(x, groups)
    used = (n + 255) // 256
    g = host(groups)[:2 * used].reshape(used, 2)
    assert not np.isnan(g).any(), "every group of the tensor is written"
    xs = host(x).astype(np.float64)
    want = np.add.reduceat(xs * xs, np.arange(0, n, 256))
    assert np.allclose(g[:, 0], want, rtol=2e-6, atol=0), "group sums of squares"
    peaks = np.maximum.reduceat(np.abs(host(x)), np.arange(0, n, 256))
    assert np.array_equal(g[:, 1], peaks), "group peaks"
    if 2 * used < groups.numel():
        assert np.isnan(host(groups)[2 * used:]).all(), "nothing past the tensor's groups is written"
    norm = float(np.sqrt((xs * xs).sum()))
    for name, threshold, clip in settings(norm):
        got = both_ways(ops, x, groups, threshold, clip, "%s n=%d" % (name, n))
        assert abs(got - norm) <= 1e-6 * norm


@pytest.mark.parametrize("n", NO_GROUPS + [4096])
def test_tensors_without_group_sums_are_read(ops, n):
    """Length not a multiple of 4, or a pointer that is not 16-byte aligned: the producers leave the
    buffer alone and the consumer reads the tensor."""
    base = gpu(wl.normal(9200 + n % 89, n + 1, std=0.3))
    x = base[1:] if n == 4096 else base[:n]
    groups = poisoned(ops, x)
    ops.norm_groups(x, groups)
    assert np.isnan(host(groups)).all()
    norm = float(np.sqrt((host(x).astype(np.float64) ** 2).sum()))
    for name, threshold, clip in settings(norm):
        both_ways(ops, x, groups, threshold, clip, "%s n=%d, no groups" % (name, n))


@pytest.mark.parametrize("bad", ["nan", "inf", "-inf"])
def test_nan_and_infinity_show_the_same_way(ops, bad):
    n = 3 * 8192 + 512
    xs = wl.normal(9300, n, std=0.3)
    xs[12345] = float(bad)
    x = gpu(xs)
    groups = poisoned(ops, x)
    ops.norm_groups(x, groups)
    for name, threshold, clip in settings(1.0):
        a, b = x.clone(), x.clone()
        na = torch.zeros(1, device=x.device); nb = torch.ones(1, device=x.device)
        ops.rescale_clip(a, threshold, clip, na)
        ops.rescale_clip_from_groups(b, groups, threshold, clip, nb)
        assert_bit_exact(host(nb).view(np.int32), host(na).view(np.int32), "norm bits, %s %s" % (bad, name))
        assert_bit_exact(host(b).view(np.int32), host(a).view(np.int32), "tensor bits, %s %s" % (bad, name))


@pytest.mark.parametrize("first", [False, True])
@pytest.mark.parametrize("act", ["linear", "leaky"])
@pytest.mark.parametrize("n", [1024, 8192 + 260, 16 * 64 * 38 * 38, 1024 * 8192 + 8192 + 4, 1023])
def test_shortcut_backward_leaves_the_group_sums_of_grad(ops, n, act, first):
    delta = gpu(wl.normal(9400, n, std=0.4))
    pre = gpu(wl.normal(9401, n)) if act != "linear" else None
    frm = gpu(wl.normal(9402, n, std=0.2))
    grad = gpu(wl.normal(9403, n, std=0.2))
    d2, f2, g2 = delta.clone(), frm.clone(), grad.clone()
    plain = ops.shortcut_backward_first if first else ops.shortcut_backward
    plain(delta, frm, grad, act, 0.75, 1.25, pre)
    groups = poisoned(ops, g2)
    ops.shortcut_backward_norm(d2, f2, g2, groups, act, 0.75, 1.25, pre, first=first)
    what = "n=%d %s first=%s" % (n, act, first)
    assert_bit_exact(host(d2), host(delta), "delta, " + what)
    assert_bit_exact(host(f2), host(frm), "from_delta, " + what)
    assert_bit_exact(host(g2), host(grad), "grad, " + what)
    norm = float(grad.double().norm())
    for name, threshold, clip in settings(norm):
        both_ways(ops, g2, groups, threshold, clip, name + " " + what)


@pytest.mark.parametrize("n", [4, 1024, 16 * 255 * 19 * 19, 1024 * 8192 + 260, 999])
def test_axpy_leaves_the_group_sums_of_y(ops, n):
    x = gpu(wl.normal(9500, n, std=0.4))
    y = gpu(wl.normal(9501, n, std=0.2))
    y2 = y.clone()
    ops.axpy(0.5, x, y)
    groups = poisoned(ops, y2)
    ops.axpy_norm(0.5, x, y2, groups)
    assert_bit_exact(host(y2), host(y), "y n=%d" % n)
    norm = float(y.double().norm())
    for name, threshold, clip in settings(norm):
        both_ways(ops, y2, groups, threshold, clip, "%s after axpy n=%d" % (name, n))


def test_an_unaligned_operand_still_leaves_the_group_sums(ops):
    """grad aligned, delta not: the flat 128-bit kernel cannot run, the group sums are formed by a
    read of grad after the plain kernel."""
    n = 8192 + 512
    base = gpu(wl.normal(9600, n + 1, std=0.4))
    delta = base[1:]
    frm = gpu(wl.normal(9601, n, std=0.2)); grad = gpu(wl.normal(9602, n, std=0.2))
    d2, f2, g2 = copy_of(delta), frm.clone(), grad.clone()
    ops.shortcut_backward(delta, frm, grad, "linear", 1.0, 1.0)
    groups = poisoned(ops, g2)
    ops.shortcut_backward_norm(d2, f2, g2, groups, "linear", 1.0, 1.0)
    assert_bit_exact(host(g2), host(grad), "grad")
    assert not np.isnan(host(groups)[:2 * ((n + 255) // 256)]).any()
    both_ways(ops, g2, groups, 0.5 * float(grad.double().norm()), 0.05, "unaligned delta")


def test_errors(ops):
    from pixienn_amd.capi import PxError
    x = gpu(np.zeros(1024, np.float32))
    with pytest.raises(PxError):
        ops.rescale_clip_from_groups(x, None, 1.0, 0.0)
    with pytest.raises(PxError):
        ops.shortcut_backward_norm(x, x.clone(), None, ops.norm_groups_like(x))
    with pytest.raises(PxError):
        ops.shortcut_backward_norm(x, x.clone(), x.clone(), None)
