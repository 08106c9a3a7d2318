"""Helpers shared by the GPU parity tests."""
import numpy as np

F = np.float32


def gpu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    import torch
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


def ulp_distance(a, b):
    """Distance in units in the last place between two float32 arrays (NaN == NaN -> 0)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    ia = a.view(np.int32).astype(np.int64)
    ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7FFFFFFF), ia)
    ib = np.where(ib < 0, -(ib & 0x7FFFFFFF), ib)
    d = np.abs(ia - ib)
    both_nan = np.isnan(a) & np.isnan(b)
    return np.where(both_nan, 0, d)


def assert_bit_exact(got, want, what=""):
    got = np.ascontiguousarray(got)
    want = np.ascontiguousarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if got.dtype == np.float32:
        same = (got.view(np.int32) == want.view(np.int32)) | (np.isnan(got) & np.isnan(want))
    else:
        same = got == want
    if not same.all():
        bad = np.argwhere(~same)
        i = tuple(bad[0])
        raise AssertionError("%s: %d of %d elements differ, first at %s: got %r want %r"
                             % (what, len(bad), same.size, i, got[i], want[i]))


def assert_close(got, want, rtol, floor, what=""):
    """|got - want| <= rtol * max(|want|, floor), element-wise.

    `floor` is the magnitude below which a result is the difference of larger intermediates
    (e.g. x_hat*scale + bias cancelling): there the bound is rtol relative to that magnitude.
    """
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert np.isfinite(got).all() == np.isfinite(want).all(), what
    err = np.abs(got - want)
    bound = rtol * np.maximum(np.abs(want), floor)
    bad = err > bound
    if bad.any():
        i = tuple(np.argwhere(bad)[0])
        here = float(np.broadcast_to(np.asarray(floor, dtype=np.float64), want.shape)[i])
        raise AssertionError("%s: %d of %d beyond rtol %g (floor %g there); first at %s: got %.9g want %.9g; "
                             "worst rel %.3g" % (what, int(bad.sum()), bad.size, rtol, here, i, got[i], want[i],
                                                 float(np.max(err / np.maximum(np.abs(want), floor)))))


def max_rel(got, want, floor):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), floor)))


def detection_records(oracle, rows):
    """rows of [left, top, width, height, batch, class, prob] -> detection records in that order."""
    rec = np.zeros(len(rows), oracle.DETECTION_DTYPE)
    for i, (x, y, w, h, b, c, p) in enumerate(rows):
        rec[i] = (x, y, w, h, p, b, c, i)
    return rec


def random_detections(oracle, seed, n, batch, classes, clusters, spread=6.0):
    """Overlapping boxes around a few centres per image (pixienn_amd.workloads.detection_clusters)."""
    from pixienn_amd import workloads
    assert workloads.DETECTION_DTYPE == oracle.DETECTION_DTYPE
    return workloads.detection_clusters(seed, n, batch, classes, clusters, spread)
