"""The entry points inside a HIP graph: a layer sequence is captured once and replayed several
times on new data, with eager work and synchronisations in between; every replay must give
exactly what the same calls give when launched eagerly."""
import numpy as np
import pytest

from pixienn_amd import workloads as wl
from util import F, gpu, host

pytestmark = pytest.mark.gpu


def test_layer_sequence_in_a_graph_matches_eager():
    import torch
    from pixienn_amd import ops
    N, C, S, K = 4, 128, 38, 80
    dev = "cuda"
    scale, bias, rmean0, rvar0 = (gpu(a) for a in wl.bn_params(9000, C))
    truths_np, counts_np = wl.yolo_truths(9001, N)
    truths, counts = gpu(truths_np), gpu(counts_np)
    mask = wl.YOLOV3_MASKS[38]

    # static buffers of the captured sequence
    x = torch.zeros((N, C, S, S), device=dev); d_in = torch.zeros_like(x)
    head_in = torch.zeros((N, 3 * (K + 5), S, S), device=dev)
    buf = dict(y=torch.empty_like(x), mean=torch.zeros(C, device=dev), var=torch.zeros(C, device=dev),
               rmean=rmean0.clone(), rvar=rvar0.clone(), su=torch.zeros(C, device=dev), bu=torch.zeros(C, device=dev),
               d=torch.empty_like(x), pool=torch.empty((N, C, S // 2, S // 2), device=dev),
               idx=torch.empty((N, C, S // 2, S // 2), device=dev, dtype=torch.int32),
               up=torch.empty_like(x), head_out=torch.empty_like(head_in), head_delta=torch.empty_like(head_in),
               stats=torch.zeros(12, device=dev), cost=torch.zeros(1, device=dev), norm=torch.zeros(1, device=dev),
               w=torch.zeros(C * 9, device=dev), wd=torch.zeros(C * 9, device=dev))

    def sequence(b):
        ops.bn_train_act_forward(x, b["y"], b["mean"], b["var"], b["rmean"], b["rvar"], scale, bias, "leaky")
        ops.maxpool_forward(b["y"], b["pool"], b["idx"], 2, 2, 1)
        ops.upsample_forward(b["pool"], b["up"], 2, 1.0)
        b["d"].copy_(d_in)
        ops.rescale_clip(b["d"], 50.0, 0.5, norm_out=b["norm"])
        ops.bn_act_backward(b["d"], x, b["mean"], b["var"], scale, bias, b["su"], b["bu"], "leaky")
        ops.yolo_forward_train(head_in, b["head_out"], b["head_delta"], truths, counts, truths.shape[1], mask,
                               wl.YOLOV3_ANCHORS, b["stats"], b["cost"], N, K, S, S, 608, 608, 0.7, 1.0, 1.0, 2.0,
                               0.1, 1.0)
        b["wd"].add_(1.0)
        ops.sgd_update(b["w"], b["wd"], 16, 1e-3, 0.9, 5e-4, True)

    def load(step):
        x.copy_(gpu(wl.normal(9100 + step, tuple(x.shape))))
        d_in.copy_(gpu(wl.normal(9200 + step, tuple(x.shape))))
        head_in.copy_(gpu(wl.normal(9300 + step, tuple(head_in.shape), std=2.0)))

    load(0)
    sequence({k: v.clone() for k, v in buf.items()})       # first call: the library allocates its workspace
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        sequence(buf)
    eager = {k: v.clone() for k, v in buf.items()}
    for k in ("rmean", "rvar"):
        eager[k].copy_({"rmean": rmean0, "rvar": rvar0}[k]); buf[k].copy_(eager[k])
    for k in ("su", "bu", "w", "wd"):
        eager[k].zero_(); buf[k].zero_()
    for step in range(1, 4):
        load(step)
        graph.replay()
        torch.cuda.synchronize()
        sequence(eager)                                      # eager work between the replays
        torch.cuda.synchronize()
        for k in buf:
            assert torch.equal(buf[k], eager[k]), "replay %d differs from eager in %s" % (step, k)
    assert float(buf["stats"][6]) > 0 and float(buf["norm"][0]) > 50.0


@pytest.mark.parametrize("capacity", [512, 1 << 14], ids=["one-workgroup", "sorted"])
def test_inference_postprocessing_in_a_graph_matches_eager(capacity):
    """decode -> detections of two heads into one list -> nms, captured once and replayed on new
    logits: the counter is cleared by a kernel, the record count never leaves the device."""
    import torch
    from pixienn_amd import ops
    N, K = 2, 5
    heads = [(13, [3, 4, 5]), (26, [0, 1, 2])]
    thr = 0.9 if capacity == 512 else 0.3
    dev = "cuda"
    logits = [torch.zeros((N, 3 * (K + 5), W, W), device=dev) for W, _ in heads]

    def make():
        return dict(decoded=[torch.empty_like(l) for l in logits],
                    records=torch.zeros((capacity, 8), dtype=torch.int32, device=dev),
                    count=torch.zeros(1, dtype=torch.int32, device=dev),
                    kept=torch.zeros((capacity, 8), dtype=torch.int32, device=dev),
                    kept_count=torch.zeros(1, dtype=torch.int32, device=dev),
                    ws=torch.empty(max(256, int(ops.capi.load().pxh_nms_workspace_bytes(capacity))), dtype=torch.uint8,
                                   device=dev))

    def sequence(b):
        b["count"].zero_()
        base = 0
        for (W, mask), raw, dec in zip(heads, logits, b["decoded"]):
            ops.yolo_activate(raw, dec, N, 3, K, W * W)
            ops.yolo_detections_append(dec, N, mask, wl.TINY_ANCHORS, K, W, W, 416, 416, thr, base, b["records"],
                                       b["count"], image_width=640, image_height=480)
            base += N * 3 * W * W * K
        ops.capi.call("pxh_nms", b["records"].data_ptr(), b["count"].data_ptr(), capacity, N, K, 0.45,
                      b["kept"].data_ptr(), b["kept_count"].data_ptr(), b["ws"].data_ptr(),
                      b["ws"].numel(), torch.cuda.current_stream().cuda_stream)

    def load(step):
        for i, l in enumerate(logits):
            l.copy_(gpu(wl.normal(9400 + 10 * step + i, tuple(l.shape), std=1.5)))

    def survivors(b):
        n = int(b["kept_count"].item())
        return n, b["kept"][:n].clone()

    load(0)
    static, eager = make(), make()
    sequence(eager)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        sequence(static)
    seen = set()
    for step in range(1, 4):
        load(step)
        graph.replay()
        torch.cuda.synchronize()
        sequence(eager)
        torch.cuda.synchronize()
        n_graph, kept_graph = survivors(static)
        n_eager, kept_eager = survivors(eager)
        # a list that overflows keeps whichever records came first: the case must fit
        assert 0 < int(static["count"].item()) == int(eager["count"].item()) <= capacity, (step, static["count"])
        assert 0 < n_graph == n_eager, (step, n_graph, n_eager)
        assert torch.equal(kept_graph, kept_eager), "replay %d differs from eager" % step
        seen.add(n_graph)
    assert len(seen) > 1, "the replays must have seen different data"


def test_library_workspace_keeps_handed_out_blocks_and_refuses_to_grow_under_capture():
    """The per-device workspace behind NULL-workspace calls: a larger request gives a new block but the
    earlier one stays allocated (a graph captured with its address replays into live memory); growth
    inside a capture is refused with PXH_ERR_WORKSPACE, and pxh_reserve_workspace beforehand avoids it."""
    import torch
    from pixienn_amd import capi, ops
    lib = capi.load()
    small = lib.pxh_debug_library_workspace(1 << 10)
    assert small, capi.last_error()
    assert lib.pxh_debug_library_workspace(1 << 12) == small, "a request that fits must not move the buffer"

    # a sequence captured against the current block ...
    N, C, S = 2, 8, 64
    x = gpu(wl.normal(9500, (N, C, S, S)))
    y = torch.empty_like(x); y_eager = torch.empty_like(x)
    mean, var = torch.zeros(C, device="cuda"), torch.zeros(C, device="cuda")
    scale, bias, rmean, rvar = (gpu(a) for a in wl.bn_params(9501, C))

    def forward(out):
        ops.bn_train_act_forward(x, out, mean, var, rmean.clone(), rvar.clone(), scale, bias, "leaky")

    forward(y_eager)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        forward(y)

    # ... then the workspace is outgrown: the graph still replays correctly, on memory that is still there
    big_bytes = 48 << 20
    assert lib.pxh_reserve_workspace(big_bytes) == 0, capi.last_error()
    big = lib.pxh_debug_library_workspace(big_bytes)
    assert big and big != small
    scribble = torch.full((8 << 20,), float("nan"), device="cuda")      # would land on a freed block
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(y, y_eager)
    del scribble

    # growth while capturing is refused, and the capture survives it
    huge_need = lib.pxh_nms_workspace_bytes(1 << 22)
    assert huge_need > big_bytes
    cap = 1 << 22
    rec = torch.zeros((8,), dtype=torch.int32, device="cuda")
    cnt = torch.zeros(1, dtype=torch.int32, device="cuda")
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2):
        rc = capi.call_raw("pxh_nms", rec.data_ptr(), cnt.data_ptr(), cap, 1, 1, 0.5, y.data_ptr(), cnt.data_ptr(),
                           None, 0, torch.cuda.current_stream().cuda_stream)
        y.add_(1.0)
    assert rc == -3 and "pxh_reserve_workspace" in capi.last_error(), (rc, capi.last_error())
    g2.replay()
    torch.cuda.synchronize()
    assert torch.equal(y, y_eager + 1.0)
    # a slowly rising request at least doubles the buffer, so the blocks left behind stay a fraction of it
    assert lib.pxh_reserve_workspace(huge_need) == 0, capi.last_error()
    grown = lib.pxh_debug_library_workspace(huge_need)
    assert lib.pxh_debug_library_workspace(huge_need + (1 << 20)) != grown
    assert lib.pxh_debug_library_workspace(2 * huge_need) == lib.pxh_debug_library_workspace(huge_need + (2 << 20))
