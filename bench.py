#!/usr/bin/env python3
"""Benchmark of the non-convolution layer kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

A step is one pass of the headline workload: the fused BN-inference + bias + activation
epilogue over every YOLOv3-tiny conv-output shape at batch 64, for leaky, mish and logistic
(21 launches, 2.9 GB of tensors read and as much written).  W warm-up steps, then exactly K
timed steps bracketed by device synchronisation; rank 0 prints ONE JSON line.

value      algorithmic GB/s of the timed steps (8 bytes per element: read x, write y), inputs
           resident in HBM before the timed region starts
roofline   the leaky epilogue kernel: algorithmic bytes per launch / its mean launch duration
           from HIP events recorded on the launch stream inside the timed region
extras     the other kernels of the path (max-pool, upsample, shortcut, YOLO head, BN training
           forward/backward, Adam) at the baseline's shapes, measured after the timed region
           and reported in the same line; rows under 70 % of the HBM peak carry the time of a plain
           copy of the same bytes, the largest shape of every family the CPU checker's time
noconv_ms_per_batch_yolov3_608  one YOLOv3 training step at batch 16, non-conv kernels in model order
config0_yolov3_tiny_forward_batch1  configs[0]: the tiny network's non-conv forward at batch 1, GPU and CPU
cpu_baseline  the CPU checker (a port of the reference's single-threaded CPU path) timed on a
           bounded sample of the same workload on this host, one core
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
EPILOGUE_BATCH = 64
EPILOGUE_ACTS = ["leaky", "mish", "logistic"]

# HBM bytes per launch of the leaky epilogue kernel relative to its algorithmic bytes, from two
# rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) of this script, each scaled by what the counter
# reads for the 2 x 512 MiB plain copy below (profiles/epilogue_sweep_hbm_traffic.txt)
EPILOGUE_TRAFFIC_RATIO = 0.9999


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-extras", action="store_true", help="skip the other kernels of the path")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--cpu-batch", type=int, default=64, help="images per shape in the CPU sample")
    ap.add_argument("--plain-step", action="store_true",
                    help="with --only-model-order: the step as the reference runs it only, none of the optional forms "
                         "(for a kernel trace whose shares are those of one step)")
    ap.add_argument("--only-heads", action="store_true",
                    help="run only the YOLO head rows: decode, training pass, loss form, detections (for a kernel "
                         "trace of those kernels)")
    ap.add_argument("--only-model-order", action="store_true",
                    help="run only the YOLOv3 training step in model order (for a kernel trace of that step)")
    return ap.parse_args()


class Timer:
    """Duration of a launch sequence from HIP events on the stream it runs on: the median over a few
    trials of the mean over the repetitions.

    The repetitions are recorded into one HIP graph and the graph is replayed between the two
    events: a launch through Python and ctypes costs several microseconds of host time, more than
    the small kernels of this path run, and the graph takes that out of the measurement.  If the
    capture fails the repetitions are launched eagerly."""

    def __init__(self, torch):
        self.torch = torch
        self.use_graphs = True
        self.trials = 5
        self.last_min = 0.0

    def time(self, fn, reps, warm=2, rotate=1, prepare=None):
        """fn(i) launches one repetition using buffer set i % rotate.  Returns ms per repetition.
        prepare() runs untimed before every trial (for a kernel that changes what it will do next
        time on the same data)."""
        t = self.torch
        if rotate > 1:      # every buffer set in every replay, each as often as the others
            reps = -(-reps // rotate) * rotate
        if prepare:
            prepare()
        for i in range(max(warm, rotate)):
            fn(i % rotate)
        t.cuda.synchronize()
        graph = None
        if self.use_graphs:
            try:
                graph = t.cuda.CUDAGraph()
                with t.cuda.graph(graph):
                    for i in range(reps):
                        fn(i % rotate)
                graph.replay()
                t.cuda.synchronize()
            except Exception as e:      # noqa: BLE001 - any capture problem means: measure eagerly
                log("graph capture failed (%s): timing eagerly" % e)
                graph = None
                self.use_graphs = False
                t.cuda.synchronize()
        # several trials of the whole repetition sequence: the median is reported, the minimum kept
        samples = []
        for _ in range(self.trials):
            if prepare:
                prepare()
                t.cuda.synchronize()
            start = t.cuda.Event(enable_timing=True)
            stop = t.cuda.Event(enable_timing=True)
            start.record()
            if graph is not None:
                graph.replay()
            else:
                for i in range(reps):
                    fn(i % rotate)
            stop.record()
            t.cuda.synchronize()
            samples.append(start.elapsed_time(stop) / reps)
        samples.sort()
        self.last_min = samples[0]
        return samples[len(samples) // 2]


def rotation_for(bytes_per_set, llc_bytes=256 << 20, cap=96):
    """Distinct buffer sets needed so that a set has left the 256 MB last-level cache before
    it is touched again: more than twice the cache of distinct bytes between two uses of a set.  (The
    cap only bounds the number of allocations for sets under 6 MB; no row here is that small.)"""
    n = int(llc_bytes * 2 // max(1, bytes_per_set)) + 1
    return max(1, min(cap, n))


def epilogue_workload(torch, wl):
    """Resident tensors of the headline sweep: (channels, size, x, y, params) per shape."""
    dev = torch.device("cuda:0")
    shapes = []
    gen = torch.Generator(device=dev)
    for i, (c, s) in enumerate(wl.YOLOV3_TINY_CONV_SHAPES):
        gen.manual_seed(3000 + i)
        x = torch.randn((EPILOGUE_BATCH, c, s, s), device=dev, generator=gen)
        y = torch.empty_like(x)
        scale, bias, mean, var = (torch.from_numpy(a).to(dev) for a in wl.bn_params(2000 + i, c))
        shapes.append(dict(c=c, s=s, x=x, y=y, scale=scale, bias=bias, mean=mean, var=var,
                           elems=x.numel()))
    return shapes


def fold_weights(ops, shapes):
    """What a layer does once after loading its weights: fold the per-channel constants."""
    for sh in shapes:
        sh["folded"] = ops.bn_fold(sh["mean"], sh["var"], sh["scale"], sh["bias"])


def run_epilogue_step(ops, shapes, events=None, torch=None, raw=False, bracket=None):
    """One pass of the sweep.  With `events`, one HIP-event pair brackets an activation's
    group of 7 launches (an event between two kernels would add its own few microseconds to
    every launch it brackets): every activation's, or only those named in `bracket`."""
    for act in EPILOGUE_ACTS:
        timed = events is not None and (bracket is None or act in bracket)
        if timed:
            a = torch.cuda.Event(enable_timing=True)
            b = torch.cuda.Event(enable_timing=True)
            a.record()
        for sh in shapes:
            if raw:
                ops.bn_infer_act_forward(sh["x"], sh["y"], sh["mean"], sh["var"], sh["scale"], sh["bias"], act)
            else:
                ops.bn_folded_act_forward(sh["x"], sh["y"], sh["folded"], act)
        if timed:
            b.record()
            events.append((act, a, b))


def same_bytes_copier(torch, ops, timer):
    """Returns copy_same_bytes(bytes, cap=None): the time of a plain copy (half the bytes read, half
    written, through the route kernel) of the same size, over buffers rotated as the row's are: what
    one launch of this size costs on this part whatever it computes.  Cached per size rounded to 2 %."""
    import numpy as np
    cache = {}
    dev = torch.device("cuda")

    def copy_same_bytes(bytes_, cap=None):
        n = max(1024, int(bytes_ // 8) // 256 * 256)
        key = (int(round(np.log(n) / np.log(1.02))), cap)
        if key not in cache:
            rot = rotation_for(8 * n) if cap is None else rotation_for(8 * n, cap=cap)
            src = [torch.empty((1, n), device=dev).normal_() for _ in range(rot)]
            dst = [torch.empty((1, n), device=dev) for _ in range(rot)]
            saved = timer.last_min
            cache[key] = timer.time(lambda i: ops.route_forward(src[i], dst[i], 0), 20, rotate=rot)
            timer.last_min = saved
            del src, dst
        return cache[key]

    return copy_same_bytes


def stream_mix_ms(torch, capi, timer, reads, writes, n):
    """A kernel with no arithmetic that reads `reads` and writes `writes` streams of n floats, launched as the
    library launches its streaming kernels, over buffers rotated past the cache: what that mix of reads
    and writes costs on this part whatever is computed (pxh_debug_stream_mix, a test hook)."""
    import ctypes
    n = n // 4 * 4
    rot = rotation_for(4 * n * (reads + writes))
    dev = torch.device("cuda")
    sets = []
    for _ in range(rot):
        ins = [torch.empty(n, device=dev).normal_() for _ in range(reads)]
        outs = [torch.empty(n, device=dev) for _ in range(writes)]
        pin = (ctypes.c_void_p * reads)(*[t.data_ptr() for t in ins])
        pout = (ctypes.c_void_p * writes)(*[t.data_ptr() for t in outs])
        sets.append((ins, outs, pin, pout))
    saved = timer.last_min
    ms = timer.time(lambda i: capi.call("pxh_debug_stream_mix", reads, writes, n, ctypes.addressof(sets[i][2]),
                                        ctypes.addressof(sets[i][3]), torch.cuda.current_stream().cuda_stream),
                    10, rotate=rot)
    timer.last_min = saved
    return ms


def measure_model_order(torch, ops, wl, timer, N=16, plain_only=False):
    """One training step of YOLOv3 @608 at batch N with every non-convolution kernel launched in the
    model's own layer order on tensors of their own (21 GB): forward (per layer the delta zero-fill
    of Layer::forward, then the layer), backward in reverse (per layer the gradient rescale + clip
    of Layer::backward with the thresholds of yolov3.yml, 100 and 10, then the layer), update (the
    same helpers once more on every layer's delta and on each of the 222 update buffers, then Adam
    on the 222 parameter tensors, all through tables of tensors kept on the device: one or two launches
    per operation).
    The convolutions' GEMMs are not run: a conv layer reads a resident conv result and its input
    gradient goes nowhere.  Each phase is timed as one HIP graph."""
    dev = torch.device("cuda")
    layers = wl.yolov3_layers(608)
    T = []
    for l in layers:
        shape = (N, l["c"], l["s"], l["s"])
        t = dict(y=torch.empty(shape, device=dev), d=torch.zeros(shape, device=dev))
        if l["type"] == "conv":
            t["x"] = torch.randn(shape, device=dev)
            c = l["c"]
            t["bias"] = torch.zeros(c, device=dev); t["bu"] = torch.zeros(c, device=dev)
            if l["bn"]:
                scale, bias, rmean, rvar = (torch.from_numpy(a).to(dev) for a in wl.bn_params(2000 + len(T), c))
                t.update(scale=scale, bias=bias, rmean=rmean, rvar=rvar, mean=torch.zeros(c, device=dev),
                         var=torch.zeros(c, device=dev), su=torch.zeros(c, device=dev))
        elif l["type"] == "yolo":
            t["stats"] = torch.zeros(12, device=dev); t["cost"] = torch.zeros(1, device=dev)
        T.append(t)
    truths_np, counts_np = wl.yolo_truths(5100, N)
    truths = torch.from_numpy(truths_np).to(dev); counts = torch.from_numpy(counts_np).to(dev)
    # the parameters as the engine holds them: 222 tensors (weights, biases, scales per convolution), here as
    # 256-byte aligned views into one buffer per kind
    sizes = wl.yolov3_parameter_tensors(608)
    starts, at = [], 0
    for n_, _ in sizes:
        starts.append(at); at += (n_ + 63) // 64 * 64
    w = 0.02 * torch.randn(at, device=dev); g = 1e-3 * torch.randn(at, device=dev)
    m = torch.zeros(at, device=dev); v = torch.zeros(at, device=dev)
    views = lambda flat: [flat[o:o + n_] for o, (n_, _) in zip(starts, sizes)]
    pw, pg, pm, pv = views(w), views(g), views(m), views(v)
    decayed = [d_ for _, d_ in sizes]
    launches = dict(forward=0, backward=0, update=0)

    def absorbed(i):            # an upsample writes into (and reads its delta from) the route that follows
        return layers[i]["type"] == "upsample"

    # deltas that a shortcut is the first to write in the backward pass (the layer in front of it and
    # its `from` layer): with pxh_shortcut_backward_first they are overwritten, not cleared and added to
    overwritten = set()
    for i, l in enumerate(layers):
        if l["type"] == "shortcut":
            overwritten.update((i - 1, l["frm"]))

    # convolutions whose output only the shortcut behind them reads (every residual block of YOLOv3): the
    # shortcut can ride on the convolution's epilogue (pxh_bn_train_act_shortcut_forward), and in the backward
    # pass the convolution works on the shortcut's delta itself (alpha = 1: the two are the same values)
    read_elsewhere = set()
    for i, l in enumerate(layers):
        if l["type"] == "shortcut":
            read_elsewhere.add(l["frm"])
        elif l["type"] == "route":
            read_elsewhere.update(l["sources"])
    rides = {i - 1: i for i, l in enumerate(layers)
             if l["type"] == "shortcut" and layers[i - 1]["type"] == "conv" and layers[i - 1]["bn"]
             and (i - 1) not in read_elsewhere}

    head_table = ops.yolo_head_table([dict(input=T[i - 1]["y"], output=T[i]["y"], delta=T[i]["d"], masks=l["mask"],
                                           width=l["s"], height=l["s"], stats=T[i]["stats"], cost=T[i]["cost"],
                                           ignore_thresh=0.7, truth_thresh=1.0)
                                      for i, l in enumerate(layers) if l["type"] == "yolo"])

    def forward(_, first_writer=False, fills_together=False, heads_apart=False, shortcut_rides=False):
        n = 0
        # (a head's delta is not cleared either: the training pass writes every element of it)
        cleared = [t["d"] for i, t in enumerate(T) if not absorbed(i) and layers[i]["type"] != "yolo"
                   and not (first_writer and i in overwritten)]
        if fills_together:      # the deltas of all layers cleared at the start of the pass, in a few launches
            ops.fill_multi(cleared, 0.0)
        n += len(cleared)
        for i, (l, t) in enumerate(zip(layers, T)):
            if not fills_together and not absorbed(i) and l["type"] != "yolo" and not (first_writer and i in overwritten):
                ops.fill(t["d"], 0.0)
            kind = l["type"]
            if shortcut_rides and kind == "conv" and i in rides:
                sc = rides[i]
                ops.bn_train_act_shortcut_forward(t["x"], T[sc]["y"], t["mean"], t["var"], t["rmean"], t["rvar"],
                                                  t["scale"], t["bias"], "leaky", T[layers[sc]["frm"]]["y"])
            elif shortcut_rides and kind == "shortcut" and i - 1 in rides:
                n -= 1
            elif kind == "conv" and l["bn"]:
                ops.bn_train_act_forward(t["x"], t["y"], t["mean"], t["var"], t["rmean"], t["rvar"], t["scale"],
                                         t["bias"], "leaky")
            elif kind == "conv":
                ops.bias_act_forward(t["x"], t["y"], t["bias"], "linear")
            elif kind == "shortcut":
                ops.shortcut_forward(T[i - 1]["y"], T[l["frm"]]["y"], t["y"], "linear")
            elif kind == "upsample":
                ops.upsample_forward_into(T[i - 1]["y"], T[i + 1]["y"], 0, 2, 1.0)
            elif kind == "route" and len(l["sources"]) == 1:
                ops.route_forward(T[l["sources"][0]]["y"], t["y"], 0)
            elif kind == "route":
                up, other = l["sources"]
                ops.route_forward(T[other]["y"], t["y"], layers[up]["c"] * l["s"] * l["s"])
            elif kind == "yolo" and heads_apart:
                ops.yolo_forward_train(T[i - 1]["y"], t["y"], t["d"], truths, counts, truths.shape[1], l["mask"],
                                       wl.YOLOV3_ANCHORS, t["stats"], t["cost"], N, 80, l["s"], l["s"], 608, 608,
                                       0.7, 1.0, 1.0, 1.0, 1.0, 1.0)
            n += 1
        if not heads_apart:
            # nothing reads a head's delta or cost before backward: the heads wait for the last one and
            # run as one pass (pxh_yolo_forward_train_heads)
            ops.yolo_forward_train_heads(None, truths, counts, truths.shape[1], wl.YOLOV3_ANCHORS, N, 80, 608, 608,
                                         table=head_table[0])
            n -= len(head_table[0]) - 1
        launches["forward"] = n

    # deltas whose last writer before their layer's backward is a shortcut or a YOLO head (the layer in
    # front of each: nothing else reads its output): that kernel can leave the norm and the peak behind
    # (pxh_shortcut_backward_norm, pxh_axpy_norm) and the rescale + clip of that delta need not read it
    groups = {i - 1: ops.norm_groups_like(T[i - 1]["d"]) for i, l in enumerate(layers)
              if l["type"] in ("shortcut", "yolo")}

    def backward(_, first_writer=False, norm_from_writer=False, two_calls=False, shortcut_rides=False,
                 shortcut_clipped=False):
        n = 0
        for i in reversed(range(len(layers))):
            l, t = layers[i], T[i]
            kind = l["type"]
            if shortcut_rides and kind == "shortcut" and i - 1 in rides:
                # the shortcut's own rescale + clip, its delta to the `from` layer (first writer), and
                # nothing to the convolution in front, which takes this delta as its own
                if shortcut_clipped:        # ... as one call that reads the delta once
                    ops.shortcut_backward_clipped(t["d"], T[l["frm"]]["d"], None, "linear", first=True, threshold=100.0,
                                                  clip=10.0)
                    n += 1
                    continue
                ops.rescale_clip(t["d"], 100.0, 10.0)
                ops.shortcut_backward_first(t["d"], T[l["frm"]]["d"], None, "linear")
                n += 2
                continue
            if shortcut_clipped and kind == "shortcut" and first_writer and not norm_from_writer:
                ops.shortcut_backward_clipped(t["d"], T[l["frm"]]["d"], T[i - 1]["d"], "linear", first=True,
                                              threshold=100.0, clip=10.0)
                n += 1
                continue
            if shortcut_rides and kind == "conv" and i in rides:
                ops.bn_act_backward_clipped(T[rides[i]]["d"], t["x"], t["mean"], t["var"], t["scale"], t["bias"],
                                            t["su"], t["bu"], "leaky", 100.0, 10.0)
                n += 1
                continue
            # a convolution's rescale + clip rides on its epilogue's backward (pxh_*_backward_clipped) unless
            # the kernel that wrote its delta last left the norm behind; `two_calls`: as two calls, for comparison
            fused = kind == "conv" and not two_calls and not (norm_from_writer and i in groups)
            if not absorbed(i) and not fused:
                if norm_from_writer and i in groups:
                    ops.rescale_clip_from_groups(t["d"], groups[i], 100.0, 10.0)
                else:
                    ops.rescale_clip(t["d"], 100.0, 10.0)
                n += 1
            if kind == "yolo" and norm_from_writer:
                ops.axpy_norm(1.0, t["d"], T[i - 1]["d"], groups[i - 1])
            elif kind == "shortcut" and norm_from_writer:
                ops.shortcut_backward_norm(t["d"], T[l["frm"]]["d"], T[i - 1]["d"], groups[i - 1], "linear",
                                           first=first_writer)
            elif kind == "yolo":
                ops.axpy(1.0, t["d"], T[i - 1]["d"])
            elif kind == "conv" and l["bn"] and fused:
                ops.bn_act_backward_clipped(t["d"], t["x"], t["mean"], t["var"], t["scale"], t["bias"], t["su"],
                                            t["bu"], "leaky", 100.0, 10.0)
            elif kind == "conv" and l["bn"]:
                ops.bn_act_backward(t["d"], t["x"], t["mean"], t["var"], t["scale"], t["bias"], t["su"], t["bu"],
                                    "leaky")
            elif kind == "conv" and fused:
                ops.bias_act_backward_clipped(t["d"], None, t["bu"], "linear", 100.0, 10.0)
            elif kind == "conv":
                ops.bias_act_backward(t["d"], None, t["bu"], "linear")
            elif kind == "shortcut" and first_writer:
                ops.shortcut_backward_first(t["d"], T[l["frm"]]["d"], T[i - 1]["d"], "linear")
            elif kind == "shortcut":
                ops.shortcut_backward(t["d"], T[l["frm"]]["d"], T[i - 1]["d"], "linear")
            elif kind == "upsample":
                ops.upsample_backward_from(T[i + 1]["d"], 0, T[i - 1]["d"], 2, 1.0)
            elif kind == "route" and len(l["sources"]) == 1:
                ops.route_backward(t["d"], T[l["sources"][0]]["d"], 0)
            elif kind == "route":
                up, other = l["sources"]
                ops.route_backward(t["d"], T[other]["d"], layers[up]["c"] * l["s"] * l["s"])
            n += 1
        launches["backward"] = n

    # the tensors of update(), as tables kept on the device (what ParameterSet builds once)
    delta_table = ops.TensorTable([[t["d"] for i, t in enumerate(T) if not absorbed(i)]])
    hook_table = ops.TensorTable([pg])
    adam_table = ops.TensorTable([pw, pg, pm, pv], decayed)

    def update(_, touch_delta=True):
        n = 0
        if touch_delta:         # the reference's update() passes every delta through the helpers once more
            delta_table.rescale_clip(100.0, 10.0); n += delta_table.count
        # the hooks on every update buffer, each with its own norm, then Adam: one launch each for all tensors
        hook_table.rescale_clip(100.0, 10.0)
        adam_table.adam_update(N, 1, 1e-3, decay=5e-4)
        launches["update"] = n + 2

    out = {}
    for name, fn in (("forward", forward), ("backward", backward), ("update", update)):
        out[name + "_ms"] = round(timer.time(fn, 3, warm=1), 3)
    out["total_ms"] = round(out["forward_ms"] + out["backward_ms"] + out["update_ms"], 3)
    # nothing reads a delta after backward: the pass over them in update() is dead work that a host
    # may drop (Context::helpersTouchDeltaInUpdate of the C++ layer interface)
    out["calls"] = dict(launches)
    if plain_only:
        del T, w, g, m, v
        torch.cuda.empty_cache()
        return out
    # the same backward with every convolution's rescale + clip as a call of its own in front of the
    # epilogue's backward (pxh_rescale_clip, then pxh_bn_act_backward): what the fused call saves
    out["backward_rescale_clip_as_its_own_call_ms"] = round(timer.time(lambda i: backward(i, two_calls=True), 3, warm=1), 3)
    out["update_without_delta_pass_ms"] = round(timer.time(lambda i: update(i, False), 3, warm=1), 3)
    # the 23 shortcuts as first writers of the 46 deltas they reach first: no zero-fill of those,
    # no read of them in the shortcut's backward (an option of the C++ layer interface, "first_writer")
    # every head where it sits in the graph, one call each: what the single pass over all heads saves
    out["forward_heads_one_call_each_ms"] = round(timer.time(lambda i: forward(i, heads_apart=True), 3, warm=1), 3)
    out["forward_fills_together_ms"] = round(timer.time(lambda i: forward(i, False, True), 3, warm=1), 3)
    out["forward_first_writer_ms"] = round(timer.time(lambda i: forward(i, True, True), 3, warm=1), 3)
    # (a first-writer shortcut's targets are plain functions of its delta: the rescale + clip that opens its backward
    # and the backward itself run as one call that reads the delta once, pxh_shortcut_backward_clipped;
    # `..._shortcut_helpers_apart_ms`: as the two calls, for comparison)
    out["backward_first_writer_ms"] = round(timer.time(lambda i: backward(i, True, shortcut_clipped=True), 3, warm=1), 3)
    out["backward_first_writer_shortcut_helpers_apart_ms"] = round(timer.time(lambda i: backward(i, True), 3, warm=1), 3)
    # the 23 shortcuts and 3 heads leave the norm and peak of the delta they write last: 26 deltas are not
    # read for their norm ("leaves_norm" of the C++ layer interface); same values to the bit
    out["backward_norm_from_writer_ms"] = round(timer.time(lambda i: backward(i, False, True), 3, warm=1), 3)
    out["backward_first_writer_norm_from_writer_ms"] = round(timer.time(lambda i: backward(i, True, True), 3, warm=1), 3)
    out["deltas_with_norm_from_writer"] = len(groups)
    # the shortcut of a residual block on the epilogue of the convolution in front of it (first-writer forms
    # everywhere else): no pass of its own forward, and backward the convolution takes the shortcut's delta
    out["forward_shortcut_in_epilogue_ms"] = round(timer.time(lambda i: forward(i, True, True, shortcut_rides=True), 3, warm=1), 3)
    out["backward_shortcut_in_epilogue_ms"] = round(timer.time(
        lambda i: backward(i, True, shortcut_rides=True, shortcut_clipped=True), 3, warm=1), 3)
    out["backward_shortcut_in_epilogue_shortcut_helpers_apart_ms"] = round(timer.time(
        lambda i: backward(i, True, shortcut_rides=True), 3, warm=1), 3)
    out["shortcuts_in_epilogue"] = len(rides)
    # the leanest step: no dead pass in update(), and whichever of the lean forward and backward forms is
    # faster here (since the rescale + clip rides on the convolutions' own backward, leaving the norm with
    # the writer no longer pays for them)
    lean_forward = min(("forward_first_writer_ms", "forward_shortcut_in_epilogue_ms"), key=lambda k: out[k])
    lean_backward = min(("backward_first_writer_ms", "backward_first_writer_norm_from_writer_ms",
                         "backward_shortcut_in_epilogue_ms"), key=lambda k: out[k])
    out["leanest_forward"] = lean_forward
    out["leanest_backward"] = lean_backward
    out["leanest_total_ms"] = round(out[lean_forward] + out[lean_backward] + out["update_without_delta_pass_ms"], 3)
    out["elements_per_tensor_kind"] = int(sum(N * l["c"] * l["s"] * l["s"] for l in layers))
    del T, w, g, m, v
    torch.cuda.empty_cache()
    return out


def measure_extras(torch, ops, wl, timer, capi, cpu=None, only_heads=False):
    """The other kernels of the path at the baseline's shapes.  Returns (rows, ms_per_batch).  `cpu`:
    cpu_rows(), attached to the rows it has a figure for."""
    import numpy as np
    dev = torch.device("cuda:0")
    rows = []

    copy_same_bytes = same_bytes_copier(torch, ops, timer)

    def add(name, shape, bytes_, ms, note="", streaming=True, cache_warm=False):
        gbs = bytes_ / (ms * 1e-3) / 1e9
        row = dict(kernel=name, shape=shape, MB=round(bytes_ / 1e6, 1), ms=round(ms, 4),
                   ms_min=round(timer.last_min, 4), GBps=round(gbs, 1), frac=round(gbs / HBM_PEAK_GBS, 3), note=note)
        if cache_warm:      # timed on one buffer that stays in the last-level cache: not an HBM figure
            row["cache_warm"] = True
        # below the 70 % bar: how long a plain copy of the same bytes takes, i.e. how much of the gap is
        # the cost of a launch of that size (vs_copy = copy time / this row's time; 1 = as fast as a copy)
        if streaming and row["frac"] < 0.70 and bytes_ <= (1 << 30):
            c_ms = copy_same_bytes(bytes_)
            row["copy_same_bytes_ms"] = round(c_ms, 4)
            row["vs_copy"] = round(c_ms / ms, 3)
        rows.append(row)
        return ms

    def randn(*shape):
        return torch.randn(shape, device=dev)

    N = 16
    if not only_heads:      # (the sections in front of the heads)
        # ---- route concat of YOLOv3 @608: 256x38^2 (upsampled) ++ 512x38^2, and 128x76^2 ++ 256x76^2.
        # The upsample in front writes its channels straight into the concat buffer (timed below, same
        # bytes as the dense form), so the route moves the other source only.
        for (c1, c2, s) in [(256, 512, 38), (128, 256, 76)]:
            e = N * c2 * s * s
            e_up = N * c1 * s * s
            rot = rotation_for(5 * e_up)      # the smallest of the three launches sets the number of buffer sets
            bs = [randn(N, c2, s, s) for _ in range(rot)]
            rs = [torch.empty((N, c1 + c2, s, s), device=dev) for _ in range(rot)]
            ms = timer.time(lambda i: ops.route_forward(bs[i], rs[i], c1 * s * s), 20, rotate=rot)
            add("route_fwd", "%dx(%d+)%dx%d^2" % (N, c1, c2, s), 8 * e, ms, "the %d-channel source, 8B/elem" % c2)
            ms = timer.time(lambda i: ops.route_backward(rs[i], bs[i], c1 * s * s), 20, rotate=rot)
            add("route_bwd", "%dx(%d+)%dx%d^2" % (N, c1, c2, s), 12 * e, ms, "the %d-channel source, 12B/elem" % c2)
            xs = [randn(N, c1, s // 2, s // 2) for _ in range(rot)]
            ms = timer.time(lambda i: ops.upsample_forward_into(xs[i], rs[i], 0, 2, 1.0), 20, rotate=rot)
            add("upsample_fwd(into route)", "%dx%dx%d^2" % (N, c1, s // 2), 5 * e_up, ms, "same bytes as upsample_fwd; "
                "not in ms/batch twice")
            del bs, rs, xs
        # ---- max-pool 2x2 s2 forward + backward (config 2)
        for c, s in wl.YOLOV3_MAXPOOL_SHAPES:
            e_in = N * c * s * s
            e_out = e_in // 4
            rot = rotation_for(4 * e_in + 8 * e_out)
            xs = [randn(N, c, s, s) for _ in range(rot)]
            outs = [torch.empty((N, c, s // 2, s // 2), device=dev) for _ in range(rot)]
            idxs = [torch.empty((N, c, s // 2, s // 2), device=dev, dtype=torch.int32) for _ in range(rot)]
            ms = timer.time(lambda i: ops.maxpool_forward(xs[i], outs[i], idxs[i], 2, 2, 1), 20, rotate=rot)
            add("maxpool_fwd", "%dx%dx%d^2" % (N, c, s), 4 * e_in + 8 * e_out, ms, "4B/in + 8B/out")
            deltas = [randn(N, c, s // 2, s // 2) for _ in range(rot)]
            ms = timer.time(lambda i: ops.maxpool_backward(deltas[i], idxs[i], xs[i], 2, 2, 1), 20, rotate=rot)
            add("maxpool_bwd", "%dx%dx%d^2" % (N, c, s), 8 * e_out + 8 * e_in, ms, "full-grad RMW: 8B/out + 8B/in")
            del xs, outs, idxs, deltas
        # ---- the inference epilogue with the 2x2 / 2 pool behind it in one pass (YOLOv3-tiny, batch 64: the
        # headline sweep's own shapes that a pool follows), against the two calls one after the other
        scale_t, bias_t, rmean_t, rvar_t = (torch.from_numpy(a_).to(dev) for a_ in wl.bn_params(2900, 1024))
        for c, s in ((16, 416), (32, 208), (64, 104), (128, 52), (256, 26)):
            n64 = 64
            e_in = n64 * c * s * s
            rot = rotation_for(5 * e_in)
            xs = [randn(n64, c, s, s) for _ in range(rot)]
            ys = [torch.empty((n64, c, s, s), device=dev) for _ in range(min(rot, 3))]
            outs = [torch.empty((n64, c, s // 2, s // 2), device=dev) for _ in range(rot)]
            idxs = [torch.empty((n64, c, s // 2, s // 2), device=dev, dtype=torch.int32) for _ in range(min(rot, 3))]
            folded = ops.bn_fold(rmean_t[:c].contiguous(), rvar_t[:c].contiguous(), scale_t[:c].contiguous(),
                                 bias_t[:c].contiguous())
            ms = timer.time(lambda i: ops.bn_folded_act_maxpool_forward(xs[i], outs[i], folded, "leaky"), 20, rotate=rot)

            def two(i):
                ops.bn_folded_act_forward(xs[i], ys[i % len(ys)], folded, "leaky")
                ops.maxpool_forward(ys[i % len(ys)], outs[i], idxs[i % len(idxs)], 2, 2, 1)

            ms_two = timer.time(two, 20, rotate=rot)
            add("epilogue+maxpool(leaky, inference)", "%dx%dx%d^2" % (n64, c, s), 5 * e_in, ms,
                "4B/in + 1B/in out; the two calls (8B + 6B per input element) %.4f ms" % ms_two)
            rows[-1]["two_calls_ms"] = round(ms_two, 4)
            del xs, ys, outs, idxs
        # ---- upsample x2 forward + backward
        for c, s in wl.YOLOV3_UPSAMPLE_SHAPES:
            e_in = N * c * s * s
            e_out = 4 * e_in
            rot = rotation_for(4 * e_in + 4 * e_out)
            xs = [randn(N, c, s, s) for _ in range(rot)]
            outs = [torch.empty((N, c, 2 * s, 2 * s), device=dev) for _ in range(rot)]
            ms_f = timer.time(lambda i: ops.upsample_forward(xs[i], outs[i], 2, 1.0), 50, rotate=rot)
            add("upsample_fwd", "%dx%dx%d^2" % (N, c, s), 4 * e_in + 4 * e_out, ms_f, "4B/in + 4B/out")
            ms_b = timer.time(lambda i: ops.upsample_backward(outs[i], xs[i], 2, 1.0), 50, rotate=rot)
            add("upsample_bwd", "%dx%dx%d^2" % (N, c, s), 4 * e_out + 8 * e_in, ms_b, "4B/out + 8B/in")
            del xs, outs
        # ---- shortcut forward + backward
        shortcut_ms = {}
        for c, s, count in wl.YOLOV3_SHORTCUT_SHAPES:
            e = N * c * s * s
            rot = rotation_for(12 * e)
            a = [randn(N, c, s, s) for _ in range(rot)]
            b = [randn(N, c, s, s) for _ in range(rot)]
            o = [torch.empty((N, c, s, s), device=dev) for _ in range(rot)]
            ms_f = timer.time(lambda i: ops.shortcut_forward(a[i], b[i], o[i], "linear"), 20, rotate=rot)
            add("shortcut_fwd", "%dx%dx%d^2" % (N, c, s), 12 * e, ms_f, "12B/elem")
            ms_b = timer.time(lambda i: ops.shortcut_backward(o[i], a[i], b[i], "linear"), 20, rotate=rot)
            add("shortcut_bwd", "%dx%dx%d^2" % (N, c, s), 20 * e, ms_b, "20B/elem")
            # the same on the same buffers, also leaving the norm and peak of what it wrote to grad
            groups = [ops.norm_groups_like(b[0]) for _ in range(rot)]
            ms_n = timer.time(lambda i: ops.shortcut_backward_norm(o[i], a[i], b[i], groups[i], "linear"), 20, rotate=rot)
            add("shortcut_bwd+norm", "%dx%dx%d^2" % (N, c, s), 20 * e, ms_n, "20B/elem + 8B per 256 values of grad")
            del groups
            # a first writer with Layer::backward's rescale + clip in front, as one call (the delta read once when
            # nothing changes: thresholds far away) and as the two calls it stands for
            ms_c = timer.time(lambda i: ops.shortcut_backward_clipped(o[i], a[i], b[i], "linear", first=True,
                                                                      threshold=1e9, clip=1e9), 20, rotate=rot)
            def two_calls(i):
                ops.rescale_clip(o[i], 1e9, 1e9)
                ops.shortcut_backward_first(o[i], a[i], b[i], "linear")
            ms_2 = timer.time(two_calls, 20, rotate=rot)
            add("shortcut_bwd_first+clip", "%dx%dx%d^2" % (N, c, s), 12 * e, ms_c,
                "rescale + clip of the delta, then the first writer's backward: 12B/elem; as two calls (16B/elem) %.4f ms"
                % ms_2)
            shortcut_ms[(c, s)] = (ms_f, ms_b, count)
            del a, b, o
        # ---- the delta zero-fill of Layer::forward (include/Layer.h:377-383): write-only, 4 B per element
        for c, s in [(32, 608), (256, 76), (1024, 19)]:
            e = N * c * s * s
            rot = rotation_for(4 * e)
            ds_ = [torch.empty((N, c, s, s), device=dev) for _ in range(rot)]
            ms = timer.time(lambda i: ops.fill(ds_[i], 0.0), 20, rotate=rot)
            add("fill(delta = 0)", "%dx%dx%d^2" % (N, c, s), 4 * e, ms, "4B/elem written")
            del ds_
    # ---- YOLO head (config 3): batch 64, and batch 16 for the training step's own heads
    stats = torch.zeros(12, device=dev)
    cost = torch.zeros(1, device=dev)
    head_ms = {}
    for NB, s in [(64, s_) for s_ in wl.YOLOV3_HEAD_SIZES] + [(N, s_) for s_ in wl.YOLOV3_HEAD_SIZES]:
        truths_np, counts_np = wl.yolo_truths(5100, NB)
        truths = torch.from_numpy(truths_np).to(dev)
        counts = torch.from_numpy(counts_np).to(dev)
        e = NB * 255 * s * s
        rot = rotation_for(4 * e)        # the loss form touches little more than one of a set's three tensors
        xin = [2.0 * randn(NB, 255, s, s) for _ in range(rot)]
        out = [torch.empty((NB, 255, s, s), device=dev) for _ in range(rot)]
        dl = [torch.empty((NB, 255, s, s), device=dev) for _ in range(rot)]
        ms_d = timer.time(lambda i: ops.yolo_activate(xin[i], out[i], NB, 3, 80, s * s), 20, rotate=rot)
        add("yolo_decode", "%dx255x%d^2" % (NB, s), 8 * e, ms_d, "8B/elem")
        ms_t = timer.time(lambda i: ops.yolo_forward_train(
            xin[i], out[i], dl[i], truths, counts, truths.shape[1], wl.YOLOV3_MASKS[s], wl.YOLOV3_ANCHORS, stats,
            cost, NB, 80, s, s, 608, 608, 0.7, 1.0, 1.0, 2.0, 0.1, 1.0), 20, rotate=rot)
        add("yolo_decode+delta+cost", "%dx255x%d^2" % (NB, s), 12 * e, ms_t, "fused 12B/elem")
        head_ms[(NB, s)] = (ms_d, ms_t)
        # the reference's own split: loss from the decoded head with host-assigned positives
        acls, aanc, abox = wl.yolo_assign_targets(truths_np, counts_np, wl.YOLOV3_MASKS[s], wl.YOLOV3_ANCHORS, s, s,
                                                  608, 608)
        tabs = [torch.from_numpy(t).to(dev) for t in (acls, aanc, abox)]
        gmasks = torch.tensor(wl.YOLOV3_MASKS[s], device=dev, dtype=torch.int32)
        ganch = torch.tensor(wl.YOLOV3_ANCHORS, device=dev, dtype=torch.float32)
        ms_l = timer.time(lambda i: ops.yolo_loss(out[i], dl[i], truths, counts, truths.shape[1], tabs[0], tabs[1],
                                                  tabs[2], gmasks, ganch, stats, cost, NB, 9, 80, s, s, 608, 608,
                                                  0.7, 1.0, 1.0, 2.0, 0.1, 1.0), 20, rotate=rot)
        add("yolo_delta+cost", "%dx255x%d^2" % (NB, s), (4 + 4 * 5 / 85) * e, ms_l, "decoded input, 4.24B/elem")
        if s == 76 and NB == 64:
            # detections of the decoded head at a confidence threshold of 0.5: the objectness row of every
            # slot, the box and class rows of the slots that pass (about half of them on these logits)
            cap = 1 << 22
            rec = torch.empty((cap, 8), device=dev, dtype=torch.int32)
            cnt = torch.zeros(1, device=dev, dtype=torch.int32)
            m = np.ascontiguousarray(wl.YOLOV3_MASKS[s], dtype=np.int32)
            a = np.ascontiguousarray(wl.YOLOV3_ANCHORS, dtype=np.int32)

            # ... and at 0.998, where about one slot in a thousand passes, as on a trained network's
            # output: the objectness row is nearly all that is read
            slots = NB * 3 * s * s
            for thr, label in [(0.5, ".5"), (0.998, ".998")]:
                def detect(i, thr=thr):
                    capi.call("pxh_yolo_detections", out[i].data_ptr(), NB, m.ctypes.data, len(m), a.ctypes.data,
                              len(a) // 2, 80, s, s, 608, 608, 0, 0, thr, rec.data_ptr(), cap, cnt.data_ptr(),
                              torch.cuda.current_stream().cuda_stream)

                ms_det = timer.time(detect, 10, rotate=rot)
                found = int(cnt.item())
                passing = float((out[0].view(NB, 3, 85, s * s)[:, :, 4] >= thr).float().mean())
                add("yolo_detections(thr %s)" % label, "%dx255x%d^2" % (NB, s),
                    4 * slots * (1 + passing * 84) + 32 * min(found, cap), ms_det,
                    "%d records; %.2g%% of the slots pass" % (found, 100 * passing), streaming=False)
            del rec
        del xin, out, dl
    # ---- the three heads of the model in one pass (pxh_yolo_forward_train_heads): the small heads' chains of
    # dependent steps run under the class rows of the large one
    for NB in (64, N):
        truths_np, counts_np = wl.yolo_truths(5100, NB)
        truths = torch.from_numpy(truths_np).to(dev)
        counts = torch.from_numpy(counts_np).to(dev)
        e_all = sum(NB * 255 * s * s for s in wl.YOLOV3_HEAD_SIZES)
        rot = rotation_for(12 * e_all)
        sets = []
        for _ in range(rot):
            heads = [dict(input=2.0 * randn(NB, 255, s, s), output=torch.empty((NB, 255, s, s), device=dev),
                          delta=torch.empty((NB, 255, s, s), device=dev), masks=wl.YOLOV3_MASKS[s], width=s, height=s,
                          stats=torch.zeros(12, device=dev), cost=torch.zeros(1, device=dev), ignore_thresh=0.7,
                          truth_thresh=1.0, coord_scale=1.0, object_scale=2.0, noobject_scale=0.1, class_scale=1.0)
                     for s in wl.YOLOV3_HEAD_SIZES]
            sets.append((heads, ops.yolo_head_table(heads)))
        ms_h = timer.time(lambda i: ops.yolo_forward_train_heads(None, truths, counts, truths.shape[1], wl.YOLOV3_ANCHORS,
                                                                 NB, 80, 608, 608, table=sets[i][1][0]), 20, rotate=rot)
        separately = sum(head_ms[(NB, s)][1] for s in wl.YOLOV3_HEAD_SIZES)
        add("yolo_decode+delta+cost x3", "%dx255x{19,38,76}^2" % NB, 12 * e_all, ms_h,
            "the three heads in one pass, 12B/elem; one call per head: %.4f ms" % separately)
        # the pass reads one stream and writes two: the same mix without any arithmetic, same bytes
        mix_ms = stream_mix_ms(torch, capi, timer, 1, 2, e_all)
        rows[-1]["copy_same_mix_ms"] = round(mix_ms, 4)
        rows[-1]["vs_same_mix"] = round(mix_ms / ms_h, 3)
        head_ms[(NB, "all")] = (0.0, ms_h)
        del sets
    if only_heads:
        return rows, 0.0
    # ---- non-maximum suppression of device-resident records: an inference-sized list (one image, one
    # launch) and a validation-sized one (64 images, low confidence threshold).  Not a streaming kernel:
    # the time is comparisons between records, the bytes column is just the records read and written.
    for n_rec, images, clusters, cap in [(100, 1, 6, 512), (100000, 64, 8, 1 << 17)]:
        recs_np = wl.detection_clusters(7, n_rec, images, 80, clusters)
        recs = torch.zeros((cap, 8), dtype=torch.int32, device=dev)
        recs[:n_rec] = torch.from_numpy(recs_np.view(np.int32).reshape(-1, 8)).to(dev)
        cnt = torch.tensor([n_rec], dtype=torch.int32, device=dev)
        kept = torch.empty_like(recs)
        kept_cnt = torch.zeros(1, dtype=torch.int32, device=dev)
        ws_bytes = int(capi.load().pxh_nms_workspace_bytes(cap))
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)

        def suppress(i):
            capi.call("pxh_nms", recs.data_ptr(), cnt.data_ptr(), cap, images, 80, 0.45, kept.data_ptr(),
                      kept_cnt.data_ptr(), ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream)

        ms = timer.time(suppress, 10)
        add("nms(thr .45)", "%d records, %d image%s" % (n_rec, images, "s" if images > 1 else ""), 64 * n_rec, ms,
            "%d kept; not bandwidth bound" % int(kept_cnt.item()), streaming=False)
        del recs, kept, ws
    # ---- BN training forward / backward (config 4): batch 16 @608, 13 shapes
    bn_ms = {}
    for (c, s), count in zip(wl.YOLOV3_BN_SHAPES, wl.YOLOV3_BN_COUNTS):
        e = N * c * s * s
        rot = rotation_for(8 * e)        # the forward touches 8 of a set's 12 bytes per element
        x = [randn(N, c, s, s) for _ in range(rot)]
        y = [torch.empty((N, c, s, s), device=dev) for _ in range(rot)]
        d = [randn(N, c, s, s) for _ in range(rot)]
        scale, bias, rmean, rvar = (torch.from_numpy(a).to(dev) for a in wl.bn_params(2000 + c, c))
        mean = torch.zeros(c, device=dev); var = torch.ones(c, device=dev)
        su = torch.zeros(c, device=dev); bu = torch.zeros(c, device=dev)
        ms_f = timer.time(lambda i: ops.bn_train_act_forward(x[i], y[i], mean, var, rmean, rvar, scale, bias, "leaky"),
                          10, rotate=rot)
        # shapes whose channel slice fits one workgroup (and with 96 channels or more) run as ONE launch that
        # reads x once: their rows count the bytes that launch moves (8 / 16 B per element), not the 12 / 20 of
        # the three-launch form
        vec = (s * s) % 4 == 0
        vectors = -(-N * s * s // (4 if vec else 1))
        per_thread = -(-vectors // 1024)
        one_launch = c >= 96 and (per_thread <= 8 or (vec and per_thread <= 24))
        add("bn_train_fwd(leaky)", "%dx%dx%d^2" % (N, c, s), (8 if one_launch else 12) * e, ms_f,
            "one launch: x read once, 8B per elem (three launches move 12)" if one_launch
            else "stats 4B + apply 8B per elem; x kept")
        if (c, s) in [(sc, ss) for sc, ss, _ in wl.YOLOV3_SHORTCUT_SHAPES]:
            # the residual block's shortcut in the same pass: one more stream read (the block's input, here `d`),
            # against this row + the shortcut's own 12 B/elem pass
            ms_s = timer.time(lambda i: ops.bn_train_act_shortcut_forward(x[i], y[i], mean, var, rmean, rvar, scale,
                                                                          bias, "leaky", d[i]), 10, rotate=rot)
            add("bn_train_fwd+shortcut(leaky)", "%dx%dx%d^2" % (N, c, s), (12 if one_launch else 16) * e, ms_s,
                "y = act(bn(x)) + from in the layer's own pass; the layer alone %.4f ms, then a shortcut of 12B/elem" % ms_f)
        ms_b = timer.time(lambda i: ops.bn_act_backward(d[i], x[i], mean, var, scale, bias, su, bu, "leaky"),
                          10, rotate=rot)
        add("bn_bwd(leaky)", "%dx%dx%d^2" % (N, c, s), (16 if one_launch else 20) * e, ms_b,
            "one launch: delta once, x twice, 16B per elem (three launches move 20)" if one_launch
            else "sums 8B + dx 12B per elem; pre recomputed")
        # the same with Layer::backward's rescale + clip riding on it (thresholds far away: nothing changes,
        # as in the model-order step); same bytes as the plain backward, against backward + a 4 B/elem norm read
        ms_c = timer.time(lambda i: ops.bn_act_backward_clipped(d[i], x[i], mean, var, scale, bias, su, bu, "leaky",
                                                                1e30, 1e30), 10, rotate=rot)
        add("bn_bwd_clipped(leaky)", "%dx%dx%d^2" % (N, c, s), (16 if one_launch else 20) * e, ms_c,
            "rescale + clip decided in the backward's own first pass; plain backward %.4f ms" % ms_b)
        if (c, s) in ((64, 304), (256, 76)):
            # ... and when the norm is beyond the threshold (every call rescales; the clamp is far away): the sums
            # of the first pass still serve, multiplied by the factor; the one-launch form rewrites dx once more
            ms_r = timer.time(lambda i: ops.bn_act_backward_clipped(d[i], x[i], mean, var, scale, bias, su, bu, "leaky",
                                                                    1e-6, 1e30), 10, rotate=rot)
            add("bn_bwd_clipped(rescaling)", "%dx%dx%d^2" % (N, c, s), ((16 if one_launch else 20) + (8 if one_launch else 0)) * e,
                ms_r, "the delta is rescaled on every call; as two calls this costs a 12 B/elem rescale_clip + the backward")
        if one_launch:
            # both conventions in the row: the bytes this launch moves (frac above) and the 12 / 20 B per
            # element that the three-launch form moves, which is the figure the per-kernel bar was written for
            fwd_row = [r for r in rows if r["kernel"] == "bn_train_fwd(leaky)"][-1]
            bwd_row = [r for r in rows if r["kernel"] == "bn_bwd(leaky)"][-1]
            for row, per_elem, ms in ((fwd_row, 12, ms_f), (bwd_row, 20, ms_b)):
                row["three_launch_bytes_MB"] = round(per_elem * e / 1e6, 1)
                row["frac_of_peak_at_three_launch_bytes"] = round(per_elem * e / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 3)
        bn_ms[(c, s)] = (ms_f, ms_b, count)
        del x, y, d
    # ---- linear bias epilogue of the three head convs at batch 16
    for c, s in wl.YOLOV3_HEAD_CONV_SHAPES:
        e = N * c * s * s
        rot = rotation_for(4 * e)
        xs = [randn(N, c, s, s) for _ in range(rot)]
        bias = randn(c)
        ms = timer.time(lambda i: ops.bias_act_forward(xs[i], xs[i], bias, "linear"), 20, rotate=rot)
        add("bias_fwd(linear)", "%dx%dx%d^2" % (N, c, s), 8 * e, ms, "in place")
        del xs
        bn_ms[("head", s)] = (ms, 0.0, 1)
    # ---- Adam (config 4): 61.9M parameters, 10 steps
    P = wl.YOLOV3_PARAMS
    w = 0.02 * randn(P); g = 1e-3 * randn(P)
    m = torch.zeros(P, device=dev); v = torch.zeros(P, device=dev)
    d = torch.empty(P, device=dev)
    step = [0]

    def adam_step(i):
        step[0] += 1
        ops.adam_update(w, d, m, v, 16, min(step[0], 1000), 1e-3, 0.9, 0.999, 1e-8, 5e-4, True)

    # the call consumes (zeroes) the update buffer, so after the first repetition the gradients are zero:
    # the kernel moves the same bytes and does the same arithmetic whatever the values, and nothing warms
    # a cache for it between repetitions (2 GB per launch), as for the many-tensor rows below
    d.copy_(g)
    ms_adam = timer.time(adam_step, 10)
    add("adam_update", "%d params" % P, 32 * P, ms_adam, "32B/param, L2 folded into the update; gradients zero after the first repetition")
    # four streams read and four written, no arithmetic: what the update's mix of reads and writes costs
    mix_ms = stream_mix_ms(torch, capi, timer, 4, 4, P)
    rows[-1]["copy_same_mix_ms"] = round(mix_ms, 4)
    rows[-1]["vs_same_mix"] = round(mix_ms / ms_adam, 3)
    add("copy_same_mix(4 read + 4 written)", "%d floats per stream" % P, 32 * P, mix_ms,
        "no arithmetic: the ceiling of Adam's traffic mix; a 1+1 copy of these bytes runs at 6.5 TB/s")
    ms_adamw = timer.time(lambda i: ops.adam_update(w, d, m, v, 16, 7, 1e-3, 0.9, 0.999, 1e-8, 5e-4, 2), 10)
    add("adam_update(decoupled decay)", "%d params" % P, 32 * P, ms_adamw,
        "32B/param; the decay as the baseline's configuration words it; not in ms/batch (the reference's form is)")

    # ---- SGD with momentum over the same buffer (the optimiser of the shipped presets)
    ms_sgd = timer.time(lambda i: ops.sgd_update(w, d, 16, 1e-3, 0.9, 5e-4, True), 10)
    add("sgd_update", "%d params" % P, 16 * P, ms_sgd, "16B/param; not in ms/batch (Adam is)")
    # ---- the same parameters as the engine holds them: 222 tensors (three per convolution), updated through
    # the entry points that take many tensors per launch, and one call per tensor beside it
    sizes = wl.yolov3_parameter_tensors(608)
    starts, at = [], 0
    for n_, _ in sizes:
        starts.append(at); at += (n_ + 63) // 64 * 64
    assert at <= w.numel() + 64 * len(sizes)
    big = [torch.zeros(at, device=dev) for _ in range(4)]
    big[0].normal_(0, 0.02); big[1].normal_(0, 1e-3)
    pw, pd, pm, pv = ([flat[o:o + n_] for o, (n_, _) in zip(starts, sizes)] for flat in big)
    decayed = [d_ for _, d_ in sizes]
    ms = timer.time(lambda i: ops.adam_update_multi(pw, pd, pm, pv, 16, 1, 1e-3, 0.9, 0.999, 1e-8, 5e-4, decayed), 10)
    add("adam_update_multi", "%d tensors, %d params" % (len(sizes), P), 32 * P, ms, "7 launches; gradients already zero after the first")

    def one_by_one(i):
        for k in range(len(sizes)):
            ops.adam_update(pw[k], pd[k], pm[k], pv[k], 16, 1, 1e-3, 0.9, 0.999, 1e-8, 5e-4, decayed[k])

    ms = timer.time(one_by_one, 3)
    add("adam_update x222", "%d tensors, %d params" % (len(sizes), P), 32 * P, ms, "one call per tensor, for comparison",
        streaming=False)
    ms = timer.time(lambda i: ops.sgd_update_multi(pw, pd, 16, 1e-3, 0.9, 5e-4, decayed), 10)
    add("sgd_update_multi", "%d tensors, %d params" % (len(sizes), P), 16 * P, ms, "7 launches")
    ms = timer.time(lambda i: ops.rescale_clip_multi(pd, 100.0, 10.0), 10)
    add("rescale_clip_multi(no-op)", "%d update buffers" % len(sizes), 4 * P, ms, "14 launches; norm only, 4B/param")

    # ... and through tables kept on the device: one launch per operation (two for the hooks)
    t_adam = ops.TensorTable([pw, pd, pm, pv], decayed)
    ms = timer.time(lambda i: t_adam.adam_update(16, 1, 1e-3, 0.9, 0.999, 1e-8, 5e-4), 10)
    add("adam_update_table", "%d tensors, %d params" % (len(sizes), P), 32 * P, ms, "1 launch")
    ms = timer.time(lambda i: t_adam.sgd_update(16, 1e-3, 0.9, 5e-4), 10)
    add("sgd_update_table", "%d tensors, %d params" % (len(sizes), P), 16 * P, ms, "1 launch")
    t_hooks = ops.TensorTable([pd])
    ms = timer.time(lambda i: t_hooks.rescale_clip(100.0, 10.0), 10)
    add("rescale_clip_table(no-op)", "%d update buffers" % len(sizes), 4 * P, ms, "2 launches; norm only, 4B/param")
    t_adam.close(); t_hooks.close()

    def hooks_one_by_one(i):
        for k in range(len(sizes)):
            ops.rescale_clip(pd[k], 100.0, 10.0)

    ms = timer.time(hooks_one_by_one, 3)
    add("rescale_clip x222(no-op)", "%d update buffers" % len(sizes), 4 * P, ms,
        "one call (two launches) per buffer, for comparison", streaming=False)
    del w, g, m, v, d, big, pw, pd, pm, pv
    # ---- gradient rescale + clamp of a delta tensor: 4B/elem for the norm, 8B/elem to rewrite
    for c, s_ in [(256, 76), (64, 304)]:
        e = N * c * s_ * s_
        rot = rotation_for(12 * e)
        xs = [randn(N, c, s_, s_) for _ in range(rot)]
        # fresh values before every trial and one call per buffer: a second call on the same data
        # would find nothing left to change and skip the rewrite
        def refill():
            for x in xs:
                x.normal_()

        ms = timer.time(lambda i: ops.rescale_clip(xs[i], 1e-3, 1e-6), rot, warm=0, rotate=rot, prepare=refill)
        add("rescale_clip", "%dx%dx%d^2" % (N, c, s_), 12 * e, ms, "norm 4B + rewrite 8B per elem")
        ms = timer.time(lambda i: ops.rescale_clip(xs[i], 1e30, 0.0), 10, rotate=rot)
        add("rescale_clip(no-op)", "%dx%dx%d^2" % (N, c, s_), 4 * e, ms, "below the threshold: norm only, 4B/elem")
        # the same verdict from the group sums that the kernel which wrote the tensor left behind
        # (pxh_shortcut_backward_norm, pxh_axpy_norm): the tensor is not read
        groups = [ops.norm_groups_like(xs[0]) for _ in range(rot)]
        for x, g in zip(xs, groups):
            ops.norm_groups(x, g)
        ms = timer.time(lambda i: ops.rescale_clip_from_groups(xs[i], groups[i], 1e30, 0.0), 10, rotate=rot)
        add("rescale_clip_from_groups(no-op)", "%dx%dx%d^2" % (N, c, s_), 8 * (e // 256), ms,
            "two launches, 8 B per 256 values read; against the row above", streaming=False)
        del xs, groups

    # ---- non-conv ms per batch, YOLOv3 @608, batch 16, one training step:
    # 72 BN'd conv epilogues fwd+bwd, 3 bias epilogues, 23 shortcuts fwd+bwd, 2 upsamples and 2 route
    # concats fwd+bwd, the four max-pools of the data-movement configuration fwd+bwd, 3 heads (fused
    # decode+delta) measured at batch 16, Adam
    total = 0.0
    for key, (f, b, count) in bn_ms.items():
        total += (f + b) * count
    for key, (f, b, count) in shortcut_ms.items():
        total += (f + b) * count
    for r in rows:
        if r["kernel"] in ("upsample_fwd", "upsample_bwd", "maxpool_fwd", "maxpool_bwd", "route_fwd", "route_bwd"):
            total += r["ms"]
    total += head_ms[(N, "all")][1]      # the three heads as one pass
    total += ms_adam
    # the CPU checker beside the largest shape of every family
    if cpu is not None:
        for r in rows:
            r.update(cpu.get((r["kernel"], r["shape"]), {}))
    return rows, total


def measure_config0(torch, ops, wl, timer, with_cpu=True):
    """configs[0]: the non-convolution layers of a YOLOv3-tiny inference forward at batch 1, 3x416x416
    (the 24 layers of the reference's yolov3-tiny.yml, driven in model order as Model::forward does,
    include/Model.h:1740-1759).  Every conv result is a resident N(0,1) tensor of the real shape; each
    conv layer's epilogue (folded BN + leaky, or bias alone for the two head convs), the six max-pools,
    the upsample, the two routes and the two head decodes run in layer order, once eagerly launched
    and once as one HIP graph.  Beside it the CPU checker on the same tensors, one core, per layer kind."""
    import numpy as np
    dev = torch.device("cuda:0")
    layers = wl.yolov3_tiny_layers(416)
    T = []
    for i, l in enumerate(layers):
        c, s = l["c"], l["s"]
        t = {}
        if l["type"] == "conv":
            t["x"] = torch.from_numpy(wl.normal(3000 + i, (1, c, s, s))).to(dev)
            t["y"] = torch.empty_like(t["x"])
            scale, bias, mean, var = wl.bn_params(2000 + i, c)
            t["host"] = (scale, bias, mean, var)
            t["bias"] = torch.from_numpy(bias).to(dev)
            if l["bn"]:
                t["folded"] = ops.bn_fold(*(torch.from_numpy(a).to(dev) for a in (mean, var, scale, bias)))
        elif l["type"] == "maxpool":
            o = s if l["stride"] == 1 else s // 2
            t["y"] = torch.empty((1, c, o, o), device=dev)
            t["idx"] = torch.empty((1, c, o, o), device=dev, dtype=torch.int32)
        else:
            t["y"] = torch.empty((1, c, s, s), device=dev)
        T.append(t)

    def forward(_):
        for i, (l, t) in enumerate(zip(layers, T)):
            kind = l["type"]
            if kind == "conv" and l["bn"]:
                ops.bn_folded_act_forward(t["x"], t["y"], t["folded"], l["act"])
            elif kind == "conv":
                ops.bias_act_forward(t["x"], t["y"], t["bias"], l["act"])
            elif kind == "maxpool":
                ops.maxpool_forward(T[i - 1]["y"], t["y"], t["idx"], 2, l["stride"], 1)
            elif kind == "upsample":
                ops.upsample_forward(T[i - 1]["y"], t["y"], 2, 1.0)
            elif kind == "route":
                offset = 0
                for src in l["sources"]:
                    ops.route_forward(T[src]["y"], t["y"], offset)
                    offset += layers[src]["c"] * l["s"] * l["s"]
            elif kind == "yolo":
                ops.yolo_activate(T[i - 1]["y"], t["y"], 1, 3, 80, l["s"] * l["s"])

    # the lean forward: the five 2 x 2 / 2 pools on the epilogue of the convolution in front of them
    # (pxh_bn_folded_act_maxpool_forward; the convolution's own output is written only where a route reads it),
    # and the upsample straight into the route behind it
    routed = {src for l in layers if l["type"] == "route" for src in l["sources"]}
    pooled_by = {i: i + 1 for i, l in enumerate(layers[:-1])
                 if l["type"] == "conv" and l["bn"] and layers[i + 1]["type"] == "maxpool" and layers[i + 1]["stride"] == 2}

    def forward_pools_ride(_):
        for i, (l, t) in enumerate(zip(layers, T)):
            kind = l["type"]
            if i in pooled_by:
                ops.bn_folded_act_maxpool_forward(t["x"], T[pooled_by[i]]["y"], t["folded"], l["act"],
                                                  y=t["y"] if i in routed else None)
            elif kind == "maxpool" and i - 1 in pooled_by:
                continue
            elif kind == "conv" and l["bn"]:
                ops.bn_folded_act_forward(t["x"], t["y"], t["folded"], l["act"])
            elif kind == "conv":
                ops.bias_act_forward(t["x"], t["y"], t["bias"], l["act"])
            elif kind == "maxpool":
                ops.maxpool_forward(T[i - 1]["y"], t["y"], t["idx"], 2, l["stride"], 1)
            elif kind == "upsample":
                # straight into the route that follows (pxh_upsample_strided): that source is not copied again
                ops.upsample_forward_into(T[i - 1]["y"], T[i + 1]["y"], 0, 2, 1.0)
            elif kind == "route":
                offset = 0
                for src in l["sources"]:
                    if layers[src]["type"] != "upsample":
                        ops.route_forward(T[src]["y"], t["y"], offset)
                    offset += layers[src]["c"] * l["s"] * l["s"]
            elif kind == "yolo":
                ops.yolo_activate(T[i - 1]["y"], t["y"], 1, 3, 80, l["s"] * l["s"])

    out = dict(workload="YOLOv3-tiny inference forward, batch 1, 416x416: non-conv layers in model order "
                        "(13 conv epilogues, 6 max-pools, 1 upsample, 2 routes, 2 head decodes; 27 launches)")
    out["gpu_graph_ms"] = round(timer.time(forward, 5, warm=2), 4)
    timer.use_graphs, saved = False, timer.use_graphs
    out["gpu_eager_ms"] = round(timer.time(forward, 5, warm=2), 4)
    timer.use_graphs = saved
    # the same outputs with the pools riding and the upsample writing into its route: 21 launches
    watched = list(pooled_by.values()) + [i for i, l in enumerate(layers) if l["type"] == "route"]
    plain_outputs = {p: T[p]["y"].clone() for p in watched}
    for p in watched:
        T[p]["y"].fill_(-1.0)
    out["gpu_graph_pools_ride_ms"] = round(timer.time(forward_pools_ride, 5, warm=2), 4)
    out["pools_riding"] = len(pooled_by)
    out["pools_ride_same_outputs"] = all(bool(torch.equal(T[p]["y"], plain_outputs[p])) for p in watched)
    del plain_outputs
    elems = sum(int(t["y"].numel()) for t in T)
    out["elements_written"] = elems
    if with_cpu:
        import oracle
        oracle.lib()
        F = np.float32
        by_kind = {}
        H = [None] * len(layers)

        def timed(kind, fn):
            t0 = time.perf_counter()
            fn()
            by_kind[kind] = by_kind.get(kind, 0.0) + (time.perf_counter() - t0) * 1e3

        for i, (l, t) in enumerate(zip(layers, T)):
            kind, c, s = l["type"], l["c"], l["s"]
            if kind == "conv":
                y = t["x"].cpu().numpy().copy()
                scale, bias, mean, var = t["host"]
                if l["bn"]:
                    timed("conv epilogue", lambda: oracle.conv_epilogue_forward(
                        True, False, l["act"], 1, c, s, s, y, None, np.zeros(c, F), np.zeros(c, F), mean.copy(),
                        var.copy(), scale, bias, None, None))
                else:
                    timed("conv epilogue", lambda: oracle.conv_epilogue_forward(
                        False, False, l["act"], 1, c, s, s, y, None, None, None, None, None, None, bias, None, None))
                H[i] = y
            elif kind == "maxpool":
                o = s if l["stride"] == 1 else s // 2
                y = np.empty((1, c, o, o), F); idx = np.empty((1, c, o, o), np.int32)
                timed("max-pool", lambda: oracle.maxpool_forward(H[i - 1], y, idx, 1, c, s, s, o, o, 2, l["stride"], 1))
                H[i] = y
            elif kind == "upsample":
                y = np.empty((1, c, s, s), F)
                timed("upsample", lambda: oracle.upsample(H[i - 1], s // 2, s // 2, c, 1, 2, True, 1.0, None, y))
                H[i] = y
            elif kind == "route":
                y = np.empty((1, c * s * s), F)

                def concat():
                    offset = 0
                    for src in l["sources"]:
                        oracle.route_forward(H[src].reshape(1, -1), y, offset)
                        offset += layers[src]["c"] * s * s

                timed("route", concat)
                H[i] = y.reshape(1, c, s, s)
            elif kind == "yolo":
                cfg, keep = oracle.yolo_cfg(1, s, s, 80, l["mask"], wl.TINY_ANCHORS, 416, 416)
                y = np.zeros_like(H[i - 1])
                timed("yolo decode", lambda: oracle.yolo_decode(cfg, H[i - 1], y))
                H[i] = y
        out["cpu_ms_by_layer_kind"] = {k: round(v, 3) for k, v in by_kind.items()}
        out["cpu_ms"] = round(sum(by_kind.values()), 3)
        out["cpu_cores"] = 1
        # the chain's last tensors agree: the two runs did the same work
        last = T[-1]["y"].cpu().numpy()
        out["gpu_matches_cpu"] = bool(np.allclose(last, H[-1], rtol=1e-5, atol=1e-6))
    return out


def cpu_rows(wl):
    """The CPU checker (one core) on one image -- or, for the per-channel reductions, on two channels at
    the full batch -- of the largest shape of each kernel family, scaled to the batch: milliseconds keyed
    by (kernel, shape) as the extras rows name them."""
    import numpy as np
    import oracle
    oracle.lib()
    F = np.float32
    N = 16
    out = {}

    def ms_of(fn, scale):
        # the second of two runs: the first also pays for the first touch of freshly allocated pages
        best = None
        for _ in range(2):
            t0 = time.perf_counter()
            fn()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        return best * 1e3 * scale

    def note(kernel, shape, ms, sample):
        out[(kernel, shape)] = dict(cpu_ms=round(ms, 2), cpu_sample=sample)

    # max-pool 16x64x304^2
    c, s = 64, 304
    x = wl.normal(1, (1, c, s, s)); y = np.empty((1, c, s // 2, s // 2), F); idx = np.empty(y.shape, np.int32)
    note("maxpool_fwd", "%dx%dx%d^2" % (N, c, s), ms_of(lambda: oracle.maxpool_forward(x, y, idx, 1, c, s, s, s // 2, s // 2, 2, 2, 1), N),
         "1 image x %d" % N)
    d = wl.normal(2, y.shape); g = x.copy()
    note("maxpool_bwd", "%dx%dx%d^2" % (N, c, s), ms_of(lambda: oracle.maxpool_backward(d, idx, g), N), "1 image x %d" % N)
    # upsample 16x128x38^2 -> 76^2
    c, s = 128, 38
    x = wl.normal(3, (1, c, s, s)); y = np.empty((1, c, 2 * s, 2 * s), F)
    note("upsample_fwd", "%dx%dx%d^2" % (N, c, s), ms_of(lambda: oracle.upsample(x, s, s, c, 1, 2, True, 1.0, None, y), N),
         "1 image x %d" % N)
    acc = x.copy()
    note("upsample_bwd", "%dx%dx%d^2" % (N, c, s), ms_of(lambda: oracle.upsample(x, s, s, c, 1, 2, False, 1.0, acc, y), N),
         "1 image x %d" % N)
    # shortcut 16x64x304^2
    c, s = 64, 304
    a = wl.normal(4, (1, c, s, s)); b = wl.normal(5, a.shape); o = np.empty_like(a); pre = np.empty_like(a)
    note("shortcut_fwd", "%dx%dx%d^2" % (N, c, s),
         ms_of(lambda: oracle.shortcut_forward("linear", 1, s, s, c, a, b, 1.0, 1.0, o, pre), N), "1 image x %d" % N)
    fd = b.copy(); gr = a.copy()
    note("shortcut_bwd", "%dx%dx%d^2" % (N, c, s),
         ms_of(lambda: oracle.shortcut_backward("linear", 1, s, s, c, o, pre, fd, gr, 1.0, 1.0), N), "1 image x %d" % N)
    # route: the 256-channel source of 16x(128+)256x76^2
    c1, c2, s = 128, 256, 76
    src = wl.normal(6, (1, c2 * s * s)); dst = np.empty((1, (c1 + c2) * s * s), F)
    note("route_fwd", "%dx(%d+)%dx%d^2" % (N, c1, c2, s), ms_of(lambda: oracle.route_forward(src, dst, c1 * s * s), N),
         "1 image x %d" % N)
    note("route_bwd", "%dx(%d+)%dx%d^2" % (N, c1, c2, s), ms_of(lambda: oracle.route_backward(dst, src, c1 * s * s), N),
         "1 image x %d" % N)
    # YOLO head 64x255x76^2: decode, and the training pass with that image's truths
    NB, s = 64, 76
    x = wl.normal(7, (1, 255, s, s), std=2.0)
    truths, counts = wl.yolo_truths(5100, NB)
    cfg, keep = oracle.yolo_cfg(1, s, s, 80, wl.YOLOV3_MASKS[s], wl.YOLOV3_ANCHORS, 608, 608, ignore_thresh=0.7,
                                object_scale=2.0, noobject_scale=0.1)
    y = np.zeros_like(x); dl = np.zeros_like(x)
    note("yolo_decode", "%dx255x%d^2" % (NB, s), ms_of(lambda: oracle.yolo_decode(cfg, x, y), NB), "1 image x %d" % NB)
    note("yolo_decode+delta+cost", "%dx255x%d^2" % (NB, s),
         ms_of(lambda: oracle.yolo_forward(cfg, x, np.ascontiguousarray(truths[:1]), np.ascontiguousarray(counts[:1]),
                                           truths.shape[1], y, dl), NB), "1 image x %d" % NB)
    # BN training forward and backward 16x32x608^2: two channels at the full batch
    c, s, sub = 32, 608, 2
    x = wl.normal(8, (N, sub, s, s)); scale, bias, rm, rv = wl.bn_params(9, sub)
    outp = x.copy(); pre = np.empty_like(x); xs = np.empty_like(x); xn = np.empty_like(x)
    mean = np.zeros(sub, F); var = np.zeros(sub, F)
    note("bn_train_fwd(leaky)", "%dx%dx%d^2" % (N, c, s),
         ms_of(lambda: oracle.conv_epilogue_forward(True, True, "leaky", N, sub, s, s, outp, pre, mean, var, rm, rv, scale,
                                                    bias, xs, xn), c / sub), "%d of %d channels at batch %d, x %d" % (sub, c, N, c // sub))
    dd = wl.normal(10, x.shape); su = np.zeros(sub, F); bu = np.zeros(sub, F); md = np.zeros(sub, F); vd = np.zeros(sub, F)
    note("bn_bwd(leaky)", "%dx%dx%d^2" % (N, c, s),
         ms_of(lambda: oracle.conv_epilogue_backward(True, "leaky", N, sub, s, s, dd, pre, mean, var, md, vd, scale, su, bu,
                                                     xs, xn), c / sub), "%d of %d channels at batch %d, x %d" % (sub, c, N, c // sub))
    # Adam, SGD and the gradient helpers on 4 M parameters, scaled to the 61.9 M of the model
    P, n = wl.YOLOV3_PARAMS, 4 << 20
    w = wl.normal(11, n, std=0.02); g = wl.normal(12, n, std=1e-3); m = np.zeros(n, F); v = np.zeros(n, F)
    note("adam_update", "%d params" % P, ms_of(lambda: oracle.adam_update(w, g, m, v, 16, 1, 1e-3, 0.9, 0.999, 1e-8, 5e-4, True), P / n),
         "%d parameters x %.1f" % (n, P / n))
    g = wl.normal(12, n, std=1e-3)
    note("sgd_update", "%d params" % P, ms_of(lambda: oracle.sgd_update(w, g, 16, 1e-3, 0.9, 5e-4, True), P / n),
         "%d parameters x %.1f" % (n, P / n))
    e = N * 64 * 304 * 304
    g = wl.normal(13, n)
    note("rescale_clip", "%dx%dx%d^2" % (N, 64, 304), ms_of(lambda: oracle.rescale_clip(g, 1e-3, 1e-6), e / n),
         "%d values x %.1f" % (n, e / n))
    return out


def calibration_copy(torch, ops, timer):
    """A plain copy of known size (512 MiB read, 512 MiB written) through the route kernel: the
    launch the hardware traffic counters are scaled by, and the practical ceiling of this HBM."""
    n = 128 << 20
    src = torch.randn((1, n), device="cuda:0")
    dst = torch.empty_like(src)
    ms = timer.time(lambda i: ops.route_forward(src, dst, 0), 10)
    gbs = 8.0 * n / (ms * 1e-3) / 1e9
    return dict(kernel="stream_kernel<4, true, RouteOp<false>>", elems=n, bytes=8 * n, ms=round(ms, 4),
                GBps=round(gbs, 1), frac=round(gbs / HBM_PEAK_GBS, 3))


def cpu_baseline(wl, batch):
    """The CPU checker on `batch` images per shape of the same sweep, one core."""
    import numpy as np
    import oracle
    oracle.lib()
    F = np.float32
    elems = 0
    t_total = 0.0
    for i, (c, s) in enumerate(wl.YOLOV3_TINY_CONV_SHAPES):
        x = wl.normal(3000 + i, (batch, c, s, s))
        scale, bias, mean, var = wl.bn_params(2000 + i, c)
        for act in EPILOGUE_ACTS:
            y = x.copy()
            t0 = time.perf_counter()
            oracle.conv_epilogue_forward(True, False, act, batch, c, s, s, y, None, np.zeros(c, F), np.zeros(c, F),
                                         mean, var, scale, bias, None, None)
            t_total += time.perf_counter() - t0
            elems += x.size
    return dict(value=round(8.0 * elems / t_total / 1e9, 3), unit="GB/s", cores=1, kind="port",
                sample="same 7 shapes x 3 activations at batch %d (%.1f M elements, %.1f s)"
                       % (batch, elems / 1e6, t_total),
                host_cpus=os.cpu_count())


MAX_LINE_BYTES = 4096      # whoever keeps only the tail of stdout must still find the whole record in it


def clean(obj):
    """The same structure with non-finite floats replaced by None, so that the line is strict JSON."""
    if isinstance(obj, float):
        return obj if obj == obj and abs(obj) != float("inf") else None
    if isinstance(obj, dict):
        return {k: clean(v) for k, v in obj.items()}
    if isinstance(obj, (list, tuple)):
        return [clean(v) for v in obj]
    return obj


def write_details(details, folder=None):
    """Writes the per-shape and per-kernel rows to a file beside the script (they are also on stderr as
    they are measured) and returns its path relative to the script, or None if it cannot be written."""
    folder = folder or os.path.join(ROOT, "gpurun_out")
    try:
        os.makedirs(folder, exist_ok=True)
        path = os.path.join(folder, "bench_details.json")
        with open(path, "w") as f:
            json.dump(clean(details), f, indent=1, allow_nan=False)
        return os.path.relpath(path, ROOT)
    except OSError as e:
        log("details not written: %s" % e)
        return None


def final_line(steps, warmup, value, ms_per_step, bytes_step, launches_per_step, roofline, cpu, model_order,
               layer_kernels_sum_ms, value_raw, value_graph, config0, details_file=None):
    """The ONE line of stdout: the record of the run, a few kB of strict JSON.  Everything that is a
    table (rows per shape, per kernel, the phases of the model-order step) goes to stderr and to the
    details file; from them this line keeps scalars only."""
    mo = model_order or {}
    c0 = config0 or {}
    line = {
        "metric": "fused BN+act epilogue GB/s (% of HBM peak); non-conv ms/batch YOLOv3 608",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[1]: fused BN-inference+bias+activation epilogue sweep, NCHW fp32, N=64, "
                               "7 YOLOv3-tiny conv-output shapes x {leaky, mish, logistic}; per-channel constants "
                               "folded once before the timed region",
                   "bytes_per_step": int(bytes_step), "launches_per_step": launches_per_step,
                   "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2)},
        "roofline": roofline,
        "cpu_baseline": cpu,
        # the second half of the metric: one training step of YOLOv3 @608 at batch 16, every non-conv kernel
        # launched in model order with what the Layer base class adds around each layer (three HIP graphs);
        # beside it the leanest form of the same step and the plain sum of the layer kernels' own rows
        "noconv_ms_per_batch_yolov3_608": mo.get("total_ms"),
        "noconv_ms_per_batch_yolov3_608_leanest": mo.get("leanest_total_ms"),
        "noconv_layer_kernels_sum_ms_yolov3_608": None if layer_kernels_sum_ms is None else round(layer_kernels_sum_ms, 3),
        "config0_gpu_ms": c0.get("gpu_graph_ms"),
        "config0_gpu_ms_lean": c0.get("gpu_graph_pools_ride_ms"),
        "config0_cpu_ms": c0.get("cpu_ms"),
        "value_folding_every_call": round(value_raw, 1),
        "value_as_one_hip_graph": round(value_graph, 1),
        "details": details_file,
    }
    text = json.dumps(clean(line), allow_nan=False, separators=(",", ":"))
    assert len(text) < MAX_LINE_BYTES, "the final line grew to %d bytes" % len(text)
    return text


def main():
    args = parse_args()
    if args.gpus != 1:
        log("bench.py measures one GPU: this path has no multi-GPU part (every kernel is independent per image "
            "and per channel); run with --gpus 1")
        sys.exit(2)
    import torch
    from pixienn_amd import capi, ops, workloads as wl
    if not os.path.exists(capi.LIB_PATH):
        from pixienn_amd import build
        build.build_library()      # nothing built yet: build; there is no other path
    capi.load()      # fails loudly when the HIP library is missing
    assert torch.cuda.is_available(), "no GPU visible"
    torch.cuda.set_device(0)
    timer = Timer(torch)
    if args.only_model_order:
        print(json.dumps({"noconv_step_in_model_order_yolov3_608": measure_model_order(torch, ops, wl, timer,
                                                                                        plain_only=args.plain_step)}),
              flush=True)
        return

    if args.only_heads:
        rows, _ = measure_extras(torch, ops, wl, timer, capi, only_heads=True)
        for r in rows:
            log("%-26s %-22s %9.1f MB %8.4f ms %8.1f GB/s  %4.1f%%  %s%s" % (
                r["kernel"], r["shape"], r["MB"], r["ms"], r["GBps"], 100 * r["frac"],
                ("same mix of streams, no arithmetic %.4f ms (%.2f)  " % (r["copy_same_mix_ms"], r["vs_same_mix"]))
                if "vs_same_mix" in r else "", r["note"]))
        print(json.dumps({"yolo_heads": rows}), flush=True)
        return

    shapes = epilogue_workload(torch, wl)
    fold_weights(ops, shapes)
    elems_sweep = sum(sh["elems"] for sh in shapes)
    elems_step = elems_sweep * len(EPILOGUE_ACTS)
    bytes_step = 8.0 * elems_step

    for _ in range(args.warmup):
        run_epilogue_step(ops, shapes)
    torch.cuda.synchronize()
    # the timed region: HIP events around the roofline kernel's group of launches only (every event pair costs
    # the step a few microseconds); the other activations' groups are bracketed in a few more steps after it
    events = []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_epilogue_step(ops, shapes, events, torch, bracket=("leaky",))
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    value = bytes_step / (ms_per_step * 1e-3) / 1e9
    others = tuple(a for a in EPILOGUE_ACTS if a != "leaky")
    for _ in range(min(args.steps, 20)):
        run_epilogue_step(ops, shapes, events, torch, bracket=others)
    torch.cuda.synchronize()

    # per-activation kernel figures from the event pairs
    group_ms = {}
    for act, a, b in events:
        group_ms.setdefault(act, []).append(a.elapsed_time(b))
    per_act = {}
    for act, v in group_ms.items():
        ms = sum(v) / len(v)
        per_act[act] = dict(ms_per_sweep=round(ms, 4), GBps=round(8.0 * elems_sweep / (ms * 1e-3) / 1e9, 1))
        log("epilogue %-9s sweep of %d shapes: %8.4f ms %8.1f GB/s" % (act, len(shapes), ms, per_act[act]["GBps"]))
    launches = len(shapes)
    leaky_ms = sum(group_ms["leaky"]) / len(group_ms["leaky"])
    achieved = 8.0 * elems_sweep / (leaky_ms * 1e-3) / 1e9
    bytes_per_launch = 8.0 * elems_sweep / launches
    roofline = dict(bound="hbm", achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=round(achieved / HBM_PEAK_GBS, 4),
                    traffic=None if EPILOGUE_TRAFFIC_RATIO is None else round(EPILOGUE_TRAFFIC_RATIO * bytes_per_launch),
                    traffic_source="profiles/epilogue_sweep_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE of "
                                   "this script; not measured in this run)",
                    kernel="epilogue_fwd_kernel<PXH_LEAKY, true, *>",
                    bytes_per_launch=round(bytes_per_launch),
                    mean_launch_ms=round(leaky_ms / launches, 5))

    # the same step through the two-launch entry point that folds the constants on every call
    for _ in range(2):
        run_epilogue_step(ops, shapes, raw=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_epilogue_step(ops, shapes, raw=True)
    torch.cuda.synchronize()
    value_raw = bytes_step / ((time.perf_counter() - t0) / args.steps) / 1e9
    log("whole sweep: %.1f GB/s with folded constants, %.1f GB/s folding on every call" % (value, value_raw))

    # the same step with its 21 launches recorded in a HIP graph (what a host that captures its layer
    # sequence runs): no gaps between the launches, nothing else changes
    graph_ms = timer.time(lambda i: run_epilogue_step(ops, shapes), 10, warm=1)
    value_graph = bytes_step / (graph_ms * 1e-3) / 1e9
    log("whole sweep as one HIP graph: %.4f ms per step, %.1f GB/s" % (graph_ms, value_graph))

    # per shape, each measured alone over rotating buffers (HIP events around 20 launches)
    per_shape = []
    if not args.no_extras:
        copy_of_size = same_bytes_copier(torch, ops, timer)
        for sh in shapes:
            rot = rotation_for(8 * sh["elems"])
            xs = [sh["x"]] + [torch.randn_like(sh["x"]) for _ in range(rot - 1)]
            ys = [sh["y"]] + [torch.empty_like(sh["y"]) for _ in range(rot - 1)]
            for act in EPILOGUE_ACTS:
                ms = timer.time(lambda i: ops.bn_folded_act_forward(xs[i], ys[i], sh["folded"], act), 20, rotate=rot)
                r = dict(act=act, shape="%dx%dx%d^2" % (EPILOGUE_BATCH, sh["c"], sh["s"]), ms=round(ms, 4),
                         ms_min=round(timer.last_min, 4), GBps=round(8.0 * sh["elems"] / (ms * 1e-3) / 1e9, 1))
                if r["GBps"] < 0.70 * HBM_PEAK_GBS:      # as for the other kernels' rows under the bar
                    c_ms = copy_of_size(8 * sh["elems"])
                    r["copy_same_bytes_ms"] = round(c_ms, 4)
                    r["vs_copy"] = round(c_ms / ms, 3)
                per_shape.append(r)
                log("epilogue %-9s %-16s %8.4f ms %8.1f GB/s%s" % (r["act"], r["shape"], r["ms"], r["GBps"],
                    ("  copy of the same bytes %.4f ms (%.2f)" % (r["copy_same_bytes_ms"], r["vs_copy"]))
                    if "vs_copy" in r else ""))
            del xs, ys

    copy_row = calibration_copy(torch, ops, timer)
    log("plain copy of 2 x 512 MiB: %.4f ms %.1f GB/s" % (copy_row["ms"], copy_row["GBps"]))

    extras, ms_batch, model_order, config0 = (None, None, None, None)
    if not args.no_extras:
        config0 = measure_config0(torch, ops, wl, timer, with_cpu=not args.no_cpu)
        log("configs[0], YOLOv3-tiny inference forward at batch 1, non-conv layers in model order:", config0)
        cpu_by_row = None
        if not args.no_cpu:
            t0 = time.perf_counter()
            cpu_by_row = cpu_rows(wl)
            log("CPU checker on the largest shape of every kernel family: %.1f s" % (time.perf_counter() - t0))
        extras, ms_batch = measure_extras(torch, ops, wl, timer, capi, cpu_by_row)
        for r in extras:
            log("%-26s %-22s %9.1f MB %8.4f ms %8.1f GB/s  %4.1f%%  %s%s%s"
                % (r["kernel"], r["shape"], r["MB"], r["ms"], r["GBps"], 100 * r["frac"],
                   (("copy of the same bytes %.4f ms (%.2f)  " % (r["copy_same_bytes_ms"], r["vs_copy"]))
                    if "vs_copy" in r else "") +
                   (("same mix of streams, no arithmetic %.4f ms (%.2f)  " % (r["copy_same_mix_ms"], r["vs_same_mix"]))
                    if "vs_same_mix" in r else ""),
                   ("cpu %.1f ms  " % r["cpu_ms"]) if "cpu_ms" in r else "", r["note"]))
        log("sum of the layer kernels of one YOLOv3 @608 training step at batch 16: %.3f ms" % ms_batch)
        model_order = measure_model_order(torch, ops, wl, timer)
        log("the same step in model order, with the Layer base's fills and gradient helpers:", model_order)

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(wl, args.cpu_batch)
        log("cpu baseline:", cpu)

    details = {
        "noconv_step_in_model_order_yolov3_608": model_order,
        "config0_yolov3_tiny_forward_batch1": config0,
        "plain_copy": copy_row,
        "per_activation": per_act,
        "per_shape": per_shape,
        "extras": extras,
    }
    line = final_line(args.steps, args.warmup, value, ms_per_step, bytes_step, len(shapes) * len(EPILOGUE_ACTS),
                      roofline, cpu, model_order, ms_batch, value_raw, value_graph, config0,
                      details_file=write_details(details))
    print(line, flush=True)


if __name__ == "__main__":
    main()
