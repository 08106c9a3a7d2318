"""Torch-tensor front-end over the C ABI: argument checking and stream plumbing only.

Every function launches on torch's current HIP stream and returns without synchronising.
Tensors must be fp32 (int32 for indices), contiguous and on a HIP device.
"""
import ctypes

import numpy as np
import torch

from . import capi, workloads
from .capi import PxError, act_id, call, ptr


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _chk(t, dtype=torch.float32, name="tensor"):
    if t is None:
        return
    if not isinstance(t, torch.Tensor):
        raise PxError("%s: torch.Tensor expected" % name)
    if not t.is_cuda:
        raise PxError("%s must live on the GPU (got %s); there is no CPU path" % (name, t.device))
    if t.dtype != dtype:
        raise PxError("%s must be %s (got %s)" % (name, dtype, t.dtype))
    if not t.is_contiguous():
        raise PxError("%s must be contiguous" % name)


def _chk_all(*ts):
    for t in ts:
        _chk(t)


def _nchw(x):
    if x.dim() != 4:
        raise PxError("NCHW tensor expected, got %d dims" % x.dim())
    n, c, h, w = x.shape
    return n, c, h * w


# ---------------------------------------------------------------- epilogue forward
def bn_infer_act_forward(x, y, rolling_mean, rolling_var, scale, bias, activation, pre_activation=None,
                         workspace=None):
    _chk_all(x, y, rolling_mean, rolling_var, scale, bias, pre_activation)
    n, c, s = _nchw(x)
    wb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    call("pxh_bn_infer_act_forward", ptr(x), ptr(y), ptr(pre_activation), ptr(rolling_mean), ptr(rolling_var),
         ptr(scale), ptr(bias), n, c, s, act_id(activation), ptr(workspace), wb, _stream())
    return y


def bn_fold(rolling_mean, rolling_var, scale, bias, folded=None):
    """Folds the per-channel inference constants; returns the folded buffer."""
    _chk_all(rolling_mean, rolling_var, scale, bias)
    c = rolling_mean.numel()
    if folded is None:
        folded = torch.empty(int(capi.load().pxh_bn_folded_bytes(c)) // 4, device=rolling_mean.device,
                             dtype=torch.float32)
    _chk(folded)
    call("pxh_bn_fold", ptr(rolling_mean), ptr(rolling_var), ptr(scale), ptr(bias), c, ptr(folded), _stream())
    return folded


def bn_folded_act_forward(x, y, folded, activation, pre_activation=None):
    _chk_all(x, y, folded, pre_activation)
    n, c, s = _nchw(x)
    call("pxh_bn_folded_act_forward", ptr(x), ptr(y), ptr(pre_activation), ptr(folded), n, c, s,
         act_id(activation), _stream())
    return y


def bias_act_forward(x, y, bias, activation, pre_activation=None):
    _chk_all(x, y, bias, pre_activation)
    n, c, s = _nchw(x)
    call("pxh_bias_act_forward", ptr(x), ptr(y), ptr(pre_activation), ptr(bias), n, c, s, act_id(activation),
         _stream())
    return y


def bn_workspace_bytes(batch, channels, spatial):
    return int(capi.load().pxh_bn_workspace_bytes(batch, channels, spatial))


def bn_train_act_forward(x, y, mean, var, rolling_mean, rolling_var, scale, bias, activation,
                         pre_activation=None, x_saved=None, x_norm=None, workspace=None):
    _chk_all(x, y, mean, var, rolling_mean, rolling_var, scale, bias, pre_activation, x_saved, x_norm)
    n, c, s = _nchw(x)
    wb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    call("pxh_bn_train_act_forward", ptr(x), ptr(y), ptr(pre_activation), ptr(x_saved), ptr(x_norm), ptr(mean),
         ptr(var), ptr(rolling_mean), ptr(rolling_var), ptr(scale), ptr(bias), n, c, s, act_id(activation),
         ptr(workspace), wb, _stream())
    return y


def bn_stats(x, mean, var, workspace=None):
    _chk_all(x, mean, var)
    n, c, s = _nchw(x)
    wb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    call("pxh_bn_stats", ptr(x), ptr(mean), ptr(var), n, c, s, ptr(workspace), wb, _stream())


# ---------------------------------------------------------------- epilogue backward
def bn_train_act_shortcut_forward(x, y, mean, var, rolling_mean, rolling_var, scale, bias, activation, from_, alpha=1.0,
                                  beta=1.0, pre_activation=None, x_saved=None, x_norm=None, workspace=None):
    """bn_train_act_forward with the linear shortcut that follows the layer: y = alpha*act(pre) + beta*from_."""
    _chk_all(x, y, mean, var, rolling_mean, rolling_var, scale, bias, from_, pre_activation, x_saved, x_norm)
    n, c, s = _nchw(x)
    wb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    call("pxh_bn_train_act_shortcut_forward", ptr(x), ptr(y), ptr(pre_activation), ptr(x_saved), ptr(x_norm), ptr(mean),
         ptr(var), ptr(rolling_mean), ptr(rolling_var), ptr(scale), ptr(bias), ptr(from_), float(alpha), float(beta),
         n, c, s, act_id(activation), ptr(workspace), wb, _stream())


def bn_folded_act_shortcut_forward(x, y, folded, activation, from_, alpha=1.0, beta=1.0, pre_activation=None):
    """bn_folded_act_forward with the linear shortcut that follows the layer."""
    _chk_all(x, y, from_, pre_activation)
    n, c, s = _nchw(x)
    call("pxh_bn_folded_act_shortcut_forward", ptr(x), ptr(y), ptr(pre_activation), ptr(folded), ptr(from_),
         float(alpha), float(beta), n, c, s, act_id(activation), _stream())


def bn_folded_act_maxpool_forward(x, pooled, folded, activation, y=None):
    """bn_folded_act_forward with the 2x2 / 2 max-pool that follows the layer; x is [N, C, H, W]."""
    _chk_all(x, pooled, y)
    n, c, h, w = x.shape
    call("pxh_bn_folded_act_maxpool_forward", ptr(x), ptr(y), ptr(pooled), ptr(folded), n, c, h, w, act_id(activation),
         _stream())


def bn_act_backward(delta, x, mean, var, scale, bias, scale_updates, bias_updates, activation,
                    pre_activation=None, mean_delta=None, var_delta=None, workspace=None):
    _chk_all(delta, x, mean, var, scale, bias, scale_updates, bias_updates, pre_activation, mean_delta, var_delta)
    n, c, s = _nchw(delta)
    wb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    call("pxh_bn_act_backward", ptr(delta), ptr(x), ptr(pre_activation), ptr(mean), ptr(var), ptr(scale), ptr(bias),
         ptr(scale_updates), ptr(bias_updates), ptr(mean_delta), ptr(var_delta), n, c, s, act_id(activation),
         ptr(workspace), wb, _stream())
    return delta


def bias_act_backward(delta, pre_activation, bias_updates, activation, workspace=None):
    _chk_all(delta, pre_activation, bias_updates)
    n, c, s = _nchw(delta)
    wb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    call("pxh_bias_act_backward", ptr(delta), ptr(pre_activation), ptr(bias_updates), n, c, s, act_id(activation),
         ptr(workspace), wb, _stream())
    return delta


def bn_act_backward_clipped(delta, x, mean, var, scale, bias, scale_updates, bias_updates, activation, threshold,
                            clip, norm_out=None, pre_activation=None, mean_delta=None, var_delta=None, workspace=None):
    """rescale_clip(delta, threshold, clip) then bn_act_backward, without the read of delta for its norm."""
    _chk_all(delta, x, mean, var, scale, bias, scale_updates, bias_updates, pre_activation, mean_delta, var_delta,
             norm_out)
    n, c, s = _nchw(delta)
    wb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    call("pxh_bn_act_backward_clipped", ptr(delta), ptr(x), ptr(pre_activation), ptr(mean), ptr(var), ptr(scale),
         ptr(bias), ptr(scale_updates), ptr(bias_updates), ptr(mean_delta), ptr(var_delta), n, c, s,
         act_id(activation), float(threshold), float(clip), ptr(norm_out), ptr(workspace), wb, _stream())
    return delta


def bias_act_backward_clipped(delta, pre_activation, bias_updates, activation, threshold, clip, norm_out=None,
                              workspace=None):
    """rescale_clip(delta, threshold, clip) then bias_act_backward, without the read of delta for its norm."""
    _chk_all(delta, pre_activation, bias_updates, norm_out)
    n, c, s = _nchw(delta)
    wb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    call("pxh_bias_act_backward_clipped", ptr(delta), ptr(pre_activation), ptr(bias_updates), n, c, s,
         act_id(activation), float(threshold), float(clip), ptr(norm_out), ptr(workspace), wb, _stream())
    return delta


# ---------------------------------------------------------------- stand-alone pieces
def activate(activation, x):
    _chk(x)
    call("pxh_activate", act_id(activation), ptr(x), x.numel(), _stream())
    return x


def gradient(activation, x, delta):
    _chk_all(x, delta)
    call("pxh_gradient", act_id(activation), ptr(x), x.numel(), ptr(delta), _stream())
    return delta


def add_bias(output, bias, batch, n, size):
    _chk_all(output, bias)
    call("pxh_add_bias", ptr(output), ptr(bias), batch, n, size, _stream())


def backward_bias(bias_updates, delta, batch, n, size):
    _chk_all(bias_updates, delta)
    call("pxh_backward_bias", ptr(bias_updates), ptr(delta), batch, n, size, None, 0, _stream())


def fill(x, value):
    if x.dtype == torch.int32:
        _chk(x, torch.int32)
        call("pxh_fill_i32", ptr(x), x.numel(), int(value), _stream())
    else:
        _chk(x)
        call("pxh_fill_f32", ptr(x), x.numel(), float(value), _stream())
    return x


def constrain(alpha, x):
    _chk(x)
    call("pxh_constrain", x.numel(), float(alpha), ptr(x), _stream())


def mul(x, y):
    _chk_all(x, y)
    call("pxh_mul", x.numel(), ptr(x), ptr(y), _stream())


def axpy(alpha, x, y):
    _chk_all(x, y)
    call("pxh_axpy", x.numel(), float(alpha), ptr(x), ptr(y), _stream())


def route_forward(layer_output, route_output, offset):
    """Copies one source layer into its slice of a concatenation (include/RouteLayer.h:91-113).
    layer_output [N, ...] packed; route_output [N, ...]; offset in floats within a route image."""
    _chk_all(layer_output, route_output)
    batch = layer_output.shape[0]
    call("pxh_route_forward", ptr(layer_output), ptr(route_output), batch, layer_output.numel() // max(1, batch),
         route_output.numel() // max(1, batch), int(offset), _stream())


def route_backward(route_delta, layer_delta, offset):
    """layer_delta += the layer's slice of route_delta (include/RouteLayer.h:115-137)."""
    _chk_all(route_delta, layer_delta)
    batch = layer_delta.shape[0]
    call("pxh_route_backward", ptr(route_delta), ptr(layer_delta), batch, layer_delta.numel() // max(1, batch),
         route_delta.numel() // max(1, batch), int(offset), _stream())


# ---------------------------------------------------------------- max-pool / upsample / shortcut
def maxpool_out_dim(n, kernel, stride, padding):
    """include/MaxPoolLayer.h:62-63 of the reference."""
    return (n + padding - kernel) // stride + 1


def maxpool_forward(x, out, indexes, kernel, stride, padding):
    _chk_all(x, out)
    _chk(indexes, torch.int32, "indexes")
    n, c, ih, iw = x.shape
    oh, ow = out.shape[2], out.shape[3]
    call("pxh_maxpool_forward", ptr(x), ptr(out), ptr(indexes), n, c, ih, iw, oh, ow, kernel, stride, padding,
         _stream())


def maxpool_backward(delta, indexes, grad, kernel, stride, padding):
    _chk_all(delta, grad)
    _chk(indexes, torch.int32, "indexes")
    n, c, ih, iw = grad.shape
    oh, ow = delta.shape[2], delta.shape[3]
    call("pxh_maxpool_backward", ptr(delta), ptr(indexes), ptr(grad), n, c, ih, iw, oh, ow, kernel, stride, padding,
         _stream())


def maxpool_backward_scatter(delta, indexes, grad):
    _chk_all(delta, grad)
    _chk(indexes, torch.int32, "indexes")
    call("pxh_maxpool_backward_scatter", ptr(delta), ptr(indexes), ptr(grad), delta.numel(), _stream())


def upsample_forward(x, out, stride=2, scale=1.0):
    _chk_all(x, out)
    n, c, h, w = x.shape
    call("pxh_upsample", ptr(x), w, h, c, n, stride, 1, float(scale), None, ptr(out), _stream())


def upsample_backward(delta, grad, stride=2, scale=1.0):
    _chk_all(delta, grad)
    n, c, h, w = grad.shape
    call("pxh_upsample", None, w, h, c, n, stride, 0, float(scale), ptr(grad), ptr(delta), _stream())


def upsample_forward_into(x, buffer, channel_offset, stride=2, scale=1.0):
    """Upsample x straight into channels [channel_offset, channel_offset + C) of a wider NCHW buffer."""
    _chk_all(x, buffer)
    n, c, h, w = x.shape
    plane = buffer.shape[2] * buffer.shape[3]
    if buffer.shape[0] != n or buffer.shape[2] != h * stride or buffer.shape[3] != w * stride \
            or channel_offset < 0 or channel_offset + c > buffer.shape[1]:
        raise ValueError("buffer %s cannot hold %s upsampled by %d at channel %d"
                         % (tuple(buffer.shape), tuple(x.shape), stride, channel_offset))
    call("pxh_upsample_strided", ptr(x), w, h, c, n, stride, 1, float(scale), None,
         ptr(buffer) + 4 * channel_offset * plane, buffer.shape[1] * plane, _stream())


def upsample_backward_from(buffer_delta, channel_offset, grad, stride=2, scale=1.0):
    """Backward of upsample_forward_into: reads the delta slice of the wider buffer in place."""
    _chk_all(buffer_delta, grad)
    n, c, h, w = grad.shape
    plane = buffer_delta.shape[2] * buffer_delta.shape[3]
    if buffer_delta.shape[0] != n or buffer_delta.shape[2] != h * stride or buffer_delta.shape[3] != w * stride \
            or channel_offset < 0 or channel_offset + c > buffer_delta.shape[1]:
        raise ValueError("buffer %s does not hold %s upsampled by %d at channel %d"
                         % (tuple(buffer_delta.shape), tuple(grad.shape), stride, channel_offset))
    call("pxh_upsample_strided", None, w, h, c, n, stride, 0, float(scale), ptr(grad),
         ptr(buffer_delta) + 4 * channel_offset * plane, buffer_delta.shape[1] * plane, _stream())


def shortcut(batch, w1, h1, c1, add, w2, h2, c2, s1, s2, out):
    _chk_all(add, out)
    call("pxh_shortcut", batch, w1, h1, c1, ptr(add), w2, h2, c2, float(s1), float(s2), ptr(out), _stream())


def shortcut_forward(inp, from_output, output, activation="linear", alpha=1.0, beta=1.0, pre_activation=None):
    _chk_all(inp, from_output, output, pre_activation)
    call("pxh_shortcut_forward", ptr(inp), ptr(from_output), ptr(output), ptr(pre_activation), inp.numel(),
         float(alpha), float(beta), act_id(activation), _stream())


def shortcut_backward(delta, from_delta, grad=None, activation="linear", alpha=1.0, beta=1.0, pre_activation=None):
    _chk_all(delta, from_delta, grad, pre_activation)
    call("pxh_shortcut_backward", ptr(delta), ptr(pre_activation), ptr(from_delta), ptr(grad), delta.numel(),
         float(alpha), float(beta), act_id(activation), _stream())


def shortcut_backward_first(delta, from_delta, grad=None, activation="linear", alpha=1.0, beta=1.0,
                            pre_activation=None):
    """shortcut_backward for the first writer of both targets: overwrites instead of accumulating."""
    _chk_all(delta, from_delta, grad, pre_activation)
    call("pxh_shortcut_backward_first", ptr(delta), ptr(pre_activation), ptr(from_delta), ptr(grad), delta.numel(),
         float(alpha), float(beta), act_id(activation), _stream())


def shortcut_backward_clipped(delta, from_delta, grad=None, activation="linear", alpha=1.0, beta=1.0,
                              pre_activation=None, first=True, threshold=0.0, clip=0.0, norm_out=None, workspace=None):
    """rescale_clip(delta, threshold, clip, norm_out), then the shortcut's backward (first writer or accumulating)."""
    _chk_all(delta, from_delta, grad, pre_activation, norm_out, workspace)
    wb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    call("pxh_shortcut_backward_clipped", ptr(delta), ptr(pre_activation), ptr(from_delta), ptr(grad), delta.numel(),
         float(alpha), float(beta), act_id(activation), int(bool(first)), float(threshold), float(clip), ptr(norm_out),
         ptr(workspace), wb, _stream())


# ---------------------------------------------------------------- YOLO head
def yolo_activate(inp, out, batch, masks, classes, area):
    _chk_all(inp, out)
    call("pxh_yolo_activate", ptr(inp), ptr(out), batch, masks, classes, area, _stream())


def yolo_forward_train(inp, out, delta, truths, truth_counts, max_truth, masks, anchors, stats, cost, batch, classes,
                       width, height, net_width, net_height, ignore_thresh, truth_thresh, coord_scale=1.0,
                       object_scale=1.0, noobject_scale=1.0, class_scale=1.0, workspace=None):
    _chk_all(inp, out, delta, truths, stats, cost)
    _chk(truth_counts, torch.int32, "truth_counts")
    m = np.ascontiguousarray(masks, dtype=np.int32)
    a = np.ascontiguousarray(anchors, dtype=np.int32)
    wb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    call("pxh_yolo_forward_train", ptr(inp), ptr(out), ptr(delta), ptr(truths), ptr(truth_counts), int(max_truth),
         m.ctypes.data, a.ctypes.data, ptr(stats), ptr(cost), batch, len(m), len(a) // 2, classes, width, height,
         net_width, net_height, float(ignore_thresh), float(truth_thresh), float(coord_scale), float(object_scale),
         float(noobject_scale), float(class_scale), ptr(workspace), wb, _stream())


def yolo_head_table(heads):
    """An array of pxh_yolo_head from dicts with keys input, output, delta, masks, width, height and, optionally,
    stats, cost, ignore_thresh (0.7), truth_thresh (1), coord_scale, object_scale, noobject_scale, class_scale (1).
    Returns (array, keep-alive list)."""
    table = (capi.YoloHead * len(heads))()
    keep = []
    for t, h in zip(table, heads):
        _chk_all(h["input"], h["output"], h["delta"], h.get("stats"), h.get("cost"))
        m = np.ascontiguousarray(h["masks"], dtype=np.int32)
        keep.append(m)
        t.input, t.output, t.delta = ptr(h["input"]), ptr(h["output"]), ptr(h["delta"])
        t.masks, t.mask_count = m.ctypes.data, len(m)
        t.width, t.height = int(h["width"]), int(h["height"])
        t.ignore_thresh = float(h.get("ignore_thresh", 0.7)); t.truth_thresh = float(h.get("truth_thresh", 1.0))
        t.coord_scale = float(h.get("coord_scale", 1.0)); t.object_scale = float(h.get("object_scale", 1.0))
        t.noobject_scale = float(h.get("noobject_scale", 1.0)); t.class_scale = float(h.get("class_scale", 1.0))
        t.stats, t.cost = ptr(h.get("stats")), ptr(h.get("cost"))
    return table, keep


def yolo_forward_train_heads(heads, truths, truth_counts, max_truth, anchors, batch, classes, net_width, net_height,
                             workspace=None, table=None):
    """All heads of a model in one pass (pxh_yolo_forward_train_heads); `heads` as for yolo_head_table, or a
    table built by it beforehand."""
    _chk_all(truths)
    _chk(truth_counts, torch.int32, "truth_counts")
    keep = None
    if table is None:
        table, keep = yolo_head_table(heads)
    a = np.ascontiguousarray(anchors, dtype=np.int32)
    wb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    call("pxh_yolo_forward_train_heads", len(table), ctypes.addressof(table), ptr(truths), ptr(truth_counts),
         int(max_truth), a.ctypes.data, len(a) // 2, batch, classes, net_width, net_height, ptr(workspace), wb, _stream())
    del keep


def yolo_loss(output, delta, truths, truth_counts, max_truth, assigned_classes, assigned_anchors, assigned_boxes,
              masks, anchors, stats, cost, batch, anchor_count, classes, width, height, net_width, net_height,
              ignore_thresh, truth_thresh, coord_scale, object_scale, noobject_scale, class_scale):
    _chk_all(output, delta, truths, assigned_boxes, anchors, stats, cost)
    for t, nm in ((truth_counts, "truth_counts"), (assigned_classes, "assigned_classes"),
                  (assigned_anchors, "assigned_anchors"), (masks, "masks")):
        _chk(t, torch.int32, nm)
    call("pxh_yolo_loss", ptr(output), ptr(delta), ptr(truths), ptr(truth_counts), int(max_truth),
         ptr(assigned_classes), ptr(assigned_anchors), ptr(assigned_boxes), ptr(masks), ptr(anchors), ptr(stats),
         ptr(cost), batch, masks.numel(), anchor_count, classes, width, height, net_width, net_height,
         float(ignore_thresh), float(truth_thresh), float(coord_scale), float(object_scale), float(noobject_scale),
         float(class_scale), None, 0, _stream())


# ---------------------------------------------------------------- Adam
def adam(x, m, v, beta1, beta2, rate, eps, t):
    _chk_all(x, m, v)
    call("pxh_adam", x.numel(), ptr(x), ptr(m), ptr(v), float(beta1), float(beta2), float(rate), float(eps), int(t),
         _stream())


def adam_update(w, d, m, v, batch, t, lr, beta1=0.9, beta2=0.999, eps=1e-8, decay=0.0, apply_decay=False):
    """apply_decay: False / 0 none, True / 1 the reference's L2 term, 2 decoupled decay."""
    _chk_all(w, d, m, v)
    call("pxh_adam_update", w.numel(), ptr(w), ptr(d), ptr(m), ptr(v), int(batch), int(t), float(lr), float(beta1),
         float(beta2), float(eps), float(decay), int(apply_decay), _stream())


def _pointer_table(tensors):
    import ctypes
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def _size_table(tensors):
    import ctypes
    return (ctypes.c_size_t * len(tensors))(*[t.numel() for t in tensors])


def _flag_table(flags, count):
    import ctypes
    if flags is None:
        return None
    assert len(flags) == count
    return (ctypes.c_int * count)(*[int(bool(f)) for f in flags])


def adam_update_multi(ws, ds, ms, vs, batch, t, lr, beta1=0.9, beta2=0.999, eps=1e-8, decay=0.0, apply_decay=None):
    """pxh_adam_update for lists of tensors (one entry per parameter tensor) in a few launches."""
    _chk_all(*ws, *ds, *ms, *vs)
    count = len(ws)
    assert len(ds) == count and len(ms) == count and len(vs) == count
    for group in zip(ws, ds, ms, vs):
        assert len({x.numel() for x in group}) == 1
    call("pxh_adam_update_multi", count, _pointer_table(ws), _pointer_table(ds), _pointer_table(ms), _pointer_table(vs),
         _size_table(ws), _flag_table(apply_decay, count), int(batch), int(t), float(lr), float(beta1), float(beta2),
         float(eps), float(decay), _stream())


def sgd_update_multi(ws, ds, batch, lr, momentum, decay=0.0, apply_decay=None):
    """pxh_sgd_update for lists of tensors in a few launches."""
    _chk_all(*ws, *ds)
    count = len(ws)
    assert len(ds) == count
    call("pxh_sgd_update_multi", count, _pointer_table(ws), _pointer_table(ds), _size_table(ws),
         _flag_table(apply_decay, count), int(batch), float(lr), float(momentum), float(decay), _stream())


def sgd_update(w, d, batch, lr, momentum, decay=0.0, apply_decay=False):
    """include/ConvLayer.h:309-311 of the reference for one parameter tensor."""
    _chk_all(w, d)
    call("pxh_sgd_update", w.numel(), ptr(w), ptr(d), int(batch), float(lr), float(momentum), float(decay),
         int(bool(apply_decay)), _stream())


class TensorTable:
    """A table of tensors kept on the device (pxh_tensor_table): build once, then every operation over all
    of them is one launch.  `streams` is a list of 1, 2 or 4 lists of tensors (x | w, d | w, d, m, v)."""

    def __init__(self, streams, apply_decay=None):
        import ctypes
        count = len(streams[0])
        for group in streams:
            assert len(group) == count
            _chk_all(*group)
        for tensors in zip(*streams):
            assert len({x.numel() for x in tensors}) == 1
        flat = [t for group in streams for t in group]
        self._keep = flat                      # the tensors must outlive the table
        handle = ctypes.c_void_p()
        call("pxh_tensor_table_create", count, len(streams), _pointer_table(flat), _size_table(streams[0]),
             _flag_table(apply_decay, count), ctypes.byref(handle))
        self.handle = handle
        self.count = int(capi.load().pxh_tensor_table_count(handle))

    def close(self):
        if self.handle:
            capi.load().pxh_tensor_table_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:      # noqa: BLE001 - interpreter shutdown
            pass

    def adam_update(self, batch, t, lr, beta1=0.9, beta2=0.999, eps=1e-8, decay=0.0):
        call("pxh_adam_update_table", self.handle, int(batch), int(t), float(lr), float(beta1), float(beta2),
             float(eps), float(decay), _stream())

    def sgd_update(self, batch, lr, momentum, decay=0.0):
        call("pxh_sgd_update_table", self.handle, int(batch), float(lr), float(momentum), float(decay), _stream())

    def fill(self, value):
        call("pxh_fill_f32_table", self.handle, float(value), _stream())

    def rescale_clip(self, threshold=0.0, clip=0.0, norms=None):
        _chk(norms)
        call("pxh_rescale_clip_table", self.handle, float(threshold), float(clip), ptr(norms), _stream())


def fill_multi(xs, value):
    """pxh_fill_f32 for a list of float tensors in a few launches."""
    _chk_all(*xs)
    call("pxh_fill_f32_multi", len(xs), _pointer_table(xs), _size_table(xs), float(value), _stream())


def rescale_clip_multi(xs, threshold=0.0, clip=0.0, norms=None):
    """pxh_rescale_clip for a list of tensors in a few launches; `norms`: device float tensor, one per tensor."""
    _chk_all(*xs, norms)
    if norms is not None:
        assert norms.numel() == len(xs)
    call("pxh_rescale_clip_multi", len(xs), _pointer_table(xs), _size_table(xs), float(threshold), float(clip),
         ptr(norms), None, 0, _stream())


def rescale_clip(x, threshold=0.0, clip=0.0, norm_out=None):
    """Gradient rescale to a norm threshold, then clamp (include/Layer.h:385-397 of the reference)."""
    _chk_all(x, norm_out)
    call("pxh_rescale_clip", ptr(x), x.numel(), float(threshold), float(clip), ptr(norm_out), None, 0, _stream())


def norm_groups_like(x):
    """A group-sum buffer for a tensor of x's size (8 bytes per 256 values), on x's device."""
    import torch
    n = capi.load().pxh_norm_groups_bytes(x.numel()) // 4
    return torch.empty(max(n, 2), dtype=torch.float32, device=x.device)


def norm_groups(x, groups):
    """The group sums of x as it is."""
    _chk_all(x, groups)
    call("pxh_norm_groups", ptr(x), x.numel(), ptr(groups), _stream())


def axpy_norm(alpha, x, y, y_groups):
    """axpy that also leaves the group sums of y."""
    _chk_all(x, y, y_groups)
    call("pxh_axpy_norm", x.numel(), float(alpha), ptr(x), ptr(y), ptr(y_groups), _stream())


def shortcut_backward_norm(delta, from_delta, grad, grad_groups, activation="linear", alpha=1.0, beta=1.0,
                           pre_activation=None, first=False):
    """shortcut_backward / shortcut_backward_first that also leaves the group sums of grad."""
    _chk_all(delta, from_delta, grad, pre_activation, grad_groups)
    call("pxh_shortcut_backward_norm", ptr(delta), ptr(pre_activation), ptr(from_delta), ptr(grad), delta.numel(),
         float(alpha), float(beta), act_id(activation), int(bool(first)), ptr(grad_groups), _stream())


def rescale_clip_from_groups(x, groups, threshold=0.0, clip=0.0, norm_out=None):
    """rescale_clip that starts from the group sums the writer of x left instead of reading x for them."""
    _chk_all(x, groups, norm_out)
    call("pxh_rescale_clip_from_groups", ptr(x), x.numel(), float(threshold), float(clip), ptr(norm_out), ptr(groups),
         None, 0, _stream())


DETECTION_DTYPE = workloads.DETECTION_DTYPE


def yolo_detections(predictions, batch, masks, anchors, classes, width, height, net_width, net_height, threshold,
                    capacity, image_width=0, image_height=0):
    """Thresholded compaction of a decoded head.  Returns (records sorted into the reference's
    emission order as a numpy structured array, total number found)."""
    _chk_all(predictions)
    m = np.ascontiguousarray(masks, dtype=np.int32)
    a = np.ascontiguousarray(anchors, dtype=np.int32)
    out = torch.zeros((max(1, capacity), 8), device=predictions.device, dtype=torch.int32)
    count = torch.zeros(1, device=predictions.device, dtype=torch.int32)
    call("pxh_yolo_detections", ptr(predictions), batch, m.ctypes.data, len(m), a.ctypes.data, len(a) // 2, classes,
         width, height, net_width, net_height, int(image_width), int(image_height), float(threshold), ptr(out),
         int(capacity), ptr(count), _stream())
    torch.cuda.current_stream().synchronize()
    found = int(count.item())
    rec = out[:min(found, capacity)].cpu().numpy().view(DETECTION_DTYPE).reshape(-1)
    return rec[np.argsort(rec["order"], kind="stable")], found


def yolo_detections_append(predictions, batch, masks, anchors, classes, width, height, net_width, net_height,
                           threshold, order_base, records, count, image_width=0, image_height=0):
    """Adds the detections of one more head behind those already in `records` (an int32 tensor
    [capacity, 8] on the device); `count` is the device counter both heads share."""
    _chk_all(predictions)
    _chk(records, torch.int32, "records")
    _chk(count, torch.int32, "count")
    m = np.ascontiguousarray(masks, dtype=np.int32)
    a = np.ascontiguousarray(anchors, dtype=np.int32)
    call("pxh_yolo_detections_append", ptr(predictions), batch, m.ctypes.data, len(m), a.ctypes.data, len(a) // 2,
         classes, width, height, net_width, net_height, int(image_width), int(image_height), float(threshold),
         int(order_base), ptr(records), int(records.shape[0]), ptr(count), _stream())


def nms(records, count, batch, classes, threshold, workspace=None):
    """src/Box.cpp nms on device-resident records (int32 tensor [capacity, 8] viewed as detection
    records, device counter `count`).  Returns (kept records tensor, device counter of the kept)."""
    _chk(records, torch.int32, "records")
    _chk(count, torch.int32, "count")
    capacity = int(records.shape[0])
    kept = torch.empty_like(records)
    kept_count = torch.empty(1, device=records.device, dtype=torch.int32)
    ws_ptr, ws_bytes = (ptr(workspace), workspace.numel() * workspace.element_size()) if workspace is not None \
        else (None, 0)
    call("pxh_nms", ptr(records), ptr(count), capacity, int(batch), int(classes), float(threshold), ptr(kept),
         ptr(kept_count), ws_ptr, ws_bytes, _stream())
    return kept, kept_count


def nms_to_host(kept, kept_count):
    """Blocking copy of the survivors as a numpy structured array."""
    torch.cuda.current_stream().synchronize()
    n = int(kept_count.item())
    return kept[:n].cpu().numpy().view(DETECTION_DTYPE).reshape(-1)


def records_to_device(rec, capacity=None, device="cuda"):
    """numpy detection records -> (int32 tensor [capacity, 8], device counter)."""
    rec = np.ascontiguousarray(rec, DETECTION_DTYPE)
    capacity = max(1, len(rec)) if capacity is None else capacity
    t = torch.zeros((capacity, 8), dtype=torch.int32, device=device)
    if len(rec):
        t[:len(rec)] = torch.from_numpy(rec.view(np.int32).reshape(-1, 8)).to(device)
    count = torch.tensor([len(rec)], dtype=torch.int32, device=device)
    return t, count
