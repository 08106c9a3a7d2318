"""ctypes front-end of the CPU checker (oracle/px_oracle.c).

TEST INFRASTRUCTURE ONLY.  Import this from tests/, from __graft_entry__.smoke()
and from bench.py's cpu_baseline leg; the product package never does.

All array arguments are C-contiguous numpy arrays (float32 / int32) that the C
code reads or updates in place.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_activation.so")

ACTIVATIONS = {"leaky": 0, "linear": 1, "loggy": 2, "logistic": 3, "mish": 4,
               "relu": 5, "softplus": 6, "swish": 7, "tanh": 8}

_f32p = ctypes.POINTER(ctypes.c_float)
_i32p = ctypes.POINTER(ctypes.c_int)
_c_int, _c_float, _c_size = ctypes.c_int, ctypes.c_float, ctypes.c_size_t


def build(force=False):
    """Compile liboracle.so (and oracle/_ref when the reference tree is present)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "all"] + (["-B"] if force else []))
    return _LIB_PATH


class YoloCfg(ctypes.Structure):
    _fields_ = [("batch", _c_int), ("width", _c_int), ("height", _c_int), ("classes", _c_int),
                ("num_masks", _c_int), ("num_anchors", _c_int),
                ("mask", _i32p), ("anchors", _i32p),
                ("net_width", _c_int), ("net_height", _c_int),
                ("ignore_thresh", _c_float), ("truth_thresh", _c_float),
                ("coord_scale", _c_float), ("object_scale", _c_float),
                ("noobject_scale", _c_float), ("class_scale", _c_float)]


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.pxo_act_apply.restype = _c_float
        L.pxo_act_apply.argtypes = [_c_int, _c_float]
        L.pxo_act_gradient.restype = _c_float
        L.pxo_act_gradient.argtypes = [_c_int, _c_float]
        L.pxo_sum_array.restype = _c_float
        L.pxo_mag_array.restype = _c_float
        L.pxo_box_intersection.restype = _c_float
        L.pxo_box_union.restype = _c_float
        L.pxo_box_iou.restype = _c_float
        _lib = L
    return _lib


def ref_lib():
    """The reference's own Activation.h, compiled; None when it was never built."""
    global _ref
    if _ref is None and os.path.exists(_REF_PATH):
        _ref = ctypes.CDLL(_REF_PATH)
    return _ref


def _f(a):
    assert a is None or (a.dtype == np.float32 and a.flags.c_contiguous), "float32 C-contiguous array expected"
    return None if a is None else a.ctypes.data_as(_f32p)


def _i(a):
    assert a is None or (a.dtype == np.int32 and a.flags.c_contiguous), "int32 C-contiguous array expected"
    return None if a is None else a.ctypes.data_as(_i32p)


def act_id(act):
    return ACTIVATIONS[act] if isinstance(act, str) else int(act)


# ---------------- activations ----------------
def activate(act, x):
    lib().pxo_activate(act_id(act), _f(x), _c_size(x.size))
    return x


def gradient(act, x, delta):
    lib().pxo_gradient(act_id(act), _f(x), _c_size(x.size), _f(delta))
    return delta


def ref_activate(act, x):
    rc = ref_lib().ref_activate(act_id(act), _f(x), _c_size(x.size))
    assert rc == 0
    return x


def ref_gradient(act, x, delta):
    rc = ref_lib().ref_gradient(act_id(act), _f(x), _c_size(x.size), _f(delta))
    assert rc == 0
    return delta


# ---------------- per-channel primitives ----------------
def add_bias(out, bias, batch, n, size):
    lib().pxo_add_bias(_f(out), _f(bias), batch, n, size)


def backward_bias(bias_updates, delta, batch, n, size):
    lib().pxo_backward_bias(_f(bias_updates), _f(delta), batch, n, size)


def backward_scale(xnorm, delta, batch, n, size, scale_updates):
    lib().pxo_backward_scale(_f(xnorm), _f(delta), batch, n, size, _f(scale_updates))


def sum_array(a):
    return float(lib().pxo_sum_array(_f(a), int(a.size)))


def mag_array(a):
    return float(lib().pxo_mag_array(_f(a), _c_size(a.size)))


def mean(x, batch, filters, spatial, out):
    lib().pxo_mean(_f(x), batch, filters, spatial, _f(out))


def variance(x, mean_, batch, filters, spatial, out):
    lib().pxo_variance(_f(x), _f(mean_), batch, filters, spatial, _f(out))


def normalize(x, mean_, var, batch, filters, spatial):
    lib().pxo_normalize(_f(x), _f(mean_), _f(var), batch, filters, spatial)


def scale_bias(out, scales, batch, n, size):
    lib().pxo_scale_bias(_f(out), _f(scales), batch, n, size)


def mean_delta(delta, var, batch, filters, spatial, out):
    lib().pxo_mean_delta(_f(delta), _f(var), batch, filters, spatial, _f(out))


def variance_delta(x, delta, mean_, var, batch, filters, spatial, out):
    lib().pxo_variance_delta(_f(x), _f(delta), _f(mean_), _f(var), batch, filters, spatial, _f(out))


def normalize_delta(x, mean_, var, mean_delta_, var_delta, batch, filters, spatial, delta):
    lib().pxo_normalize_delta(_f(x), _f(mean_), _f(var), _f(mean_delta_), _f(var_delta),
                              batch, filters, spatial, _f(delta))


def constrain(alpha, x):
    lib().pxo_constrain(int(x.size), _c_float(alpha), _f(x))


# ---------------- batch norm / epilogue ----------------
def batchnorm_forward(training, batch, channels, height, width, input, output, mean_, var,
                      rolling_mean, rolling_var, scales, biases, x, xnorm, wide=False):
    lib().pxo_batchnorm_forward(int(training), batch, channels, height, width, _f(input), _f(output),
                                _f(mean_), _f(var), _f(rolling_mean), _f(rolling_var), _f(scales),
                                _f(biases), _f(x), _f(xnorm), int(wide))


def batchnorm_backward(batch, channels, height, width, delta, mean_, var, mean_delta_, var_delta,
                       scales, scale_updates, bias_updates, x, xnorm, wide=False):
    lib().pxo_batchnorm_backward(batch, channels, height, width, _f(delta), _f(mean_), _f(var),
                                 _f(mean_delta_), _f(var_delta), _f(scales), _f(scale_updates),
                                 _f(bias_updates), _f(x), _f(xnorm), int(wide))


def conv_epilogue_forward(batch_normalize, training, act, batch, channels, height, width, output,
                          pre_activation, mean_, var, rolling_mean, rolling_var, scales, biases,
                          x, xnorm, wide=False):
    lib().pxo_conv_epilogue_forward(int(batch_normalize), int(training), act_id(act), batch, channels,
                                    height, width, _f(output), _f(pre_activation), _f(mean_), _f(var),
                                    _f(rolling_mean), _f(rolling_var), _f(scales), _f(biases), _f(x),
                                    _f(xnorm), int(wide))


def conv_epilogue_backward(batch_normalize, act, batch, channels, height, width, delta, pre_activation,
                           mean_, var, mean_delta_, var_delta, scales, scale_updates, bias_updates,
                           x, xnorm, wide=False):
    lib().pxo_conv_epilogue_backward(int(batch_normalize), act_id(act), batch, channels, height, width,
                                     _f(delta), _f(pre_activation), _f(mean_), _f(var), _f(mean_delta_),
                                     _f(var_delta), _f(scales), _f(scale_updates), _f(bias_updates),
                                     _f(x), _f(xnorm), int(wide))


# ---------------- data-movement layers ----------------
def maxpool_out_dim(n, kernel, stride, padding):
    return int(lib().pxo_maxpool_out_dim(n, kernel, stride, padding))


def maxpool_forward(inp, out, indexes, batch, channels, ih, iw, oh, ow, kernel, stride, padding):
    lib().pxo_maxpool_forward(_f(inp), _f(out), _i(indexes), batch, channels, ih, iw, oh, ow,
                              kernel, stride, padding)


def maxpool_backward(delta, indexes, grad):
    lib().pxo_maxpool_backward(_f(delta), _i(indexes), _f(grad), _c_size(delta.size))


def upsample(inp, w, h, c, batch, stride, forward, scale, acc, out):
    lib().pxo_upsample(_f(inp), w, h, c, batch, stride, int(forward), _c_float(scale), _f(acc), _f(out))


def shortcut(batch, w1, h1, c1, add, w2, h2, c2, s1, s2, out):
    return int(lib().pxo_shortcut(batch, w1, h1, c1, _f(add), w2, h2, c2, _c_float(s1), _c_float(s2), _f(out)))


def shortcut_forward(act, batch, w, h, c, inp, from_output, alpha, beta, output, pre_activation):
    lib().pxo_shortcut_forward(act_id(act), batch, w, h, c, _f(inp), _f(from_output), _c_float(alpha),
                               _c_float(beta), _f(output), _f(pre_activation))


def shortcut_backward(act, batch, w, h, c, delta, pre_activation, from_delta, grad, alpha, beta):
    lib().pxo_shortcut_backward(act_id(act), batch, w, h, c, _f(delta), _f(pre_activation), _f(from_delta),
                                _f(grad), _c_float(alpha), _c_float(beta))


def axpy(alpha, x, y):
    lib().pxo_axpy(_c_size(x.size), _c_float(alpha), _f(x), _f(y))


def route_forward(layer_output, route_output, offset):
    batch = layer_output.shape[0]
    lib().pxo_route_forward(_f(layer_output), _f(route_output), batch, layer_output.size // batch,
                            route_output.size // batch, int(offset))


def route_backward(route_delta, layer_delta, offset):
    batch = layer_delta.shape[0]
    lib().pxo_route_backward(_f(route_delta), _f(layer_delta), batch, layer_delta.size // batch,
                             route_delta.size // batch, int(offset))


# ---------------- boxes / YOLO ----------------
def _box(b):
    return (ctypes.c_float * 4)(*[float(v) for v in b])


def box_intersection(a, b):
    return float(lib().pxo_box_intersection(_box(a), _box(b)))


def box_union(a, b):
    return float(lib().pxo_box_union(_box(a), _box(b)))


def box_iou(a, b):
    return float(lib().pxo_box_iou(_box(a), _box(b)))


def yolo_cfg(batch, width, height, classes, mask, anchors, net_width, net_height,
             ignore_thresh=0.5, truth_thresh=1.0, coord_scale=1.0, object_scale=1.0,
             noobject_scale=1.0, class_scale=1.0):
    """Returns (cfg, keepalive); keep the tuple alive while cfg is in use."""
    mask_a = np.ascontiguousarray(mask, dtype=np.int32)
    anch_a = np.ascontiguousarray(anchors, dtype=np.int32)
    cfg = YoloCfg(batch, width, height, classes, len(mask_a), len(anch_a) // 2, _i(mask_a), _i(anch_a),
                  net_width, net_height, ignore_thresh, truth_thresh, coord_scale, object_scale,
                  noobject_scale, class_scale)
    return cfg, (mask_a, anch_a)


def yolo_decode(cfg, inp, out):
    lib().pxo_yolo_decode(ctypes.byref(cfg), _f(inp), _f(out))


def yolo_forward(cfg, inp, truths, truth_counts, max_truth, output, delta):
    """Returns (cost, stats[12])."""
    cost = np.zeros(1, np.float32)
    stats = np.zeros(12, np.float32)
    lib().pxo_yolo_forward(ctypes.byref(cfg), _f(inp), _f(truths), _i(truth_counts), int(max_truth),
                           _f(output), _f(delta), _f(cost), _f(stats))
    return float(cost[0]), stats


def yolo_build_targets(cfg, truths, count, classes, anchors, boxes):
    return int(lib().pxo_yolo_build_targets(ctypes.byref(cfg), _f(truths), int(count), _i(classes),
                                            _i(anchors), _f(boxes)))


# ---------------- Adam ----------------
def adam_update(w, d, m, v, batch, t, lr, beta1, beta2, eps, decay, apply_decay):
    lib().pxo_adam_update(_c_size(w.size), _f(w), _f(d), _f(m), _f(v), int(batch), int(t), _c_float(lr),
                          _c_float(beta1), _c_float(beta2), _c_float(eps), _c_float(decay), int(apply_decay))


# ---------------- SGD / gradient rescale ----------------
def sgd_update(w, d, batch, lr, momentum, decay, apply_decay):
    lib().pxo_sgd_update(_c_size(w.size), _f(w), _f(d), int(batch), _c_float(lr), _c_float(momentum),
                         _c_float(decay), int(apply_decay))


def rescale_clip(x, threshold, clip):
    fn = lib().pxo_rescale_clip
    fn.restype = _c_float
    return float(fn(_f(x), _c_size(x.size), _c_float(threshold), _c_float(clip)))


# ---------------- detections ----------------
DETECTION_DTYPE = np.dtype([("x", "f4"), ("y", "f4"), ("w", "f4"), ("h", "f4"), ("prob", "f4"), ("batch", "i4"),
                            ("class_index", "i4"), ("order", "u4")])


def nms(records, threshold):
    """src/Box.cpp nms on an array of DETECTION_DTYPE records (their sequence is the input order)."""
    records = np.ascontiguousarray(records, DETECTION_DTYPE)
    out = np.zeros(max(1, len(records)), DETECTION_DTYPE)
    fn = lib().pxo_nms
    fn.restype = _c_int
    kept = fn(records.ctypes.data_as(ctypes.c_void_p), int(len(records)), _c_float(threshold),
              out.ctypes.data_as(ctypes.c_void_p))
    return out[:kept]


def yolo_detections(cfg, predictions, threshold, capacity, image_width=0, image_height=0):
    """Returns (records in the reference's emission order, total number found)."""
    out = np.zeros(max(1, capacity), DETECTION_DTYPE)
    fn = lib().pxo_yolo_detections
    fn.restype = _c_int
    found = fn(ctypes.byref(cfg), _f(predictions), _c_float(threshold), int(image_width), int(image_height),
               out.ctypes.data_as(ctypes.c_void_p), int(capacity))
    return out[:min(found, capacity)], int(found)
