"""ctypes binding of libpixienn_hip.so (the C ABI declared in include/pixienn_hip.h).

Device buffers are passed as integer addresses (e.g. torch.Tensor.data_ptr()); PyTorch is
only the allocator and stream provider.  There is no CPU fallback: a missing library or a
failed call raises PxError.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpixienn_hip.so")

ACTIVATIONS = {"leaky": 0, "linear": 1, "loggy": 2, "logistic": 3, "mish": 4,
               "relu": 5, "softplus": 6, "swish": 7, "tanh": 8}

P = ctypes.c_void_p
I = ctypes.c_int
F = ctypes.c_float
Z = ctypes.c_size_t
L = ctypes.c_longlong
U = ctypes.c_uint

# name -> argument types (every function returns int unless listed in _OTHER_RETURNS)
SIGNATURES = {
    "pxh_bn_infer_act_forward": [P, P, P, P, P, P, P, I, I, I, I, P, Z, P],
    "pxh_bn_fold": [P, P, P, P, I, P, P],
    "pxh_bn_folded_act_forward": [P, P, P, P, I, I, I, I, P],
    "pxh_bias_act_forward": [P, P, P, P, I, I, I, I, P],
    "pxh_bn_train_act_forward": [P, P, P, P, P, P, P, P, P, P, P, I, I, I, I, P, Z, P],
    "pxh_bn_train_act_forward_static": [P, P, P, P, P, P, P, P, P, P, P, I, I, I, I, P],
    "pxh_bn_train_act_shortcut_forward": [P, P, P, P, P, P, P, P, P, P, P, P, F, F, I, I, I, I, P, Z, P],
    "pxh_bn_folded_act_shortcut_forward": [P, P, P, P, P, F, F, I, I, I, I, P],
    "pxh_bn_folded_act_maxpool_forward": [P, P, P, P, I, I, I, I, I, P],
    "pxh_bn_stats": [P, P, P, I, I, I, P, Z, P],
    "pxh_bn_act_backward": [P, P, P, P, P, P, P, P, P, P, P, I, I, I, I, P, Z, P],
    "pxh_bias_act_backward": [P, P, P, I, I, I, I, P, Z, P],
    "pxh_bn_act_backward_clipped": [P, P, P, P, P, P, P, P, P, P, P, I, I, I, I, F, F, P, P, Z, P],
    "pxh_bias_act_backward_clipped": [P, P, P, I, I, I, I, F, F, P, P, Z, P],
    "pxh_activate": [I, P, Z, P],
    "pxh_gradient": [I, P, Z, P, P],
    "pxh_add_bias": [P, P, I, I, I, P],
    "pxh_backward_bias": [P, P, I, I, I, P, Z, P],
    "pxh_fill_f32": [P, Z, F, P],
    "pxh_fill_i32": [P, Z, I, P],
    "pxh_constrain": [I, F, P, P],
    "pxh_mul": [I, P, P, P],
    "pxh_axpy": [Z, F, P, P, P],
    "pxh_route_forward": [P, P, I, I, I, I, P],
    "pxh_route_backward": [P, P, I, I, I, I, P],
    "pxh_maxpool_forward": [P, P, P, I, I, I, I, I, I, I, I, I, P],
    "pxh_maxpool_backward": [P, P, P, I, I, I, I, I, I, I, I, I, P],
    "pxh_maxpool_backward_scatter": [P, P, P, I, P],
    "pxh_upsample": [P, I, I, I, I, I, I, F, P, P, P],
    "pxh_upsample_strided": [P, I, I, I, I, I, I, F, P, P, L, P],
    "pxh_shortcut": [I, I, I, I, P, I, I, I, F, F, P, P],
    "pxh_shortcut_forward": [P, P, P, P, Z, F, F, I, P],
    "pxh_shortcut_backward": [P, P, P, P, Z, F, F, I, P],
    "pxh_shortcut_backward_first": [P, P, P, P, Z, F, F, I, P],
    "pxh_yolo_activate": [P, P, I, I, I, I, P],
    "pxh_yolo_loss": [P, P, P, P, I, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, F, F, F, F, F, F, P, Z, P],
    "pxh_yolo_forward_train": [P, P, P, P, P, I, P, P, P, P, I, I, I, I, I, I, I, I, F, F, F, F, F, F, P, Z, P],
    "pxh_yolo_forward_train_heads": [I, P, P, P, I, P, I, I, I, I, I, P, Z, P],
    "pxh_sgd_update": [Z, P, P, I, F, F, F, I, P],
    "pxh_rescale_clip": [P, Z, F, F, P, P, Z, P],
    "pxh_norm_groups": [P, Z, P, P],
    "pxh_axpy_norm": [Z, F, P, P, P, P],
    "pxh_shortcut_backward_norm": [P, P, P, P, Z, F, F, I, I, P, P],
    "pxh_rescale_clip_from_groups": [P, Z, F, F, P, P, P, Z, P],
    "pxh_shortcut_backward_clipped": [P, P, P, P, Z, F, F, I, I, F, F, P, P, Z, P],
    "pxh_yolo_detections": [P, I, P, I, P, I, I, I, I, I, I, I, I, F, P, I, P, P],
    "pxh_yolo_detections_append": [P, I, P, I, P, I, I, I, I, I, I, I, I, F, U, P, I, P, P],
    "pxh_nms": [P, P, I, I, I, F, P, P, P, Z, P],
    "pxh_adam": [I, P, P, P, F, F, F, F, I, P],
    "pxh_adam_update": [Z, P, P, P, P, I, I, F, F, F, F, F, I, P],
    "pxh_adam_update_multi": [I, P, P, P, P, P, P, I, I, F, F, F, F, F, P],
    "pxh_rescale_clip_multi": [I, P, P, F, F, P, P, Z, P],
    "pxh_fill_f32_multi": [I, P, P, F, P],
    "pxh_sgd_update_multi": [I, P, P, P, P, I, F, F, F, P],
    "pxh_tensor_table_create": [I, I, P, P, P, P],
    "pxh_tensor_table_count": [P],
    "pxh_adam_update_table": [P, I, I, F, F, F, F, F, P],
    "pxh_sgd_update_table": [P, I, F, F, F, P],
    "pxh_fill_f32_table": [P, F, P],
    "pxh_rescale_clip_table": [P, F, F, P, P],
}
_OTHER_RETURNS = {
    "pxh_last_error": (ctypes.c_char_p, []),
    "pxh_abi_version": (I, []),
    "pxh_bn_workspace_bytes": (Z, [I, I, I]),
    "pxh_bn_folded_bytes": (Z, [I]),
    "pxh_bn_clipped_workspace_bytes": (Z, [I, I, I]),
    "pxh_rescale_workspace_bytes": (Z, []),
    "pxh_norm_groups_bytes": (Z, [Z]),
    "pxh_rescale_multi_workspace_bytes": (Z, []),
    "pxh_yolo_workspace_bytes": (Z, [I, I, I, I, I, I]),
    "pxh_yolo_heads_workspace_bytes": (Z, [I, P, I]),
    "pxh_nms_workspace_bytes": (Z, [I]),
    "pxh_reserve_workspace": (I, [Z]),
    "pxh_tensor_table_destroy": (None, [P]),
}
# test hooks (pixienn_amd/csrc/pixienn_hip_test.h): exported, but not part of the C ABI
_TEST_HOOKS = {
    "pxh_debug_fastdiv": (ctypes.c_uint, [ctypes.c_uint, ctypes.c_uint]),
    "pxh_debug_nms_sweeps": (I, [I]),
    "pxh_debug_library_workspace": (P, [Z]),
    "pxh_debug_yolo_tuning": (I, [I, I, I]),
    "pxh_debug_stream_mix": (I, [I, I, Z, P, P, P]),
}


class YoloHead(ctypes.Structure):
    """pxh_yolo_head of include/pixienn_hip.h."""
    _fields_ = [("input", P), ("output", P), ("delta", P), ("masks", P), ("mask_count", I), ("width", I), ("height", I),
                ("ignore_thresh", F), ("truth_thresh", F), ("coord_scale", F), ("object_scale", F),
                ("noobject_scale", F), ("class_scale", F), ("stats", P), ("cost", P)]


class PxError(RuntimeError):
    """Raised for a rejected or failed kernel call (the host-side px::Error counterpart)."""


_lib = None


def load():
    """Loads the built library; raises PxError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise PxError("libpixienn_hip.so is not built (%s); run `python -m pixienn_amd.build` "
                      "or __graft_entry__.build()" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = I
    for name, (res, args) in list(_OTHER_RETURNS.items()) + list(_TEST_HOOKS.items()):
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = res
    _lib = lib
    return lib


def declared_symbols():
    """The C ABI proper (include/pixienn_hip.h)."""
    return sorted(list(SIGNATURES) + list(_OTHER_RETURNS))


def test_hook_symbols():
    return sorted(_TEST_HOOKS)


def last_error():
    return load().pxh_last_error().decode("utf-8", "replace")


def ptr(t):
    """Device address of a torch tensor (None -> NULL)."""
    if t is None:
        return None
    if isinstance(t, int):
        return t
    return t.data_ptr()


def act_id(act):
    return ACTIVATIONS[act] if isinstance(act, str) else int(act)


def call(name, *args):
    """Calls an int-returning entry point and raises PxError on a non-zero status."""
    rc = getattr(load(), name)(*args)
    if rc != 0:
        raise PxError("%s failed (status %d): %s" % (name, rc, last_error()))
    return rc


def call_raw(name, *args):
    """Calls an entry point and returns its status without raising."""
    return getattr(load(), name)(*args)
