"""CPU-side checks of the C-ABI library: it loads, exports what include/pixienn_hip.h declares,
and rejects bad calls before anything is launched.  No compute, no GPU."""
import ctypes
import os
import re

import pytest

from pixienn_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols(path=("include", "pixienn_hip.h")):
    text = open(os.path.join(ROOT, *path)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pxh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(capi.LIB_PATH)
    names = header_symbols()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), "missing export: " + n
    # the Python binding covers the whole header, nothing more, nothing less
    assert sorted(names) == capi.declared_symbols()
    # the test hooks live in a private header, not in the installed one
    assert not [n for n in names if "debug" in n]
    hooks = header_symbols(("pixienn_amd", "csrc", "pixienn_hip_test.h"))
    assert hooks == capi.test_hook_symbols()
    for n in hooks:
        assert hasattr(lib, n), "missing test hook: " + n


def test_abi_version():
    assert capi.load().pxh_abi_version() == 2


def test_fastdiv_matches_integer_division():
    lib = capi.load()
    divisors = [1, 2, 3, 5, 7, 13, 19, 64, 85, 169, 255, 256, 361, 676, 1444, 4096, 5776, 92416, 369664, 2 ** 20 + 1,
                2 ** 30 - 1]
    for d in divisors:
        for n in [0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, 12345678, 2 ** 31 - 1, 2 ** 31 - d, 189267968]:
            if 0 <= n < 2 ** 31:
                assert lib.pxh_debug_fastdiv(n, d) == n // d, (n, d)
    import random
    r = random.Random(3)
    for _ in range(20000):
        d = r.randint(1, 2 ** 22)
        n = r.randint(0, 2 ** 31 - 1)
        assert lib.pxh_debug_fastdiv(n, d) == n // d, (n, d)


def test_rejects_bad_arguments_without_launching():
    inv = -1
    # dummy non-null addresses: validation happens before any device access
    p = 256
    assert capi.call_raw("pxh_activate", 0, None, 5, None) == inv
    assert capi.call_raw("pxh_activate", 99, p, 5, None) == inv
    assert "unknown activation" in capi.last_error()
    assert capi.call_raw("pxh_bn_infer_act_forward", p, p, None, p, p, p, p, 0, 3, 4, 0, None, 0, None) == inv
    assert capi.call_raw("pxh_bn_infer_act_forward", p, p, None, None, p, p, p, 1, 3, 4, 0, None, 0, None) == inv
    # the reference's maxpool constructor checks (include/MaxPoolLayer.h:57-59)
    assert capi.call_raw("pxh_maxpool_forward", p, p, p, 1, 1, 4, 4, 2, 2, 0, 2, 1, None) == inv
    assert "kernel must be positive" in capi.last_error()
    assert capi.call_raw("pxh_maxpool_forward", p, p, p, 1, 1, 4, 4, 2, 2, 2, 0, 1, None) == inv
    assert "stride must be positive" in capi.last_error()
    assert capi.call_raw("pxh_maxpool_forward", p, p, p, 1, 1, 4, 4, 2, 2, 2, 2, -1, None) == inv
    assert "padding cannot be negative" in capi.last_error()
    # the reference's shortcut checks (include/ShortcutLayer.h:123-124)
    assert capi.call_raw("pxh_shortcut", 1, 4, 4, 1, p, 2, 4, 1, 1.0, 1.0, p, None) == inv
    assert "equal in x and y" in capi.last_error()
    assert capi.call_raw("pxh_adam_update", 8, p, p, p, p, 0, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 0, None) == inv
    assert capi.call_raw("pxh_adam_update", 8, p, p, p, p, 1, 0, 1e-3, 0.9, 0.999, 1e-8, 0.0, 0, None) == inv
    assert capi.call_raw("pxh_upsample_strided", p, 4, 4, 2, 1, 2, 1, 1.0, None, p, 100, None) == inv
    assert "image stride" in capi.last_error()
    # tensors of 2^31 elements or more are refused, not mis-indexed
    assert capi.call_raw("pxh_bn_infer_act_forward", p, p, None, p, p, p, p, 1024, 1024, 4096, 0, None, 0, None) == -2
    with pytest.raises(capi.PxError):
        capi.call("pxh_activate", 0, None, 5, None)


def test_workspace_sizes():
    lib = capi.load()
    assert lib.pxh_bn_workspace_bytes(0, 1, 1) == 0
    small = lib.pxh_bn_workspace_bytes(16, 256, 361)
    big = lib.pxh_bn_workspace_bytes(16, 32, 608 * 608)
    assert 0 < small < big < (1 << 24)
    a256 = lambda b: (b + 255) // 256 * 256
    # the larger of the two forms of the training pass: sums of at most 2048 head workers and their 8 groups,
    # or the sums of one workgroup per head tile and one int per slot
    one = a256(2048 * 12 * 8) + a256(8 * 12 * 8)
    two = a256(64 * 3 * 23 * 12 * 8) + a256(64 * 3 * 5776 * 4)
    assert lib.pxh_yolo_workspace_bytes(64, 3, 80, 76, 76, 20) == max(one, two)
    assert lib.pxh_yolo_workspace_bytes(1, 1, 1, 1, 1, 0) == one
    assert lib.pxh_bn_folded_bytes(1024) == 1024 * 32 and lib.pxh_bn_folded_bytes(0) == 0


def test_ops_refuse_cpu_tensors():
    import torch
    from pixienn_amd import ops
    x = torch.zeros(1, 2, 4, 4)
    with pytest.raises(capi.PxError):
        ops.activate("leaky", x)


def test_a_missing_library_is_an_error_not_a_fallback(monkeypatch, tmp_path):
    """Nothing computes on the CPU in place of the kernels: without the built library every entry
    point of the binding raises, naming the file and how to build it."""
    monkeypatch.setattr(capi, "LIB_PATH", str(tmp_path / "libpixienn_hip.so"))
    monkeypatch.setattr(capi, "_lib", None)
    with pytest.raises(capi.PxError) as e:
        capi.load()
    assert "not built" in str(e.value) and "pixienn_amd.build" in str(e.value)
    with pytest.raises(capi.PxError):
        capi.call("pxh_abi_version")


def test_size_functions_and_argument_checks_need_no_device():
    """The pure size functions, and the argument checks that reject a call before anything is
    launched, work without a GPU (include/pixienn_hip.h: negative status = rejected before launch)."""
    import ctypes
    lib = capi.load()
    for n, want in ((0, 0), (1, 8), (256, 8), (257, 16), (8192, 256), (94_633_984, 94_633_984 // 256 * 8)):
        assert lib.pxh_norm_groups_bytes(n) == want
    assert lib.pxh_rescale_workspace_bytes() == 1024 * 16
    assert lib.pxh_bn_workspace_bytes(16, 256, 76 * 76) > 0
    # null pointers and impossible table shapes
    assert capi.call_raw("pxh_norm_groups", None, 1024, None, None) < 0
    assert "null" in capi.last_error()
    assert capi.call_raw("pxh_rescale_clip_from_groups", None, 1024, 1.0, 0.0, None, None, None, 0, None) < 0
    assert capi.call_raw("pxh_rescale_clip_from_groups", None, 0, 1.0, 0.0, None, None, None, 0, None) == 0      # empty: nothing to do
    assert capi.call_raw("pxh_shortcut_backward_norm", None, None, None, None, 16, 1.0, 1.0, 1, 0, None, None) < 0
    handle = ctypes.c_void_p()
    assert capi.call_raw("pxh_tensor_table_create", 3, 3, None, None, None, ctypes.byref(handle)) < 0
    assert capi.call_raw("pxh_tensor_table_create", 0, 4, None, None, None, ctypes.byref(handle)) == 0
    assert handle.value and lib.pxh_tensor_table_count(handle) == 0
    assert capi.call_raw("pxh_adam_update_table", handle, 16, 1, 1e-3, 0.9, 0.999, 1e-8, 5e-4, None) == 0      # nothing to do
    lib.pxh_tensor_table_destroy(handle)
    assert capi.call_raw("pxh_adam_update_table", None, 16, 1, 1e-3, 0.9, 0.999, 1e-8, 5e-4, None) < 0
