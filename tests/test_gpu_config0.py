"""The baseline's first configuration: the non-convolution layers of a YOLOv3-tiny inference forward
at batch 1, 3x416x416 (resources/models/yolov3-tiny.yml of the reference), GPU against the CPU
checker layer by layer.  The convolutions are out of scope: every conv result is a seeded N(0,1)
tensor of the real shape; pools, upsample, route and the heads consume what the layers before
them produced, so the whole chain of non-conv work runs at its real shapes, including the
stride-1 max-pool at 13x13 and the two 255-channel heads."""
import numpy as np
import pytest

from pixienn_amd import workloads as wl
from util import F, assert_bit_exact, assert_close, gpu, host

pytestmark = pytest.mark.gpu


def conv_epilogue(ops, oracle, layer, x_host, channels, size, bn=True, act="leaky"):
    """x_host: the synthetic conv result.  Returns (gpu output tensor, checker output)."""
    import torch
    want = x_host.copy()
    scale, bias, mean, var = wl.bn_params(2000 + layer, channels)
    if bn:
        oracle.conv_epilogue_forward(True, False, act, 1, channels, size, size, want, None, np.zeros(channels, F),
                                     np.zeros(channels, F), mean.copy(), var.copy(), scale, bias, None, None)
        y = torch.empty((1, channels, size, size), device="cuda")
        ops.bn_infer_act_forward(gpu(x_host), y, gpu(mean), gpu(var), gpu(scale), gpu(bias), act)
    else:
        oracle.conv_epilogue_forward(False, False, act, 1, channels, size, size, want, None, None, None, None, None,
                                     None, bias, None, None)
        y = torch.empty((1, channels, size, size), device="cuda")
        ops.bias_act_forward(gpu(x_host), y, gpu(bias), act)
    assert_close(host(y), want, 1e-5, 1e-3, "layer %d epilogue %dx%d^2" % (layer, channels, size))
    return y, want


def max_pool(ops, oracle, layer, y, want_in, channels, size, stride):
    import torch
    out_size = oracle.maxpool_out_dim(size, 2, stride, 1)
    out = torch.empty((1, channels, out_size, out_size), device="cuda")
    idx = torch.empty((1, channels, out_size, out_size), device="cuda", dtype=torch.int32)
    ops.maxpool_forward(y, out, idx, 2, stride, 1)
    # the checker pools what the GPU layer before produced, so that the comparison is bit for bit
    src = host(y)
    want = np.empty(out.shape, F); widx = np.empty(out.shape, np.int32)
    oracle.maxpool_forward(src, want, widx, 1, channels, size, size, out_size, out_size, 2, stride, 1)
    assert_bit_exact(host(out), want, "layer %d max-pool values" % layer)
    assert_bit_exact(host(idx), widx, "layer %d max-pool indexes" % layer)
    return out, out_size


def test_yolov3_tiny_inference_forward_non_conv_layers():
    import torch
    import oracle
    from pixienn_amd import ops
    oracle.lib()
    layer = 0
    size = 416
    y = None
    # conv(16) pool conv(32) pool conv(64) pool conv(128) pool conv(256) [route source] pool conv(512) pool(s1) conv(1024)
    route_source = None
    for channels in (16, 32, 64, 128, 256, 512):
        x = wl.normal(3000 + layer, (1, channels, size, size))
        y, want = conv_epilogue(ops, oracle, layer, x, channels, size)
        layer += 1
        if channels == 256:
            route_source = y
        stride = 1 if channels == 512 else 2
        y, size = max_pool(ops, oracle, layer, y, want, channels, size, stride)
        layer += 1
    assert size == 13
    x = wl.normal(3000 + layer, (1, 1024, 13, 13))
    y, _ = conv_epilogue(ops, oracle, layer, x, 1024, 13); layer += 1
    x = wl.normal(3000 + layer, (1, 256, 13, 13))
    y256, _ = conv_epilogue(ops, oracle, layer, x, 256, 13); layer += 1
    x = wl.normal(3000 + layer, (1, 512, 13, 13))
    conv_epilogue(ops, oracle, layer, x, 512, 13); layer += 1

    def head(layer, size, mask):
        logits_host = wl.normal(3000 + layer, (1, 255, size, size), std=2.0)
        logits, _ = conv_epilogue(ops, oracle, layer, logits_host, 255, size, bn=False, act="linear")
        cfg, keep = oracle.yolo_cfg(1, size, size, 80, mask, wl.TINY_ANCHORS, 416, 416)
        src = host(logits)
        want = np.zeros_like(src)
        oracle.yolo_decode(cfg, src, want)
        out = torch.empty_like(logits)
        ops.yolo_activate(logits, out, 1, 3, 80, size * size)
        assert_close(host(out), want, 1e-5, 1e-6, "head %d decode" % size)
        # and the detections that leave the device
        w_rec, w_found = oracle.yolo_detections(cfg, host(out), 0.5, 1 << 16)
        g_rec, g_found = ops.yolo_detections(out, 1, mask, wl.TINY_ANCHORS, 80, size, size, 416, 416, 0.5, 1 << 16)
        assert g_found == w_found > 0
        assert np.array_equal(g_rec["order"], w_rec["order"]) and np.array_equal(g_rec["prob"], w_rec["prob"])

    head(layer, 13, wl.TINY_MASKS[0]); layer += 2
    # route back to the 256x13^2 conv, 1x1 conv to 128, upsample to 26, concat with the 256x26^2 feature map
    x = wl.normal(3000 + layer, (1, 128, 13, 13))
    y128, _ = conv_epilogue(ops, oracle, layer, x, 128, 13); layer += 1
    up = torch.empty((1, 128, 26, 26), device="cuda")
    ops.upsample_forward(y128, up, 2, 1.0)
    want_up = np.empty((1, 128, 26, 26), F)
    oracle.upsample(host(y128), 13, 13, 128, 1, 2, True, 1.0, None, want_up)
    assert_bit_exact(host(up), want_up, "upsample 13 -> 26")
    layer += 1
    route = torch.empty((1, 384, 26, 26), device="cuda")
    ops.route_forward(up, route, 0)
    ops.route_forward(route_source, route, 128 * 26 * 26)
    want_route = np.empty((1, 384 * 26 * 26), F)
    oracle.route_forward(host(up).reshape(1, -1), want_route, 0)
    oracle.route_forward(host(route_source).reshape(1, -1), want_route, 128 * 26 * 26)
    assert_bit_exact(host(route).reshape(1, -1), want_route, "route concat")
    layer += 1
    x = wl.normal(3000 + layer, (1, 256, 26, 26))
    conv_epilogue(ops, oracle, layer, x, 256, 26); layer += 1
    head(layer, 26, wl.TINY_MASKS[1])
