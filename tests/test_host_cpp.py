"""The C++ layer interface (pixienn_amd/host) through its harness binary, tests/host/host_check:
a small network of every layer kind, forward, backward and update, each layer checked against
the CPU checker on the inputs the GPU layer saw."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HARNESS = os.path.join(ROOT, "tests", "host", "host_check")


def harness():
    if not os.path.exists(HARNESS):
        import __graft_entry__
        __graft_entry__.build()
    return HARNESS


def run(*args):
    proc = subprocess.run([harness()] + list(args), capture_output=True, text=True, timeout=100)
    print(proc.stdout)
    print(proc.stderr)
    return proc


def test_host_interface_rejects_bad_layers_without_a_device():
    proc = run("--cpu")
    assert proc.returncode == 0, proc.stdout
    assert "0 failed" in proc.stdout
    assert "maxpool rejects kernel 0" in proc.stdout


@pytest.mark.gpu
def test_host_interface_network_forward_backward_update():
    proc = run()
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "0 failed" in proc.stdout
    assert proc.stdout.count(" ok ") >= 40


def test_reference_side_bindings_compile_against_the_engine_interface():
    """docs/reference_patch/include/hip/*.h -- the Device::HIP specialisations a maintainer adds to the
    engine, one per layer -- compiled (g++ -fsyntax-only) against tests/host/reference_stub.h, which
    declares the engine's classes with the member names of the reference: every body names only
    members the engine has and calls the library with arguments of the declared types."""
    src = os.path.join(ROOT, "tests", "host", "patch_check.cpp")
    proc = subprocess.run(["g++", "-std=c++20", "-fsyntax-only", "-Wall", "-Wextra", "-Wno-unused-parameter",
                           "-I" + os.path.join(ROOT, "include"),
                           "-I" + os.path.join(ROOT, "docs", "reference_patch", "include"), src],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr
    assert "warning" not in proc.stderr, proc.stderr
    patch = os.path.join(ROOT, "docs", "reference_patch", "include", "hip")
    names = sorted(os.listdir(patch))
    for layer in ("ConvLayer", "BatchNormLayer", "MaxPoolLayer", "UpsampleLayer", "ShortcutLayer", "RouteLayer",
                  "YoloLayer"):
        assert layer + ".h" in names
    text = open(src).read()
    for name in names:
        assert '#include "hip/%s"' % name in text, "%s is not compiled by the check" % name
