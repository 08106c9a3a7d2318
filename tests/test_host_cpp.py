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
