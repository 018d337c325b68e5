"""Runs the C++ host-mirror test program (tests/host/host_test.cpp): the reference's operator interface
(Foundry, TensorBindings, KvPrepFusedStep, FlashAttentionStep, MetalError) re-stated in C++ over the C ABI."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "host", "host_test")


def binary():
    if not os.path.exists(BIN):  # normally built beforehand by __graft_entry__.build()
        subprocess.check_call(["make", "-s", "-C", os.path.join(HERE, "host")])
    return BIN


def test_host_logic_without_gpu():
    out = subprocess.run([binary(), "--cpu"], capture_output=True, text=True, timeout=60)
    print(out.stdout)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "0 failed checks" in out.stdout


@pytest.mark.gpu
def test_host_mirror_steps_on_gpu():
    print("[case] C++ host mirror", flush=True)
    out = subprocess.run([binary()], capture_output=True, text=True, timeout=110)
    print(out.stdout)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "0 failed checks" in out.stdout
