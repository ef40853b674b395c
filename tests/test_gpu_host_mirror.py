"""Runs the C++ device test of the host mirror (tests/host/test_host_backend.cpp).

The binary is built by __graft_entry__.build() (tests/host/Makefile); it links libargus_hip.so and
the CPU oracle and uses no torch, so it also shows the library standing on the ROCm runtime alone.
"""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "host", "test_host_backend")


def test_host_mirror_binary_is_built():
    assert os.path.exists(BIN), "run __graft_entry__.build() (make -C tests/host)"


def test_host_mirror_reports_missing_device_cleanly():
    import torch
    if torch.cuda.is_available():
        pytest.skip("device present")
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=60)
    assert r.returncode == 77 and "no HIP device" in r.stdout


@pytest.mark.gpu
def test_host_mirror_on_device():
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(r.stdout[-3000:], r.stderr[-2000:], flush=True)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "ALL PASS" in r.stdout
