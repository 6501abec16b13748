"""Runs the C++ test of the host mirror (tiny-cnn_amd/host/tiny_dnn_hip.h) on the GPU.

tests/host_cpp/test_host.cpp re-states the reference's own tests for this path
(test/test_convolutional_layer.h:133-200, test/test_fully_connected_layer.h:48-64,
test/test_max_pooling_layer.h:25-39,85-110,251-281, test/test_optimizers.h:15-190) against the
mirrored class names and checks random cases and network<sequential>::fit against the CPU oracle,
tolerance 1e-4 relative (max-pool exact). The binary is built beforehand by
`make -C tests/host_cpp` (done by __graft_entry__.build()). The file name sorts after the other
GPU tests: the binary is a child process, and `pytest -x` should not let its failure hide them.
"""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "host_cpp", "build", "test_host")


@pytest.mark.gpu
def test_host_mirror_cpp():
    assert os.path.exists(BIN), "tests/host_cpp/build/test_host has not been built"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=100)
    print(r.stdout[-4000:], r.stderr[-2000:], flush=True)
    assert r.returncode == 0, r.stdout[-2000:]
    assert " 0 failed" in r.stdout
