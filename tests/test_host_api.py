"""Runs the C++ test program of the arm_compute-compatible host layer (tests/cpp/test_host_api.cpp)."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "test_host_api")


def _run(mode):
    if not os.path.exists(BIN):
        subprocess.check_call(["make", "-s", "-C", os.path.join(HERE, "cpp")])
    r = subprocess.run([BIN, mode], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(r.stdout)
    assert r.returncode == 0, r.stdout[-3000:]
    assert " 0 failures" in r.stdout


def test_host_layer_cpu_side():
    """validate() accept/reject tables, TensorInfo layout, quantization helpers: no GPU involved."""
    _run("--cpu")


@pytest.mark.gpu
def test_host_layer_on_device():
    """NEGEMMLowpMatrixMultiplyCore / NEGEMMLowpOutputStage / NEGEMMConvolutionLayer against the oracle, tolerance 0."""
    _run("--gpu")
