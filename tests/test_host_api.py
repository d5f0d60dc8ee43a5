"""Runs the C++ test program of the arm_compute-compatible host layer (tests/cpp/test_host_api.cpp), one pytest case per
case of the program, each in a process of its own."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CPP = os.path.join(HERE, "cpp")
BIN = os.path.join(CPP, "test_host_api")

# the names the program lists (test_case_lists_match_the_program holds the two in step)
CPU_CASES = ["tensor_info", "quant_helpers", "validate_tables", "fully_connected_validate", "gemm_conv2d_validate",
             "error_paths"]
GPU_CASES = ["gemmlowp_fused_u8_host", "gemmlowp_fused_u8_device", "gemmlowp_s32_batched", "reference_small_datasets",
             "gemmlowp_accumulate_and_3d", "gemmlowp_dynamic_qinfo", "gemmlowp_per_channel_and_update", "gemmlowp_f32",
             "output_stage", "quantize_down_scale", "convolution_s8_per_channel_64", "convolution_s8_relu_16",
             "convolution_u8_6", "convolution_u8_per_channel_bounded_relu_32", "convolution_s8_per_channel_32_variant1",
             "convolution_u8_relu_6_variant1", "convolution_s8_per_channel_16_variant2", "convolution_u8_6_variant2",
             "gemm_conv2d", "stateless_operator", "stateless_operators_padded_after_configure",
             "convolution_nchw_and_stateless", "convolution_f32_destination", "fully_connected_s8_after_fc",
             "fully_connected_u8_after_fc", "fully_connected_s8_after_conv_nhwc", "fully_connected_u8_after_conv_nchw",
             "fully_connected_s8_weights_reshaped"]


@pytest.fixture(scope="session")
def program():
    """The test program, brought up to date by its Makefile (which knows what it is built from): a stale binary would
    test old code."""
    r = subprocess.run(["make", "-s", "-C", CPP], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, "building tests/cpp/test_host_api failed:\n" + r.stdout[-3000:]
    assert os.path.exists(BIN)
    return BIN


def _run(program, *args):
    r = subprocess.run([program, *args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(r.stdout)
    assert r.returncode == 0, r.stdout[-3000:]
    return r.stdout


def test_case_lists_match_the_program(program):
    assert _run(program, "--list-cpu").split() == CPU_CASES
    assert _run(program, "--list-gpu").split() == GPU_CASES


@pytest.mark.parametrize("case", CPU_CASES)
def test_host_layer_cpu_side(program, case):
    """validate() accept/reject tables, TensorInfo layout, quantization helpers: no GPU involved."""
    assert " 0 failures" in _run(program, "--case", case)


@pytest.mark.gpu
@pytest.mark.parametrize("case", GPU_CASES)
def test_host_layer_on_device(program, case):
    """The function classes of the host layer against the oracle on the device, tolerance 0."""
    assert " 0 failures" in _run(program, "--case", case)
