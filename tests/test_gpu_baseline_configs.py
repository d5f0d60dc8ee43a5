"""The five BASELINE configurations at their full sizes, through the C ABI with device-resident operands.

Where the scalar oracle would take minutes, the comparison is against the SIMD CPU baseline (itself pinned bit-for-bit to
the scalar oracle in test_oracle_fast.py) plus a slice checked against the scalar oracle directly; the F32 case is
checked on every output against an exact double-precision product (pinned to the scalar oracle on a row subset)."""
import numpy as np
import pytest

import oracle
from computelibrary_amd import capi
from gpu_util import announce, run_gemm, to_dev
from test_gpu_conv import run_conv

pytestmark = pytest.mark.gpu


def synth_llm(M, N, K, seed):
    rng = np.random.default_rng(seed)
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = np.clip(np.rint(rng.normal(0.0, 32.0, size=(K, N))), -127, 127).astype(np.int8)
    scales = rng.uniform(1e-4, 1e-3, size=N).astype(np.float32)
    mult, shift = oracle.calculate_quantized_multipliers(1.0, scales, 1.0)
    bias = np.rint(rng.normal(0.0, 2000.0, size=N)).astype(np.int32)
    return A, B, bias, mult, shift


def test_config1_qasymm8_256_cubed_both_zero_point_conventions():
    rng = np.random.default_rng(1)
    A = rng.integers(0, 256, size=(256, 256), dtype=np.uint8)
    B = rng.integers(0, 256, size=(256, 256), dtype=np.uint8)
    bias = rng.integers(-1000, 1001, size=256, dtype=np.int32)
    for ao, bo in [(-128, -127), (128, 127)]:
        want = oracle.gemmlowp_fixedpoint(A, B, bias, ao, bo, [1518500250], [8], 10, 0, 255, np.uint8)
        for device in (True, False):
            announce("config1", ao, bo, "device", device)
            got, name = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.uint8, ao, bo, bias, [1518500250], [8], 10, 0, 255,
                                 device=device)
            np.testing.assert_array_equal(got, want)
        # the two-function form of examples/neon_gemm_qasymm8.cpp: S32 GEMM, then the stand-alone output stage
        t, _ = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, device=True)
        out = np.zeros((256, 256), np.uint8)
        capi.output_stage(np.ascontiguousarray(t), bias, out, capi.requant(1518500250, 8, 10, 0, 255))
        np.testing.assert_array_equal(out, want)


def test_config2_llm_projection_2048x4096x4096():
    M, N, K = 2048, 4096, 4096
    A, B, bias, mult, shift = synth_llm(M, N, K, 2)
    fg = oracle.FastGemm(B)
    want = fg.run(A, bias, -3, 0, mult, shift, -5, -128, 127, np.int8)
    fg.close()
    rows = [0, 1, 777, 2047]
    np.testing.assert_array_equal(
        want[rows], oracle.gemmlowp_fixedpoint(A[rows], B, bias, -3, 0, mult, shift, -5, -128, 127, np.int8))
    announce("config2")
    got, name = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.int8, -3, 0, bias, mult, shift, -5, -128, 127, device=True)
    assert name.startswith("pp_"), name
    np.testing.assert_array_equal(got, want)
    inside = ((want > -128) & (want < 127)).mean()
    assert inside > 0.3  # most outputs are not clamped: the comparison is meaningful


def test_config3_decode_skinny_8x11008x4096():
    M, N, K = 8, 11008, 4096
    A, B, bias, mult, shift = synth_llm(M, N, K, 3)
    want = oracle.gemmlowp_fixedpoint(A, B, bias, -3, 0, mult, shift, -5, -128, 127, np.int8)
    announce("config3")
    got, name = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.int8, -3, 0, bias, mult, shift, -5, -128, 127, device=True)
    assert name.startswith("skinny"), name
    np.testing.assert_array_equal(got, want)
    got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.int8, -3, 0, bias, mult, shift, -5, -128, 127, device=True,
                      path=capi.PATH_MFMA)
    np.testing.assert_array_equal(got, want)


def test_config4_conv_nhwc_32x56x56x64_3x3():
    rng = np.random.default_rng(4)
    src = rng.integers(-128, 128, size=(32, 56, 56, 64), dtype=np.int8)
    w = np.clip(np.rint(rng.normal(0.0, 24.0, size=(64, 3, 3, 64))), -127, 127).astype(np.int8)
    bias = np.rint(rng.normal(0.0, 500.0, size=64)).astype(np.int32)
    mult, shift = oracle.calculate_quantized_multipliers(1.0, rng.uniform(1e-4, 1e-3, size=64).astype(np.float32), 1.0)
    # reference lowering on the CPU: im2col (pad = zero point -1) + flattened weights + SIMD GEMM with offset +1
    cols = oracle.im2col_nhwc(src, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), -1)
    fg = oracle.FastGemm(oracle.weights_reshape(w))
    want = fg.run(cols, bias, 1, 0, mult, shift, -5, -128, 127, np.int8).reshape(32, 56, 56, 64)
    fg.close()
    np.testing.assert_array_equal(
        want[:1, :3], oracle.conv_nhwc_direct(src[:1, :4], w, bias, -1, 0, mult, shift, -5, -128, 127, (1, 1),
                                              (1, 1, 1, 0))[:, :3])
    announce("config4 implicit")
    got, name = run_conv(src, w, bias, -1, 0, mult, shift, -5, -128, 127, (1, 1), (1, 1, 1, 1))
    assert name == "implicit_band_32x64", name  # (an image this large: bands of input rows staged in LDS)
    np.testing.assert_array_equal(got, want)
    announce("config4 explicit im2col")
    got, name = run_conv(src, w, bias, -1, 0, mult, shift, -5, -128, 127, (1, 1), (1, 1, 1, 1), path=1)
    assert name.startswith("im2col+"), name
    np.testing.assert_array_equal(got, want)


def test_config5_batched_s8_to_f32_k1000():
    rng = np.random.default_rng(5)
    batch, M, N, K = 16, 1024, 1024, 1000
    A = rng.integers(-128, 128, size=(batch, M, K), dtype=np.int8)
    B = rng.integers(-128, 128, size=(batch, K, N), dtype=np.int8)
    scale = float(np.float32(0.02) * np.float32(0.005))
    announce("config5")
    got, name = run_gemm(A, B, capi.EPI_F32, np.float32, 0, 0, scale=scale, device=True)
    assert name.startswith("pp_"), name
    rows = np.r_[0:24, 500:508, 1016:1024]
    for z in range(batch):
        # Every output: |acc| <= 1000 * 128 * 128 < 2^24, so the double-precision product is the exact integer, its
        # conversion to float is exact, and the one multiplication by the scale is the only rounding - which the
        # scalar oracle confirms on a row subset of every batch. Identical bits; the stated bar is 1e-5 relative.
        acc = A[z].astype(np.float64) @ B[z].astype(np.float64)
        assert np.abs(acc).max() < (1 << 24)
        want = acc.astype(np.float32) * np.float32(scale)
        np.testing.assert_array_equal(want[rows], oracle.gemmlowp_f32(A[z][rows], B[z], None, 0, 0, scale))
        np.testing.assert_array_equal(got[z].view(np.uint32), want.view(np.uint32))
    # shared B (2-D weights for every batch)
    got, _ = run_gemm(A[:3], B[0], capi.EPI_F32, np.float32, 0, 0, scale=scale, device=True)
    for z in range(3):
        np.testing.assert_array_equal(got[z][rows], oracle.gemmlowp_f32(A[z][rows], B[0], None, 0, 0, scale))


def test_negative_multiplier_takes_the_general_epilogue():
    """Multipliers < 0 never come out of calculate_quantized_multiplier but are legal inputs: the branch-free epilogue
    does not apply and the library must fall back to the general formula."""
    rng = np.random.default_rng(6)
    M, N, K = 256, 256, 128
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    mult = rng.integers(1 << 30, (1 << 31) - 1, size=N).astype(np.int32)
    mult[::7] *= -1
    mult[3] = -(1 << 31)
    shift = rng.integers(-2, 12, size=N).astype(np.int32)
    want = oracle.gemmlowp_fixedpoint(A, B, None, 5, 0, mult, shift, 1, -128, 127, np.int8)
    got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.int8, 5, 0, None, mult, shift, 1, -128, 127, device=True)
    np.testing.assert_array_equal(got, want)
    # extreme shifts: |shift| >= 32 yields 0 before the offset
    shift2 = shift.copy()
    shift2[::5] = 32
    shift2[1::5] = -32
    shift2[2::5] = 31
    mult2 = np.abs(mult.astype(np.int64)).clip(0, (1 << 31) - 1).astype(np.int32)
    want = oracle.gemmlowp_fixedpoint(A, B, None, 5, 0, mult2, shift2, 1, -128, 127, np.int8)
    got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.int8, 5, 0, None, mult2, shift2, 1, -128, 127, device=True)
    np.testing.assert_array_equal(got, want)
