"""The reference's Large GEMMLowp datasets on the GPU (tests/datasets/LargeGEMMLowpDataset.h:42-52,59-63,70-74 and
tests/datasets/GEMMLowpFusedOffsetOutputDataset.h:233-265): every K is odd (923, 873, 697, 1021, 681, 941, 364), so A
rows are not dword aligned and go through the padded copy of the A pre-pass at M up to 1023 (3025 for the 3-D output
shapes). Inputs are seeded; expected values come from the scalar CPU oracle, for the S32 cases additionally from an
exact double-precision matrix product. A dense 3-D output [N][H][D] of a 2-D GEMM with M = H*D rows is the same memory as the 2-D
output, which is how the C ABI takes it (the plane split lives in the host layer)."""
import numpy as np
import pytest

import oracle
from computelibrary_amd import capi
from gpu_util import announce, run_gemm

pytestmark = pytest.mark.gpu

# (M, N, K, a_offset, b_offset)
LARGE = [(1, 871, 923, 0, 0), (429, 871, 923, 0, 0), (7, 784, 873, -1, 3), (513, 784, 873, 0, 4),
         (872, 563, 697, -2, 0), (973, 783, 1021, 5, 13), (1023, 213, 681, -3, -2), (1011, 623, 941, -9, 1)]
# output [N][H][D] with H * D == M
LARGE_3D = [(429, 871, 923, 0, 0, (143, 3)), (1025, 213, 681, -3, 2, (205, 5)), (3025, 96, 364, 2, 3, (605, 5))]
# 3-D input and output (rows of A are the planes' rows, stacked)
LARGE_IO_3D = [(429, 871, 923, 0, 0, (143, 3)), (1025, 213, 681, -2, 5, (205, 5)), (3025, 96, 364, 2, 4, (605, 5))]


def operands(rng, M, N, K, a_dt, b_dt):
    A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(M, K)).astype(a_dt)
    B = rng.integers(np.iinfo(b_dt).min, np.iinfo(b_dt).max + 1, size=(K, N)).astype(b_dt)
    return A, B


@pytest.mark.parametrize("case", range(len(LARGE)))
@pytest.mark.parametrize("dt", [np.uint8, np.int8])
def test_large_dataset_s32(case, dt):
    M, N, K, ao, bo = LARGE[case]
    A, B = operands(np.random.default_rng(700 + case), M, N, K, dt, dt)
    want = oracle.gemmlowp_s32(A, B, ao, bo)
    exact = (A.astype(np.float64) + ao) @ (B.astype(np.float64) + bo)  # |sum| < 2^53: exact in double
    np.testing.assert_array_equal(want, exact.astype(np.int64).astype(np.int32))
    for device in (True, False):
        announce("large s32", case, (M, N, K), dt.__name__, ao, bo, "device", device)
        got, name = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, device=device)
        np.testing.assert_array_equal(got, want)
    if M > 64:
        assert name.startswith("pp_") or name.startswith("mfma"), name


@pytest.mark.parametrize("case", range(len(LARGE_3D) + len(LARGE_IO_3D)))
def test_large_dataset_3d_output_and_input(case):
    M, N, K, ao, bo, (H, D) = (LARGE_3D + LARGE_IO_3D)[case]
    assert H * D == M
    A, B = operands(np.random.default_rng(720 + case), M, N, K, np.uint8, np.uint8)
    want = oracle.gemmlowp_s32(A, B, ao, bo)
    announce("large 3d", case, (M, N, K), (H, D))
    got, _ = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, device=True)
    np.testing.assert_array_equal(got.reshape(D, H, N), want.reshape(D, H, N))


FUSED_U8 = [(429, 871, 923), (513, 784, 873), (973, 783, 1021), (1011, 623, 941), (1023, 213, 681)]
FUSED_S8_FIXEDPOINT = [(1, 871, 923), (7, 784, 873), (872, 563, 697), (973, 783, 1021)]
FUSED_S8_SCALE = [(7, 784, 873), (872, 563, 697), (1023, 213, 681)]


@pytest.mark.parametrize("case", range(len(FUSED_U8)))
def test_large_fused_uint8_fixedpoint(case):
    M, N, K = FUSED_U8[case]
    rng = np.random.default_rng(740 + case)
    A, B = operands(rng, M, N, K, np.uint8, np.uint8)
    ao, bo = int(rng.integers(-135, -120)), int(rng.integers(-135, -120))  # negated zero points near mid-range
    bias = rng.integers(-20000, 20000, size=N, dtype=np.int32)
    mult, shift = oracle.calculate_quantized_multiplier(float(rng.uniform(0.5, 2.0) * 40.0 / (K ** 0.5 * 74.0 * 74.0)))
    want = oracle.gemmlowp_fixedpoint(A, B, bias, ao, bo, [mult], [shift], 128, 0, 255, np.uint8)
    assert 0.2 < ((want > 0) & (want < 255)).mean()  # most outputs are not clamped
    for device in (True, False):
        announce("large fused u8", case, (M, N, K), ao, bo, mult, shift, "device", device)
        got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.uint8, ao, bo, bias, [mult], [shift], 128, 0, 255,
                          device=device)
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", range(len(FUSED_S8_FIXEDPOINT)))
@pytest.mark.parametrize("per_channel", [False, True])
def test_large_fused_int8_fixedpoint(case, per_channel):
    M, N, K = FUSED_S8_FIXEDPOINT[case]
    rng = np.random.default_rng(760 + case)
    A, B = operands(rng, M, N, K, np.int8, np.int8)
    ao, bo = int(rng.integers(-20, 20)), 0 if per_channel else int(rng.integers(-20, 20))
    bias = rng.integers(-20000, 20000, size=N, dtype=np.int32)
    reals = rng.uniform(0.5, 2.0, size=N if per_channel else 1) * 40.0 / (K ** 0.5 * 74.0 * 74.0)
    mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
    want = oracle.gemmlowp_fixedpoint(A, B, bias, ao, bo, mult, shift, -3, -128, 127, np.int8)
    assert 0.2 < ((want > -128) & (want < 127)).mean()
    announce("large fused s8", case, (M, N, K), ao, bo, "per_channel", per_channel)
    got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.int8, ao, bo, bias, mult, shift, -3, -128, 127, device=True)
    np.testing.assert_array_equal(got, want)


def test_large_fused_int8_fixedpoint_batched_single_row():
    """TensorShape(923, 1, 15) x TensorShape(871, 923, 15): 15 single-row products, each with its own B"""
    rng = np.random.default_rng(780)
    batch, M, N, K = 15, 1, 871, 923
    A = rng.integers(-128, 128, size=(batch, M, K), dtype=np.int8)
    B = rng.integers(-128, 128, size=(batch, K, N), dtype=np.int8)
    bias = rng.integers(-20000, 20000, size=N, dtype=np.int32)
    mult, shift = oracle.calculate_quantized_multiplier(1.0 / (K ** 0.5 * 74.0 * 74.0 / 40.0))
    announce("large fused s8 batched", (batch, M, N, K))
    got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.int8, 4, -6, bias, [mult], [shift], 2, -128, 127, device=True)
    for z in range(batch):
        np.testing.assert_array_equal(
            got[z], oracle.gemmlowp_fixedpoint(A[z], B[z], bias, 4, -6, [mult], [shift], 2, -128, 127, np.int8))


@pytest.mark.parametrize("case", range(len(FUSED_S8_SCALE)))
def test_large_fused_int8_integer_scale_stage(case):
    """QUANTIZE_DOWN: ((acc + offset) * multiplier) >> shift"""
    M, N, K = FUSED_S8_SCALE[case]
    rng = np.random.default_rng(790 + case)
    A, B = operands(rng, M, N, K, np.int8, np.int8)
    ao, bo = int(rng.integers(-20, 20)), int(rng.integers(-20, 20))
    bias = rng.integers(-20000, 20000, size=N, dtype=np.int32)
    mult, shift, off = 3, 12, int(rng.integers(-500, 500))
    want = oracle.gemmlowp_scale(A, B, bias, ao, bo, [mult], [shift], off, -128, 127, np.int8)
    assert 0.2 < ((want > -128) & (want < 127)).mean()
    announce("large fused s8 scale stage", case, (M, N, K), ao, bo)
    got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.int8, ao, bo, bias, [mult], [shift], off, -128, 127, device=True,
                      stage=capi.STAGE_SCALE)
    np.testing.assert_array_equal(got, want)
