"""The timed CPU baseline computes the same integers as the scalar oracle, at every SIMD level the host has."""
import os

import numpy as np
import pytest

import oracle


@pytest.mark.parametrize("level", ["0", "2", "5"])
@pytest.mark.parametrize("a_dt,b_dt", [(np.uint8, np.uint8), (np.int8, np.int8), (np.uint8, np.int8),
                                        (np.int8, np.uint8)])
def test_fast_equals_scalar(level, a_dt, b_dt, monkeypatch):
    monkeypatch.setenv("ORC_FAST_LEVEL", level)
    rng = np.random.default_rng(31)
    for (M, N, K, pc) in [(1, 1, 1, 0), (7, 9, 70, 0), (33, 130, 257, 1), (130, 67, 64, 1)]:
        A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(M, K)).astype(a_dt)
        B = rng.integers(np.iinfo(b_dt).min, np.iinfo(b_dt).max + 1, size=(K, N)).astype(b_dt)
        bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
        reals = np.exp(rng.uniform(np.log(1e-4), np.log(1.5), size=N if pc else 1))
        mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
        ao, bo = int(rng.integers(-100, 100)), (0 if pc else int(rng.integers(-100, 100)))
        for dst_dt, lo, hi in [(np.int8, -128, 127), (np.uint8, 0, 255), (np.int8, -3, 99)]:
            want = oracle.gemmlowp_fixedpoint(A, B, bias, ao, bo, mult, shift, -5, lo, hi, dst_dt)
            g = oracle.FastGemm(B)
            got = g.run(A, bias, ao, bo, mult, shift, -5, lo, hi, dst_dt)
            g.close()
            np.testing.assert_array_equal(got, want)
