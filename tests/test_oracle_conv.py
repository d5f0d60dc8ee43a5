"""Pins im2col, weight flattening and the conv lowering of the CPU oracle."""
import numpy as np
import pytest

import oracle


def test_im2col_fixture(golden):
    g = golden("im2col_nhwc.npz")
    for n in range(int(g["count"])):
        KH, KW, sx, sy, pl, pt, pr, pb, zp = (int(x) for x in g["p%d" % n])
        got = oracle.im2col_nhwc(g["src%d" % n], KH, KW, (sx, sy), (pl, pt, pr, pb), (1, 1), zp)
        np.testing.assert_array_equal(got, g["dst%d" % n])


def test_weights_reshape_ordering():
    OFM, KH, KW, C = 3, 2, 3, 4
    w = np.arange(OFM * KH * KW * C, dtype=np.uint8).reshape(OFM, KH, KW, C)
    b = oracle.weights_reshape(w)
    assert b.shape == (KH * KW * C, OFM)
    for o in range(OFM):
        for ky in range(KH):
            for kx in range(KW):
                for c in range(C):
                    assert b[c + kx * C + ky * C * KW, o] == w[o, ky, kx, c]


def _run_case(g, n, fn):
    sx, sy, pl, pt, pr, pb, in_zp, w_zp, out_zp, pc = (int(x) for x in g["p%d" % n])
    src, w, bias, want = g["src%d" % n], g["w%d" % n], g["bias%d" % n], g["dst%d" % n]
    in_scale, out_scale = g["scales%d" % n]
    mult, shift = oracle.calculate_quantized_multipliers(in_scale, g["wscale%d" % n], out_scale)
    lo, hi = (-128, 127) if src.dtype == np.int8 else (0, 255)
    got = fn(src, w, bias, in_zp, w_zp, mult, shift, out_zp, lo, hi, (sx, sy), (pl, pt, pr, pb))
    np.testing.assert_array_equal(got, want)


def test_conv_fixture_via_im2col_gemm(golden):
    g = golden("conv_nhwc.npz")
    for n in range(int(g["count"])):
        _run_case(g, n, oracle.conv_nhwc_gemm)


def test_conv_fixture_direct(golden):
    g = golden("conv_nhwc.npz")
    for n in range(int(g["count"])):
        _run_case(g, n, oracle.conv_nhwc_direct)


def test_conv_dilation_direct_equals_lowered():
    rng = np.random.default_rng(21)
    src = rng.integers(-128, 128, size=(2, 9, 10, 3), dtype=np.int8)
    w = rng.integers(-127, 128, size=(5, 3, 3, 3), dtype=np.int8)
    bias = rng.integers(-500, 500, size=5, dtype=np.int32)
    mult, shift = oracle.calculate_quantized_multipliers(0.02, rng.uniform(0.01, 1, 5), 1.3)
    args = (src, w, bias, -3, 0, mult, shift, 4, -128, 127, (1, 2), (2, 1, 2, 1), (2, 2))
    np.testing.assert_array_equal(oracle.conv_nhwc_direct(*args), oracle.conv_nhwc_gemm(*args))
