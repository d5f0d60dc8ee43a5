"""Pins the requantisation primitives of the CPU oracle: against outputs of the reference's own
portable code (tests/golden/*.npz, written by tests/golden/make_fixtures.py), against that code live
when oracle/_ref is built, and against an arbitrary-precision model of SQDMULH / SRSHL for the edge
cases where the reference's C++ would overflow a signed int."""
import numpy as np
import pytest

import oracle

I32_MIN, I32_MAX = -(1 << 31), (1 << 31) - 1


def wrap32(x):
    return ((int(x) + (1 << 31)) & 0xFFFFFFFF) - (1 << 31)


def model_sqdmulh(a, b):
    """Arm ARM: SQDMULH = sat32((2*a*b) >> 32), no rounding."""
    r = (2 * int(a) * int(b)) >> 32
    return min(max(r, I32_MIN), I32_MAX)


def model_srshl_right(x, e):
    """Arm ARM: SRSHL by -e = (x + 2^(e-1)) >> e in unbounded precision."""
    return int(x) if e == 0 else (int(x) + (1 << (e - 1))) >> e


def model_requant(v, m, s, off):
    if s < 0:
        r = model_sqdmulh(wrap32(int(v) * (1 << -s)), m)
    else:
        r = model_srshl_right(model_sqdmulh(v, m), s)
    return wrap32(r + off)


def test_sqdmulh_fixture(golden):
    tab = golden("requant_sweep.npz")["sqdmulh"]
    for a, b, want in tab:
        assert oracle.sqdmulh(a, b) == want


def test_requant_sweep_fixture(golden):
    tab = golden("requant_sweep.npz")["table"]
    assert tab.shape[0] > 30000
    for v, m, s, want in tab:
        assert oracle.requant_s32(v, m, s, 0) == want, (v, m, s)


def test_requant_edge_cases_against_isa_model():
    vals = [I32_MIN, I32_MIN + 1, -(1 << 30), -1, 0, 1, 1 << 30, I32_MAX, I32_MAX - 1, 123456789, -987654321]
    mults = [1 << 30, 1518500250, I32_MAX, I32_MIN, 1, -1, 0]
    for v in vals:
        for m in mults:
            assert oracle.sqdmulh(v, m) == model_sqdmulh(v, m)
            for s in range(-8, 40):
                for off in (0, 10, -5, I32_MAX):
                    assert oracle.requant_s32(v, m, s, off) == model_requant(v, m, s, off), (v, m, s, off)


def test_rounding_is_half_up_not_half_away():
    # -3 / 2 = -1.5 -> half-up gives -1 (half-away-from-zero would give -2)
    assert oracle.rounding_shift_right(-3, 1) == -1
    assert oracle.rounding_shift_right(3, 1) == 2
    assert oracle.rounding_shift_right(-5, 2) == -1
    assert oracle.rounding_shift_right(I32_MAX, 1) == 1 << 30  # no overflow of x + 2^(e-1)
    assert oracle.rounding_shift_right(I32_MAX, 31) == 1
    assert oracle.rounding_shift_right(I32_MIN, 31) == -1
    assert oracle.rounding_shift_right(12345, 32) == 0


def test_sqdmulh_is_not_rounding():
    # rounding-doubling-high-mul of (1, 2^30) would be 1 (0.5 rounds up); SQDMULH floors to 0
    assert oracle.sqdmulh(1, 1 << 30) == 0
    assert oracle.sqdmulh(-1, 1 << 30) == -1
    assert oracle.sqdmulh(I32_MIN, I32_MIN) == I32_MAX
    # the worked example: acc 1260 + bias 1, multiplier 1518500250, shift 8, offset 10 -> 13
    assert oracle.requant_s32(1261, 1518500250, 8, 10) == 13


def test_narrow_clamp():
    f = oracle.lib.orc_narrow_clamp
    assert f(300, 0, 0, 255) == 255 and f(-4, 0, 0, 255) == 0 and f(7, 0, 10, 200) == 10
    assert f(300, 1, -128, 127) == 127 and f(-300, 1, -128, 127) == -128 and f(100, 1, -5, 90) == 90


def test_quantized_multiplier_fixture(golden):
    g = golden("quant_multiplier.npz")
    for real, m, s in zip(g["real"], g["mult"], g["shift"]):
        assert oracle.calculate_quantized_multiplier(float(real)) == (m, s), real


def test_quantized_multiplier_invariants():
    rng = np.random.default_rng(5)
    for real in np.exp(rng.uniform(np.log(1e-7), np.log(100.0), size=3000)).astype(np.float32):
        m, s = oracle.calculate_quantized_multiplier(float(real))
        assert (1 << 30) <= m < (1 << 31)
        assert abs(m * 2.0 ** -31 * 2.0 ** -s - float(real)) <= float(real) * 2.0 ** -30
        assert (s <= 0) == (real >= 1.0) or (real < 1.0 and s == 0)
    assert oracle.calculate_quantized_multiplier(1.0) == (1 << 30, -1)
    assert oracle.calculate_quantized_multiplier(0.5) == (1 << 30, 0)
    assert oracle.calculate_quantized_multiplier(0.0007) == (1539316224, 10)
    # float just below one whose mantissa rounds to 2^31: renormalised
    m, s = oracle.calculate_quantized_multiplier(float(np.float32(0.99999994)))
    assert (1 << 30) <= m < (1 << 31) and s == 0
    with pytest.raises(ValueError):
        oracle.calculate_quantized_multiplier(-0.5)


@pytest.mark.skipif(not oracle.ref_available(), reason="oracle/_ref not built (needs the reference checkout)")
def test_primitives_against_live_reference():
    rng = np.random.default_rng(9)
    r = oracle.ref()
    for _ in range(20000):
        v = int(rng.integers(-(1 << 29), 1 << 29))
        m = int(rng.integers(1 << 30, 1 << 31))
        s = int(rng.integers(0, 32))
        assert oracle.requant_s32(v, m, s, 7) == r.ref_quantize_down_scalar(v, m, s, 7, I32_MIN, I32_MAX)
    for real in np.exp(rng.uniform(np.log(1e-6), np.log(30.0), size=5000)).astype(np.float32):
        assert oracle.calculate_quantized_multiplier(float(real)) == oracle.ref_calculate_quantized_multiplier(
            float(real))
