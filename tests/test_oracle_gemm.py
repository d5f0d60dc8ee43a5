"""Pins the GEMM-level functions of the CPU oracle against the fixtures the reference's portable
code produced, against exact int64 numpy arithmetic, and through the identities the algebra fixes."""
import numpy as np
import pytest

import oracle


def wrap32(x):
    return ((np.asarray(x, dtype=np.int64) + (1 << 31)) & 0xFFFFFFFF) - (1 << 31)


def exact_t(A, B, ao, bo):
    """sum_k (A+ao)(B+bo) in int64, wrapped to int32"""
    return wrap32((A.astype(np.int64) + ao) @ (B.astype(np.int64) + bo)).astype(np.int32)


def test_s32_fixture(golden):
    g = golden("gemmlowp_s32.npz")
    for n in range(int(g["count"])):
        ao, bo = (int(x) for x in g["off%d" % n])
        got = oracle.gemmlowp_s32(g["a%d" % n], g["b%d" % n], ao, bo)
        np.testing.assert_array_equal(got, g["dst%d" % n])


def test_s32_batched_fixture(golden):
    g = golden("gemmlowp_batched.npz")
    for n in range(int(g["count"])):
        A, B = g["a%d" % n], g["b%d" % n]
        ao, bo = (int(x) for x in g["off%d" % n])
        for z in range(A.shape[0]):
            got = oracle.gemmlowp_s32(A[z], B[z] if B.ndim == 3 else B, ao, bo)
            np.testing.assert_array_equal(got, g["dst%d" % n][z])


@pytest.mark.parametrize("a_dt,b_dt", [(np.uint8, np.uint8), (np.int8, np.int8), (np.uint8, np.int8),
                                        (np.int8, np.uint8)])
def test_s32_against_int64_matmul(a_dt, b_dt):
    rng = np.random.default_rng(11)
    for (M, N, K) in [(1, 1, 1), (5, 7, 300), (17, 9, 1000), (64, 48, 129)]:
        A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(M, K)).astype(a_dt)
        B = rng.integers(np.iinfo(b_dt).min, np.iinfo(b_dt).max + 1, size=(K, N)).astype(b_dt)
        for ao, bo in [(0, 0), (-128, 127), (3, 0), (0, -7), (2147480000, 5)]:
            np.testing.assert_array_equal(oracle.gemmlowp_s32(A, B, ao, bo), exact_t(A, B, ao, bo))


def test_flip_signedness_invariance():
    """x ^ 0x80 on an operand with -/+128 on its offset leaves t unchanged
    (src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:153-190)."""
    rng = np.random.default_rng(12)
    A = rng.integers(0, 256, size=(9, 77), dtype=np.uint8)
    B = rng.integers(0, 256, size=(77, 13), dtype=np.uint8)
    want = oracle.gemmlowp_s32(A, B, -5, 9)
    As = (A ^ 0x80).view(np.int8)
    Bs = (B ^ 0x80).view(np.int8)
    np.testing.assert_array_equal(oracle.gemmlowp_s32(As, B, -5 + 128, 9), want)
    np.testing.assert_array_equal(oracle.gemmlowp_s32(As, Bs, -5 + 128, 9 + 128), want)


def test_fused_fixedpoint_fixture(golden):
    g = golden("gemmlowp_fused_fixedpoint.npz")
    kinds = set()
    for n in range(int(g["count"])):
        ao, bo, roff, lo, hi, pc = (int(x) for x in g["p%d" % n])
        dst = g["dst%d" % n]
        got = oracle.gemmlowp_fixedpoint(g["a%d" % n], g["b%d" % n], g["bias%d" % n], ao, bo, g["mult%d" % n],
                                         g["shift%d" % n], roff, lo, hi, dst.dtype)
        np.testing.assert_array_equal(got, dst)
        kinds.add((dst.dtype.name, pc, bool((g["shift%d" % n] < 0).any())))
    # the fixture covers u8 / s8, per tensor / per channel, right and left shifts
    assert ("uint8", 0, True) in kinds and ("int8", 1, True) in kinds and ("int8", 0, False) in kinds


def test_output_stage_fixture(golden):
    g = golden("output_stage.npz")
    for n in range(int(g["count"])):
        mult, shift, roff, lo, hi, with_bias = (int(x) for x in g["p%d" % n])
        dst = g["dst%d" % n]
        got = oracle.output_stage_fixedpoint(g["src%d" % n], g["bias%d" % n] if with_bias else None, [mult], [shift],
                                             roff, lo, hi, dst.dtype)
        np.testing.assert_array_equal(got, dst)


def test_output_stage_scale_fixture(golden):
    """QUANTIZE_DOWN (integer multiplier) against the outputs of the reference's gemmlowp_quantize_down_scale."""
    g = golden("output_stage_scale.npz")
    kinds = set()
    for n in range(int(g["count"])):
        roff, lo, hi, with_bias = (int(x) for x in g["p%d" % n])
        dst = g["dst%d" % n]
        if lo == hi:  # "no bounded activation": only the saturation to the type is left
            lo, hi = -(1 << 31), (1 << 31) - 1
        got = oracle.output_stage_scale(g["src%d" % n], g["bias%d" % n] if with_bias else None, g["mult%d" % n],
                                        g["shift%d" % n], roff, lo, hi, dst.dtype)
        np.testing.assert_array_equal(got, dst)
        kinds.add((dst.dtype.name, len(g["mult%d" % n]) > 1, bool(with_bias)))
        inside = ((dst > np.iinfo(dst.dtype).min) & (dst < np.iinfo(dst.dtype).max)).mean()
    assert ("uint8", True, True) in kinds or ("uint8", True, False) in kinds
    assert ("int8", False, True) in kinds and ("int8", False, False) in kinds


def test_scale_stage_primitive_properties():
    """((v + off) * m) >> s: truncating (floor) shift, wrap-around product, agrees with exact integer arithmetic wherever
    nothing overflows."""
    rng = np.random.default_rng(111)
    v = rng.integers(-(1 << 20), 1 << 20, size=5000).astype(np.int64)
    for m, sft, off in ((1, 0, 0), (3, 9, -40), (255, 16, 1234), (77, 31, -5)):
        want = ((v + off) * m) >> sft  # python ints: floor division by 2^s
        got = np.array([oracle.lib.orc_requant_scale_s32(int(x), m, sft, off) for x in v[:500]])
        np.testing.assert_array_equal(got, want[:500])
    # wrap-around: the product is taken modulo 2^32 before the shift
    assert oracle.lib.orc_requant_scale_s32(1 << 30, 4, 0, 0) == 0
    assert oracle.lib.orc_requant_scale_s32((1 << 30) + 1, 4, 1, 0) == 2
    assert oracle.lib.orc_requant_scale_s32(-1, 1, 5, 0) == -1  # floor, not round-to-zero

def test_f32_fixture(golden):
    """The reference's test oracle rounds once (float(t)*scale); the NEON order this oracle follows rounds
    acc*scale and offsets*scale separately. Identical when offsets are zero, else equal to ~1 ulp of the
    larger term."""
    g = golden("gemmlowp_f32.npz")
    scale = float(g["scale"])
    for n in range(int(g["count"])):
        ao, bo = (int(x) for x in g["off%d" % n])
        A, B = g["a%d" % n], g["b%d" % n]
        got = oracle.gemmlowp_f32(A, B, None, ao, bo, scale)
        want = g["dst%d" % n]
        if ao == 0 and bo == 0:
            np.testing.assert_array_equal(got, want)
        else:
            acc = np.abs(A.astype(np.int64) @ B.astype(np.int64)).astype(np.float64) * scale
            off = np.abs(exact_t(A, B, ao, bo).astype(np.float64) * scale - (A.astype(np.int64) @ B.astype(np.int64)) * scale)
            tol = (acc + off + np.abs(want)) * 2.0 ** -23
            assert (np.abs(got.astype(np.float64) - want) <= tol).all()


def test_f32_bias_and_activation():
    rng = np.random.default_rng(13)
    A = rng.integers(-128, 128, size=(6, 40), dtype=np.int8)
    B = rng.integers(-128, 128, size=(40, 10), dtype=np.int8)
    bias = rng.normal(0, 3, size=10).astype(np.float32)
    scale = np.float32(0.02) * np.float32(0.005)
    got = oracle.gemmlowp_f32(A, B, bias, 0, 0, float(scale), 0.0, 6.0)
    acc = (A.astype(np.int32) @ B.astype(np.int32)).astype(np.float32)
    want = np.clip(acc * scale + bias, np.float32(0), np.float32(6))
    np.testing.assert_array_equal(got, want.astype(np.float32))


def _sqrdmulh_model(a, b):
    """Arm ARM, SQRDMULH (vector, 32-bit): SInt sat((2 * a * b + (1 << 31)) >> 32), with Python integers"""
    r = (2 * a * b + (1 << 31)) >> 32
    return max(-(1 << 31), min((1 << 31) - 1, r))


def _requant_s16_model(v, mult, shift, lo, hi):
    """src/core/NEON/NESymm.h:54-85 lane by lane with Python integers (the int32 left shift wraps)"""
    wrap = lambda x: ((x + (1 << 31)) % (1 << 32)) - (1 << 31)
    if shift < 0:
        r = _sqrdmulh_model(wrap(v * (1 << -shift)), mult)
    else:
        r = _sqrdmulh_model(v, mult)
        if shift > 0:
            r = (r + (1 << (shift - 1))) >> shift  # SRSHL by -shift: round half up, no overflow in big integers
    r = max(-32768, min(32767, r))
    if not (lo <= -32768 and hi >= 32767):
        r = max(lo, min(hi, r))
    return r


def test_requant_s16_against_big_integer_model_and_reference_within_one():
    rng = np.random.default_rng(16)
    edge = [0, 1, -1, 2, -2, (1 << 31) - 1, -(1 << 31), 1 << 30, -(1 << 30), 12345678, -87654321]
    for a in edge:
        for b in edge:
            assert oracle.lib.orc_sqrdmulh_s32(a, b) == _sqrdmulh_model(a, b), (a, b)
    vals = np.concatenate([np.array(edge, dtype=np.int64), rng.integers(-(1 << 31), 1 << 31, size=300),
                           rng.integers(-(1 << 17), 1 << 17, size=300)])
    for mult in [1 << 30, (1 << 31) - 1, 1518500250, 1073741825, 0, -(1 << 30)]:
        for shift in [-3, -1, 0, 1, 2, 7, 15, 31]:
            for lo, hi in [(-32768, 32767), (-(1 << 31), (1 << 31) - 1), (-100, 20000), (0, 32767)]:
                for v in vals[::7]:
                    got = oracle.lib.orc_requant_fixedpoint_s16(int(v), mult, shift, lo, hi)
                    assert got == _requant_s16_model(int(v), mult, shift, lo, hi), (v, mult, shift, lo, hi)
    # rounding vs truncating high multiply: a value where they differ, hand-checked:
    # 3 * 1518500250 = 4555500750; (x + 2^30) >> 31 = 2 (2.121 rounds to 2); 5 * 1518500250 -> 3.535 -> 4, truncating gives 3
    assert oracle.lib.orc_sqrdmulh_s32(5, 1518500250) == 4 and oracle.lib.orc_sqdmulh(5, 1518500250) == 3
    if oracle.ref_available():
        # the reference's portable oracle multiplies without rounding: never more than 1 apart, and not always equal
        src = rng.integers(-(1 << 20), 1 << 20, size=(9, 40)).astype(np.int32)
        bias = rng.integers(-1000, 1000, size=40).astype(np.int32)
        for mult, shift in [(1518500250, 4), (1 << 30, 0), (2000000000, 9)]:
            want = oracle.ref_quantize_down_fixedpoint_s16(src, bias, mult, shift, -(1 << 31), (1 << 31) - 1)
            got = oracle.output_stage_fixedpoint_s16(src, bias, mult, shift)
            d = got.astype(np.int32) - want.astype(np.int32)
            assert np.abs(d).max() <= 1 and (d >= 0).all()


def test_f32_accumulate_and_double_clamp_against_numpy_float32():
    """numpy float32 arithmetic rounds every operation separately, like the NEON instructions of
    src/core/NEON/kernels/arm_gemm/quantized.cpp:1000-1017 and src/cpu/kernels/gemmlowp/generic/neon/fp32.cpp:31-54:
    ((acc*s + bias) + prev) -> clamp -> + off*s -> clamp, written out independently of the C oracle."""
    rng = np.random.default_rng(14)
    A = rng.integers(-128, 128, size=(12, 64), dtype=np.int8)
    B = rng.integers(-128, 128, size=(64, 20), dtype=np.int8)
    bias = rng.normal(0, 3, size=20).astype(np.float32)
    prev = rng.normal(0, 5, size=(12, 20)).astype(np.float32)
    s = np.float32(1e-3)
    acc = (A.astype(np.int32) @ B.astype(np.int32))
    off = exact_t(A, B, 30, 20).astype(np.int64) - acc
    lo, hi = np.float32(0), np.float32(6)
    r = (acc.astype(np.float32) * s + bias) + prev
    want_twice = np.clip(np.clip(r, lo, hi) + off.astype(np.float32) * s, lo, hi)
    want_once = np.clip(r + off.astype(np.float32) * s, lo, hi)
    got_twice = oracle.gemmlowp_f32(A, B, bias, 30, 20, float(s), 0.0, 6.0, prev=prev, act_twice=True)
    got_once = oracle.gemmlowp_f32(A, B, bias, 30, 20, float(s), 0.0, 6.0, prev=prev)
    np.testing.assert_array_equal(got_twice, want_twice)
    np.testing.assert_array_equal(got_once, want_once)
    assert (want_once != want_twice).any()
    # without accumulation the previous contents must not matter
    np.testing.assert_array_equal(oracle.gemmlowp_f32(A, B, bias, 0, 0, float(s)), acc.astype(np.float32) * s + bias)


def _half_ulps(a_bits, b_bits):
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u)
    return np.abs(key(a_bits) - key(b_bits))


def test_f16_destination_fixture(golden):
    """orc_gemmlowp_f16 against halfs the reference's own code produced (dequantization_layer<half, int32_t> and the half
    arithmetic_operation behind tests/validation/fixtures/GEMMLowpFixture.h:908-920), committed as a fixture so the pin
    holds without the reference checkout. Zero offsets: identical bits, with and without accumulation. Non-zero
    offsets: the float underneath follows the NEON order of operations (two roundings), which crosses a half rounding
    boundary now and then: never more than one half apart before the accumulation, equal almost everywhere."""
    g = golden("gemmlowp_f16.npz")
    scale = float(g["scale"])
    seen_offsets = 0
    for n in range(int(g["count"])):
        A, B, prev = g["a%d" % n], g["b%d" % n], g["prev%d" % n]
        ao, bo = (int(x) for x in g["off%d" % n])
        got = oracle.gemmlowp_f16(A, B, None, ao, bo, scale).view(np.uint16)
        acc = oracle.gemmlowp_f16(A, B, None, ao, bo, scale, prev=prev).view(np.uint16)
        if ao == 0 and bo == 0:
            np.testing.assert_array_equal(got, g["dst%d" % n])
            np.testing.assert_array_equal(acc, g["acc%d" % n])
        else:
            seen_offsets += 1
            assert _half_ulps(got, g["dst%d" % n]).max() <= 1
            assert (got == g["dst%d" % n]).mean() > 0.99 and (acc == g["acc%d" % n]).mean() > 0.99
    assert seen_offsets >= 2


@pytest.mark.skipif(not oracle.ref_available(), reason="oracle/_ref not built (needs the reference checkout)")
def test_fused_against_live_reference_config1_shape():
    """BASELINE config 1 at full size (256^3, QASYMM8, both zero-point conventions) through the reference's code."""
    rng = np.random.default_rng(1)
    A = rng.integers(0, 256, size=(256, 256), dtype=np.uint8)
    B = rng.integers(0, 256, size=(256, 256), dtype=np.uint8)
    bias = rng.integers(-1000, 1001, size=256, dtype=np.int32)
    for ao, bo in [(-128, -127), (128, 127)]:
        t = oracle.ref_gemmlowp_core(A, B, ao, bo)
        want = oracle.ref_quantize_down_fixedpoint(t, bias, [1518500250], [8], 10, 0, 255, np.uint8)
        got = oracle.gemmlowp_fixedpoint(A, B, bias, ao, bo, [1518500250], [8], 10, 0, 255, np.uint8)
        np.testing.assert_array_equal(got, want)
        if ao < 0:
            inside = ((want > 0) & (want < 255)).mean()
            assert 0.2 < inside < 0.6  # a meaningful share of outputs is not clamped


def test_half_conversion_against_numpy_and_by_construction():
    """float -> half of the oracle: every half value survives the round trip; exact midpoints between neighbouring
    halfs go to the even one; the overflow and underflow thresholds; 200k random floats against numpy's conversion
    (IEEE round-to-nearest-even)."""
    bits = np.arange(1 << 16, dtype=np.uint16)
    vals = oracle.f16_bits_to_f32(bits)
    finite = np.isfinite(vals)
    np.testing.assert_array_equal(vals[finite], bits.view(np.float16).astype(np.float32)[finite])
    np.testing.assert_array_equal(oracle.f32_to_f16_bits(vals[finite]), bits[finite])
    assert np.isnan(vals[~finite & ((bits & 0x3FF) != 0)]).all() and np.isinf(vals[(bits & 0x7FFF) == 0x7C00]).all()
    # midpoints of neighbouring positive halfs (exact in float): ties to even
    lo = np.arange(0, 0x7BFF, dtype=np.uint16)
    mid = (oracle.f16_bits_to_f32(lo).astype(np.float64) + oracle.f16_bits_to_f32(lo + 1).astype(np.float64)) / 2
    assert (mid.astype(np.float32).astype(np.float64) == mid).all()
    want = np.where(lo % 2 == 0, lo, lo + 1).astype(np.uint16)
    np.testing.assert_array_equal(oracle.f32_to_f16_bits(mid.astype(np.float32)), want)
    np.testing.assert_array_equal(oracle.f32_to_f16_bits(-mid.astype(np.float32)), want | 0x8000)
    # thresholds
    for v, h in [(65504.0, 0x7BFF), (65519.996, 0x7BFF), (65520.0, 0x7C00), (1e9, 0x7C00), (2.0 ** -24, 0x0001),
                 (2.0 ** -25, 0x0000), (np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 0x0001), (0.0, 0x0000),
                 (2.0 ** -14, 0x0400), (np.inf, 0x7C00)]:
        assert int(oracle.f32_to_f16_bits(np.float32(v)).item()) == h, v
        assert int(oracle.f32_to_f16_bits(np.float32(-v)).item()) == (h | 0x8000), v
    rng = np.random.default_rng(16)
    x = np.concatenate([rng.normal(0, 1, 50000), rng.normal(0, 1e-6, 50000), rng.normal(0, 3e4, 50000),
                        np.exp(rng.uniform(np.log(1e-9), np.log(1e6), 50000)) * rng.choice([-1, 1], 50000)]).astype(np.float32)
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(oracle.f32_to_f16_bits(x), x.astype(np.float16).view(np.uint16))


@pytest.mark.skipif(not oracle.ref_available(), reason="oracle/_ref not built (needs the reference checkout)")
def test_f16_destination_against_live_reference():
    """The reference's F16 GEMMLowp values (GEMMLowpFixture.h:908-920: half(float(s32) * scale), plus the previous halfs,
    added as halfs, when accumulating) through its own code. Without offsets the oracle must give the same bits, with
    and without accumulation; with offsets the float underneath follows the NEON rounding order (<= 1e-5 relative),
    which may cross a half rounding boundary now and then: at most one half ulp apart before the accumulation, and
    equal almost everywhere."""
    rng = np.random.default_rng(5)
    A = rng.integers(-128, 128, size=(37, 120), dtype=np.int8)
    B = rng.integers(-128, 128, size=(120, 53), dtype=np.int8)
    scale = (1.0 / 255) * (5.0 / 255)
    prev = rng.normal(0, 2, size=(37, 53)).astype(np.float16)
    t = oracle.ref_gemmlowp_core(A, B, 0, 0)
    np.testing.assert_array_equal(oracle.gemmlowp_f16(A, B, None, 0, 0, scale).view(np.uint16),
                                  oracle.ref_dequantize_s32_f16(t, scale).view(np.uint16))
    np.testing.assert_array_equal(oracle.gemmlowp_f16(A, B, None, 0, 0, scale, prev=prev).view(np.uint16),
                                  oracle.ref_dequantize_s32_f16(t, scale, prev=prev).view(np.uint16))

    def ulps(a, b):  # distance in representable halfs
        def key(h):
            u = h.view(np.uint16).astype(np.int32)
            return np.where(u & 0x8000, -(u & 0x7FFF), u)
        return np.abs(key(a) - key(b))

    t = oracle.ref_gemmlowp_core(A, B, 3, -7)
    got = oracle.gemmlowp_f16(A, B, None, 3, -7, scale)
    want = oracle.ref_dequantize_s32_f16(t, scale)
    assert ulps(got, want).max() <= 1 and (got.view(np.uint16) == want.view(np.uint16)).mean() > 0.99
    got = oracle.gemmlowp_f16(A, B, None, 3, -7, scale, prev=prev)
    want = oracle.ref_dequantize_s32_f16(t, scale, prev=prev)
    assert (got.view(np.uint16) == want.view(np.uint16)).mean() > 0.99
    # the oracle's own definition, restated with numpy's conversions
    f = oracle.gemmlowp_f32(A, B, None, 3, -7, scale)
    np.testing.assert_array_equal(oracle.gemmlowp_f16(A, B, None, 3, -7, scale).view(np.uint16), f.astype(np.float16).view(np.uint16))
    acc = (prev.astype(np.float32) + f.astype(np.float16).astype(np.float32)).astype(np.float16)
    np.testing.assert_array_equal(got.view(np.uint16), acc.view(np.uint16))
    clamped = oracle.gemmlowp_f16(A, B, None, 3, -7, scale, 0.0, 1.5, prev=prev)
    np.testing.assert_array_equal(clamped.view(np.uint16), np.clip(acc.astype(np.float32), 0.0, 1.5).astype(np.float16).view(np.uint16))
