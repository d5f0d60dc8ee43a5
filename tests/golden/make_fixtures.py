"""Writes the golden fixtures in this directory from the reference's own portable oracle.

Run in the build container (needs oracle/_ref/libaclref.so, i.e. the reference checkout):
    python tests/golden/make_fixtures.py
Every .npz holds the inputs and the outputs the reference's code produced for them; nothing of the
reference's source travels. Shapes and offsets follow the reference's own test datasets:
tests/datasets/SmallGEMMLowpDataset.h:42-52, tests/datasets/GEMMLowpFusedOffsetOutputDataset.h:120-226,
tests/validation/NEON/ConvolutionLayer.cpp:1682-1691.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.abspath(os.path.join(HERE, "..", "..")))
import oracle  # noqa: E402

SMALL_GEMMLOWP = [  # (M, N, K, a_offset, b_offset)
    (1, 1, 21, 0, 0), (13, 33, 21, 0, 0), (3, 72, 31, -2, 13), (13, 33, 52, 0, 4), (26, 33, 52, -2, 0),
    (27, 23, 31, 5, 13), (43, 21, 38, -3, -2), (72, 17, 32, -9, 1),
]
FUSED_SHAPES = [(13, 1, 21), (13, 33, 52), (27, 23, 31), (72, 16, 32), (1, 43, 21), (3, 72, 31), (72, 17, 32),
                (26, 33, 52), (43, 21, 38)]
BATCHED = [  # (batch, M, N, K, b_batched)
    (1, 3, 2, 4, 0), (1, 15, 7, 12, 0), (3, 4, 5, 2, 1), (3, 7, 29, 15, 1), (3, 7, 29, 15, 0), (4, 17, 5, 56, 1),
]
REALS = [0.0007, 0.0027621, 0.33, 0.999999, 1.0, 1.7, 3.2]


def rnd8(rng, shape, signed):
    return rng.integers(-128, 128, size=shape, dtype=np.int8) if signed else rng.integers(
        0, 256, size=shape, dtype=np.uint8)


def gemmlowp_s32():
    rng = np.random.default_rng(101)
    out = {}
    n = 0
    for signed in (0, 1):
        for (M, N, K, ao, bo) in SMALL_GEMMLOWP:
            A, B = rnd8(rng, (M, K), signed), rnd8(rng, (K, N), signed)
            out["a%d" % n], out["b%d" % n] = A, B
            out["off%d" % n] = np.array([ao, bo], dtype=np.int32)
            out["dst%d" % n] = oracle.ref_gemmlowp_core(A, B, ao, bo)
            n += 1
    # mixed sign: the reference only exports the zero-offset instantiation
    for (M, N, K, _, _) in SMALL_GEMMLOWP[:4]:
        A, B = rnd8(rng, (M, K), 0), rnd8(rng, (K, N), 1)
        out["a%d" % n], out["b%d" % n] = A, B
        out["off%d" % n] = np.array([0, 0], dtype=np.int32)
        out["dst%d" % n] = oracle.ref_gemmlowp_u8s8(A, B)
        n += 1
    out["count"] = np.array(n)
    np.savez_compressed(os.path.join(HERE, "gemmlowp_s32.npz"), **out)


def gemmlowp_batched():
    rng = np.random.default_rng(102)
    out = {}
    for n, (batch, M, N, K, bb) in enumerate(BATCHED):
        signed = n % 2
        A = rnd8(rng, (batch, M, K), signed)
        B = rnd8(rng, (batch, K, N) if bb else (K, N), signed)
        ao, bo = int(rng.integers(-20, 20)), int(rng.integers(-20, 20))
        out["a%d" % n], out["b%d" % n] = A, B
        out["off%d" % n] = np.array([ao, bo], dtype=np.int32)
        out["dst%d" % n] = oracle.ref_gemmlowp_core(A, B, ao, bo)
    out["count"] = np.array(len(BATCHED))
    np.savez_compressed(os.path.join(HERE, "gemmlowp_batched.npz"), **out)


def fused_fixedpoint():
    """GEMM (reference core) -> + bias -> FIXEDPOINT stage (reference), per tensor and per channel."""
    rng = np.random.default_rng(103)
    out = {}
    n = 0
    for signed in (0, 1):
        lo_t, hi_t = (-128, 127) if signed else (0, 255)
        for idx, (M, N, K) in enumerate(FUSED_SHAPES):
            for per_channel in (0, 1):
                if per_channel and not signed:
                    continue  # per-channel weights are QSYMM8_PER_CHANNEL (int8) with b_offset 0
                A, B = rnd8(rng, (M, K), signed), rnd8(rng, (K, N), signed)
                ao = int(rng.integers(-128, 128))
                bo = 0 if per_channel else int(rng.integers(-128, 128))
                bias = rng.integers(-2000, 2000, size=N, dtype=np.int32)
                if per_channel:
                    reals = np.exp(rng.uniform(np.log(1e-4), np.log(2.0), size=N)).astype(np.float32)
                else:
                    reals = np.array([REALS[(idx + signed) % len(REALS)]], dtype=np.float32)
                ms = [oracle.ref_calculate_quantized_multiplier(float(r)) for r in reals]
                mult = np.array([p[0] for p in ms], dtype=np.int32)
                shift = np.array([p[1] for p in ms], dtype=np.int32)
                roff = int(rng.integers(-20, 20)) if signed else int(rng.integers(0, 40))
                # bounds: the type range, or a RELU-style tightening inside it
                lo, hi = (lo_t, hi_t) if idx % 2 == 0 else (max(lo_t, roff), hi_t - 7)
                t = oracle.ref_gemmlowp_core(A, B, ao, bo)
                dst = oracle.ref_quantize_down_fixedpoint(t, bias, mult, shift, roff, lo, hi,
                                                          np.int8 if signed else np.uint8)
                for k, v in dict(a=A, b=B, bias=bias, mult=mult, shift=shift, dst=dst,
                                 p=np.array([ao, bo, roff, lo, hi, per_channel], dtype=np.int32)).items():
                    out["%s%d" % (k, n)] = v
                n += 1
    out["count"] = np.array(n)
    np.savez_compressed(os.path.join(HERE, "gemmlowp_fused_fixedpoint.npz"), **out)


def output_stage():
    """Stand-alone stage: S32 U[-6000,6000] + bias, as tests/validation/fixtures/GEMMLowpFixture.h:1255-1259."""
    rng = np.random.default_rng(104)
    out = {}
    n = 0
    for signed in (0, 1):
        lo_t, hi_t = (-128, 127) if signed else (0, 255)
        for (M, N) in [(1, 1), (7, 15), (13, 33), (5, 128), (3, 1000)]:
            for with_bias in (0, 1):
                src = rng.integers(-6000, 6001, size=(M, N), dtype=np.int32)
                bias = rng.integers(-6000, 6001, size=N, dtype=np.int32)
                mult, shift = oracle.ref_calculate_quantized_multiplier(float(rng.uniform(0.001, 0.9)))
                roff = int(rng.integers(-10, 10)) + (0 if signed else 100)
                lo, hi = (lo_t, hi_t) if n % 3 else (lo_t + 5, hi_t - 9)
                dst = oracle.ref_quantize_down_fixedpoint(src, bias if with_bias else None, [mult], [shift], roff, lo,
                                                          hi, np.int8 if signed else np.uint8)
                out["src%d" % n], out["bias%d" % n], out["dst%d" % n] = src, bias, dst
                out["p%d" % n] = np.array([mult, shift, roff, lo, hi, with_bias], dtype=np.int32)
                n += 1
    out["count"] = np.array(n)
    np.savez_compressed(os.path.join(HERE, "output_stage.npz"), **out)


def output_stage_scale():
    """QUANTIZE_DOWN with an integer multiplier, stand-alone: S32 input + bias through the reference's
    gemmlowp_quantize_down_scale (tests/validation/reference/GEMMLowp.cpp:66-104), shapes / value ranges of
    tests/validation/fixtures/GEMMLowpFixture.h (GEMMLowpQuantizeDownInt32ScaleValidationFixture), per tensor and per
    column, with and without bounds (min == max means none)."""
    rng = np.random.default_rng(110)
    out = {}
    n = 0
    for signed in (0, 1):
        lo_t, hi_t = (-128, 127) if signed else (0, 255)
        for (M, N) in [(1, 1), (7, 15), (13, 33), (5, 128), (3, 1000)]:
            for variant in range(3):
                src = rng.integers(-60000, 60001, size=(M, N), dtype=np.int32)
                bias = rng.integers(-6000, 6001, size=N, dtype=np.int32)
                per_channel = variant == 2
                cnt = N if per_channel else 1
                mult = rng.integers(1, 300, size=cnt).astype(np.int32)
                shift = rng.integers(4, 17, size=cnt).astype(np.int32)
                roff = int(rng.integers(-3000, 3000))
                lo, hi = (0, 0) if variant == 0 else (lo_t + 5, hi_t - 9)
                with_bias = (n + variant) % 2
                dst = oracle.ref_quantize_down_scale(src, bias if with_bias else None, mult, shift, roff, lo, hi,
                                                     np.int8 if signed else np.uint8)
                out["src%d" % n], out["bias%d" % n], out["dst%d" % n] = src, bias, dst
                out["mult%d" % n], out["shift%d" % n] = mult, shift
                out["p%d" % n] = np.array([roff, lo, hi, with_bias], dtype=np.int32)
                n += 1
    out["count"] = np.array(n)
    np.savez_compressed(os.path.join(HERE, "output_stage_scale.npz"), **out)


def requant_sweep():
    """The scalar primitive on inputs for which the reference's int arithmetic has no signed overflow."""
    rng = np.random.default_rng(105)
    r = oracle.ref()
    v = np.concatenate([np.array([-(1 << 30), -65537, -65536, -3, -2, -1, 0, 1, 2, 3, 65535, 65536, 1 << 30]),
                        rng.integers(-(1 << 30), 1 << 30, size=120),
                        rng.integers(-70000, 70000, size=120)]).astype(np.int32)
    mults = np.array([1 << 30, 1518500250, (1 << 31) - 1, 1073741825, 1539316224], dtype=np.int32)
    rows = []
    for m in mults:
        for s in range(-4, 32):
            vv = v if s >= 0 else v[np.abs(v.astype(np.int64)) < (1 << (30 + s))]  # no overflow of v * 2^-s
            res = np.array([r.ref_quantize_down_scalar(int(x), int(m), s, 0, -(1 << 31), (1 << 31) - 1) for x in vv],
                           dtype=np.int32)
            rows.append(np.stack([vv, np.full_like(vv, m), np.full_like(vv, s), res], axis=1))
    tab = np.concatenate(rows, axis=0)
    hi = np.array([[x, m, r.ref_asymm_int_mult(int(x), int(m))] for x in v for m in mults], dtype=np.int32)
    np.savez_compressed(os.path.join(HERE, "requant_sweep.npz"), table=tab, sqdmulh=hi)


def quant_multiplier():
    rng = np.random.default_rng(106)
    reals = np.concatenate([
        np.exp(rng.uniform(np.log(1e-6), np.log(8.0), size=4096)),
        2.0 ** np.arange(-20, 4), [0.99999994, 0.9999999, 1.0000001, 0.5, 0.25, 0.0007, 1e-4, 1e-3],
    ]).astype(np.float32)
    ms = np.array([oracle.ref_calculate_quantized_multiplier(float(x)) for x in reals], dtype=np.int32)
    np.savez_compressed(os.path.join(HERE, "quant_multiplier.npz"), real=reals, mult=ms[:, 0], shift=ms[:, 1])


def f32_dequant():
    """The reference's test oracle for the F32 output: dequantize(t) with scale a.scale*b.scale
    (tests/validation/fixtures/GEMMLowpFixture.h:868-910), scales 1/255 and 5/255 (:830-831)."""
    rng = np.random.default_rng(107)
    out = {}
    scale = np.float32(np.float32(1.0 / 255) * np.float32(5.0 / 255))
    cases = [(M, N, K, ao, bo) for (M, N, K, ao, bo) in SMALL_GEMMLOWP] + [(5, 9, 1000, 0, 0), (4, 17, 1000, 3, -4)]
    for n, (M, N, K, ao, bo) in enumerate(cases):
        A, B = rnd8(rng, (M, K), 1), rnd8(rng, (K, N), 1)
        t = oracle.ref_gemmlowp_core(A, B, ao, bo)
        out["a%d" % n], out["b%d" % n] = A, B
        out["off%d" % n] = np.array([ao, bo], dtype=np.int32)
        out["dst%d" % n] = oracle.ref_dequantize_s32(t, float(scale))
    out["count"] = np.array(len(cases))
    out["scale"] = np.array(scale, dtype=np.float32)
    np.savez_compressed(os.path.join(HERE, "gemmlowp_f32.npz"), **out)


def f16_dequant():
    """The reference's test oracle for the F16 output (tests/validation/fixtures/GEMMLowpFixture.h:908-920): the S32
    result dequantised to half with scale a.scale*b.scale, and, when accumulating, added to the previous halfs as halfs.
    Signed operands (tests/validation/NEON/GEMMLowp.cpp:598-621), with and without offsets and previous contents."""
    rng = np.random.default_rng(116)
    out = {}
    scale = np.float32(np.float32(1.0 / 255) * np.float32(5.0 / 255))
    cases = [(M, N, K, 0, 0) for (M, N, K, _, _) in SMALL_GEMMLOWP] + [(37, 53, 120, 0, 0), (5, 9, 1000, 0, 0),
                                                                      (37, 53, 120, 3, -7), (27, 23, 31, 5, 13)]
    for n, (M, N, K, ao, bo) in enumerate(cases):
        A, B = rnd8(rng, (M, K), 1), rnd8(rng, (K, N), 1)
        prev = rng.normal(0, 2, size=(M, N)).astype(np.float16)
        t = oracle.ref_gemmlowp_core(A, B, ao, bo)
        out["a%d" % n], out["b%d" % n], out["prev%d" % n] = A, B, prev
        out["off%d" % n] = np.array([ao, bo], dtype=np.int32)
        out["dst%d" % n] = oracle.ref_dequantize_s32_f16(t, float(scale)).view(np.uint16)
        out["acc%d" % n] = oracle.ref_dequantize_s32_f16(t, float(scale), prev=prev).view(np.uint16)
    out["count"] = np.array(len(cases))
    out["scale"] = np.array(scale, dtype=np.float32)
    np.savez_compressed(os.path.join(HERE, "gemmlowp_f16.npz"), **out)


IM2COL = [  # (batch, H, W, C, KH, KW, (sx, sy), (pl, pt, pr, pb), zero_point)
    (1, 5, 5, 3, 3, 3, (1, 1), (1, 1, 1, 1), 10), (2, 7, 6, 1, 3, 3, (2, 2), (0, 0, 0, 0), 0),
    (1, 6, 6, 64, 1, 1, (1, 1), (0, 0, 0, 0), -1), (1, 9, 8, 3, 5, 5, (1, 1), (2, 2, 2, 2), -1),
    (2, 8, 8, 64, 3, 3, (1, 1), (1, 1, 1, 1), -1), (1, 7, 9, 5, 3, 3, (2, 1), (1, 0, 1, 0), 3),
]


def im2col():
    rng = np.random.default_rng(108)
    out = {}
    for n, (b, H, W, Cc, KH, KW, st, pad, zp) in enumerate(IM2COL):
        src = rnd8(rng, (b, H, W, Cc), 1)
        out["src%d" % n] = src
        out["p%d" % n] = np.array([KH, KW, st[0], st[1], pad[0], pad[1], pad[2], pad[3], zp], dtype=np.int32)
        out["dst%d" % n] = oracle.ref_im2col_nhwc(src, KH, KW, st, pad, zp)
    out["count"] = np.array(len(IM2COL))
    np.savez_compressed(os.path.join(HERE, "im2col_nhwc.npz"), **out)


CONV = [  # (batch, H, W, C, OFM, KH, KW, (sx, sy), (pl, pt, pr, pb), signed, per_channel)
    (1, 4, 4, 2, 2, 3, 3, (1, 1), (1, 1, 1, 1), 1, 0), (2, 5, 7, 3, 4, 3, 3, (1, 1), (1, 1, 1, 1), 0, 0),
    (1, 27, 23, 5, 2, 3, 3, (2, 1), (0, 0, 0, 0), 0, 0), (2, 8, 8, 64, 64, 3, 3, (1, 1), (1, 1, 1, 1), 1, 1),
    (1, 9, 9, 8, 16, 3, 3, (1, 1), (1, 1, 1, 1), 0, 1), (1, 6, 6, 16, 8, 1, 1, (1, 1), (0, 0, 0, 0), 1, 1),
    (1, 11, 10, 4, 6, 5, 5, (2, 2), (2, 2, 2, 2), 1, 0),
]


def conv():
    rng = np.random.default_rng(109)
    out = {}
    for n, (b, H, W, Cc, OFM, KH, KW, st, pad, signed, pc) in enumerate(CONV):
        src = rnd8(rng, (b, H, W, Cc), signed)
        w = np.clip(np.rint(rng.normal(0, 24, size=(OFM, KH, KW, Cc))), -127, 127).astype(np.int8) if (pc or signed) \
            else rnd8(rng, (OFM, KH, KW, Cc), 0)
        bias = np.rint(rng.normal(0, 500, size=OFM)).astype(np.int32)
        in_scale, out_scale = np.float32(rng.uniform(0.01, 0.05)), np.float32(rng.uniform(0.5, 3.0))
        in_zp = int(rng.integers(-5, 5)) + (0 if signed else 120)
        out_zp = int(rng.integers(-5, 5)) + (0 if signed else 120)
        # per-channel weight scales drawn as the reference fixture does: U(0.01, 1)
        # (tests/validation/fixtures/ConvolutionLayerFixture.h:937-946)
        w_scales = rng.uniform(0.01, 1.0, size=OFM).astype(np.float32) if pc else np.array(
            [rng.uniform(0.01, 0.1)], dtype=np.float32)
        w_zp = 0 if (pc or signed) else int(rng.integers(100, 140))
        dst = oracle.ref_conv_nhwc_quantized(src, w, bias, float(in_scale), in_zp, w_scales, w_zp, float(out_scale),
                                             out_zp, st, pad, (1, 1), bool(pc))
        out["src%d" % n], out["w%d" % n], out["bias%d" % n], out["dst%d" % n] = src, w, bias, dst
        out["wscale%d" % n] = w_scales
        out["scales%d" % n] = np.array([in_scale, out_scale], dtype=np.float32)
        out["p%d" % n] = np.array([st[0], st[1], pad[0], pad[1], pad[2], pad[3], in_zp, w_zp, out_zp, pc],
                                  dtype=np.int32)
    out["count"] = np.array(len(CONV))
    np.savez_compressed(os.path.join(HERE, "conv_nhwc.npz"), **out)


if __name__ == "__main__":
    assert oracle.ref_available(), "build oracle/_ref first (make -C oracle ref)"
    every = (gemmlowp_s32, gemmlowp_batched, fused_fixedpoint, output_stage, output_stage_scale, requant_sweep,
             quant_multiplier, f32_dequant, f16_dequant, im2col, conv)
    # python tests/golden/make_fixtures.py [name ...]: only the named fixtures (all of them without arguments)
    for fn in [f for f in every if not sys.argv[1:] or f.__name__ in sys.argv[1:]]:
        fn()
        print("wrote", fn.__name__)
