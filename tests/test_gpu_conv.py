"""GPU parity of the convolution lowering (implicit GEMM and explicit im2col + GEMM) and the im2col kernel."""
import numpy as np
import pytest

import oracle
from computelibrary_amd import capi
from gpu_util import announce, to_dev

pytestmark = pytest.mark.gpu
CODE = {np.dtype(np.uint8): capi.U8, np.dtype(np.int8): capi.S8}


def run_conv(src, w, bias, in_zp, w_zp, mult, shift, out_zp, lo, hi, stride, pad, dilation=(1, 1), path=0,
             device=True, layout=capi.NHWC):
    """src [batch][H][W][C], w [OFM][KH][KW][C]; with layout NCHW they are handed over (and the result comes back)
    channel-planar, and the NHWC view of the result is returned"""
    B_, H, W, C = src.shape
    OFM, KH, KW, _ = w.shape
    if layout == capi.NCHW:
        src, w = np.ascontiguousarray(src.transpose(0, 3, 1, 2)), np.ascontiguousarray(w.transpose(0, 3, 1, 2))
    pc = len(np.atleast_1d(mult)) > 1
    rq = capi.requant(0 if pc else int(np.atleast_1d(mult)[0]), 0 if pc else int(np.atleast_1d(shift)[0]), out_zp, lo,
                      hi, pc)
    d = capi.conv_desc(B_, H, W, C, OFM, KH, KW, stride, pad, dilation, CODE[src.dtype], CODE[w.dtype],
                       CODE[src.dtype], -in_zp, -w_zp, in_zp, rq, path, layout)
    cv = capi.Conv(d)
    OH, OW = cv.out_dims()
    m = np.ascontiguousarray(mult, dtype=np.int32) if pc else None
    s = np.ascontiguousarray(shift, dtype=np.int32) if pc else None
    b = np.ascontiguousarray(bias, dtype=np.int32)
    out = np.zeros((B_, OH, OW, OFM) if layout == capi.NHWC else (B_, OFM, OH, OW), dtype=src.dtype)
    if device:
        import torch
        sd, wd, od = to_dev(src), to_dev(w), to_dev(out)
        keep = [to_dev(b), to_dev(m), to_dev(s)]
        cv.prepare(wd, *keep)
        cv.run(sd, od)
        torch.cuda.synchronize()
        out = od.cpu().numpy()
    else:
        cv.prepare(np.ascontiguousarray(w), b, m, s)
        cv.run(np.ascontiguousarray(src), out)
    name = cv.kernel_name
    cv.close()
    if layout == capi.NCHW:
        out = out.transpose(0, 2, 3, 1)
    return out, name


def test_im2col_fixture(golden):
    g = golden("im2col_nhwc.npz")
    for n in range(int(g["count"])):
        KH, KW, sx, sy, pl, pt, pr, pb, zp = (int(x) for x in g["p%d" % n])
        src, want = g["src%d" % n], g["dst%d" % n]
        B_, H, W, C = src.shape
        d = capi.conv_desc(B_, H, W, C, 1, KH, KW, (sx, sy), (pl, pt, pr, pb), pad_value=zp)
        for device in (False, True):
            announce("im2col fixture", n, src.shape, "device", device)
            if device:
                out = to_dev(np.zeros_like(want))
                capi.im2col_nhwc(d, to_dev(src), out)
                got = out.cpu().numpy()
            else:
                got = np.zeros_like(want)
                capi.im2col_nhwc(d, np.ascontiguousarray(src), got)
            np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("path", [0, 1])
def test_conv_fixture(golden, path):
    g = golden("conv_nhwc.npz")
    names = set()
    for n in range(int(g["count"])):
        sx, sy, pl, pt, pr, pb, in_zp, w_zp, out_zp, pc = (int(x) for x in g["p%d" % n])
        src, w, bias, want = g["src%d" % n], g["w%d" % n], g["bias%d" % n], g["dst%d" % n]
        in_scale, out_scale = g["scales%d" % n]
        mult, shift = oracle.calculate_quantized_multipliers(in_scale, g["wscale%d" % n], out_scale)
        lo, hi = (-128, 127) if src.dtype == np.int8 else (0, 255)
        for device in (True, False):
            announce("conv fixture", n, src.shape, w.shape, "path", path, "device", device)
            got, name = run_conv(src, w, bias, in_zp, w_zp, mult, shift, out_zp, lo, hi, (sx, sy), (pl, pt, pr, pb),
                                 path=path, device=device)
            names.add(name.split("_")[0].split("+")[0])
            np.testing.assert_array_equal(got, want)
    if path == 0:
        assert "implicit" in names  # the 64-channel cases really took the on-the-fly loader


def test_conv_seeded_strides_dilation_uint8():
    rng = np.random.default_rng(51)
    for (shape, wshape, stride, pad, dil, dt) in [
            ((2, 13, 11, 32), (24, 3, 3, 32), (2, 1), (1, 1, 1, 1), (1, 1), np.uint8),
            ((1, 12, 12, 16), (40, 3, 3, 16), (1, 1), (2, 2, 2, 2), (2, 2), np.int8),
            ((3, 9, 7, 48), (64, 1, 1, 48), (1, 1), (0, 0, 0, 0), (1, 1), np.int8),
            ((1, 10, 10, 6), (7, 3, 3, 6), (1, 1), (1, 1, 1, 1), (1, 1), np.int8)]:
        src = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max + 1, size=shape).astype(dt)
        w = rng.integers(-127, 128, size=wshape).astype(np.int8)
        bias = rng.integers(-500, 500, size=wshape[0], dtype=np.int32)
        mult, shift = oracle.calculate_quantized_multipliers(0.02, rng.uniform(0.01, 1, wshape[0]), 1.1)
        zp = 5 if dt == np.int8 else 131
        lo, hi = (-128, 127) if dt == np.int8 else (0, 255)
        want = oracle.conv_nhwc_direct(src, w, bias, zp, 0, mult, shift, -5 if dt == np.int8 else 9, lo, hi, stride,
                                       pad, dil)
        for path in (0, 1):
            announce("conv seeded", shape, wshape, stride, pad, dil, "path", path)
            got, _ = run_conv(src, w, bias, zp, 0, mult, shift, -5 if dt == np.int8 else 9, lo, hi, stride, pad, dil,
                              path=path)
            np.testing.assert_array_equal(got, want)
        # the channel-planar layout gives the same integers (the reference's NCHW im2col only orders K differently)
        for device in (True, False):
            announce("conv seeded NCHW", shape, wshape, stride, pad, dil, "device", device)
            got, _ = run_conv(src, w, bias, zp, 0, mult, shift, -5 if dt == np.int8 else 9, lo, hi, stride, pad, dil,
                              device=device, layout=capi.NCHW)
            np.testing.assert_array_equal(got, want)


def test_conv_few_output_channels_kernel():
    """Up to 64 output channels and K = KH * KW * C <= 1152 with C a multiple of 16 run on the kernel that keeps the
    weights in LDS and reads the patches straight into the matrix cores' operand layout: 1 to 6 batches of 3 k blocks
    (K from 16 to 1152, with a last batch that is partly or mostly empty), C = 16 / 32 / 48 (a k block spans several
    taps) and 64 / 128 (one tap per k block), unsigned sources (flipped in the loader, non-zero padding value), strides,
    dilation, asymmetric padding, ragged channel counts, and row counts that do not fill the last workgroup; with K <= 192
    also 65 to 256 output channels as several panels of 64. Above those limits the tiled kernels take over."""
    rng = np.random.default_rng(77)
    cases = [
        # (src shape, weights shape, stride, pad, dilation, dtype)
        ((1, 5, 5, 16), (1, 1, 1, 16), (1, 1), (0, 0, 0, 0), (1, 1), np.int8),        # K = 16
        ((2, 9, 8, 16), (7, 3, 3, 16), (1, 1), (1, 1, 1, 1), (1, 1), np.uint8),       # K = 144, taps inside a k block
        ((1, 11, 13, 32), (63, 3, 3, 32), (2, 2), (1, 0, 2, 1), (1, 1), np.int8),     # K = 288
        ((2, 8, 8, 48), (64, 3, 3, 48), (1, 1), (2, 2, 2, 2), (2, 2), np.uint8),      # K = 432, dilation 2
        ((3, 14, 14, 64), (64, 3, 3, 64), (1, 1), (1, 1, 1, 1), (1, 1), np.int8),     # K = 576 (config 4's geometry)
        ((1, 7, 9, 128), (33, 3, 3, 128), (1, 2), (1, 1, 1, 1), (1, 1), np.uint8),    # K = 1152
        ((1, 6, 6, 64), (40, 4, 4, 64), (1, 1), (1, 1, 1, 1), (1, 1), np.int8),       # K = 1024
        ((2, 20, 20, 64), (64, 1, 1, 64), (1, 1), (0, 0, 0, 0), (1, 1), np.int8),     # K = 64, 800 rows
        ((1, 9, 9, 80), (16, 3, 3, 80), (1, 1), (1, 1, 1, 1), (1, 1), np.int8),       # K = 720, C = 80
        # more than one round of workgroups on every compute unit plus a few: the last rows go out in half-size
        # workgroups, the very last of them ragged (33708 = 256 * 128 + 14 * 64 + 32 + 12 rows; 33800 rows, 7 columns)
        ((3, 106, 106, 16), (64, 1, 1, 16), (1, 1), (0, 0, 0, 0), (1, 1), np.int8),
        ((2, 130, 130, 16), (7, 3, 3, 16), (1, 1), (1, 1, 1, 1), (1, 1), np.uint8),
        # K <= 192 and up to 256 output channels: 2 to 4 panels of 64 columns against the patch a wave keeps in registers
        ((2, 20, 20, 64), (256, 1, 1, 64), (1, 1), (0, 0, 0, 0), (1, 1), np.int8),     # 4 panels, K = 64
        ((1, 15, 14, 32), (96, 1, 1, 32), (1, 1), (0, 0, 0, 0), (1, 1), np.uint8),     # 2 panels, the second half empty
        ((2, 9, 8, 16), (65, 3, 3, 16), (1, 1), (1, 1, 1, 1), (1, 1), np.uint8),       # K = 144, 65 columns: one in the second panel
        ((1, 12, 12, 128), (130, 1, 1, 128), (2, 2), (0, 0, 0, 0), (1, 1), np.int8),   # K = 128, 3 panels, stride 2, N % 4 != 0
        ((1, 10, 10, 192), (200, 1, 1, 192), (1, 1), (0, 0, 0, 0), (1, 1), np.int8),   # K = 192, the most one batch holds
    ]
    for (shape, wshape, stride, pad, dil, dt) in cases:
        src = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max + 1, size=shape).astype(dt)
        w = rng.integers(-127, 128, size=wshape).astype(np.int8)
        bias = rng.integers(-500, 500, size=wshape[0], dtype=np.int32)
        K = wshape[1] * wshape[2] * wshape[3]
        zp = 5 if dt == np.int8 else 131
        lo, hi, ozp = (-128, 127, -5) if dt == np.int8 else (0, 255, 9)
        for per_channel in (True, False):
            reals = rng.uniform(0.5, 2.0, wshape[0] if per_channel else 1) * 40.0 / (K ** 0.5 * 74.0 * 74.0)
            mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
            if per_channel and wshape[0] > 2:
                mult[1], shift[1] = 1 << 29, -1   # a multiplier below 2^30 and a left shift: not the short form
            want = oracle.conv_nhwc_direct(src, w, bias, zp, 0, mult, shift, ozp, lo, hi, stride, pad, dil)
            announce("conv few channels", shape, wshape, stride, pad, dil, dt.__name__, "per_channel", per_channel)
            got, name = run_conv(src, w, bias, zp, 0, mult, shift, ozp, lo, hi, stride, pad, dil)
            assert name.startswith("implicit_narrow"), name
            np.testing.assert_array_equal(got, want)
            assert 0.1 < ((want > lo) & (want < hi)).mean()
    # 65 output channels, K = 1168: the tiled kernel
    for (shape, wshape) in [((1, 8, 8, 64), (65, 3, 3, 64)), ((1, 6, 6, 16), (8, 9, 9, 16))]:
        src = rng.integers(-128, 128, size=shape).astype(np.int8)
        w = rng.integers(-127, 128, size=wshape).astype(np.int8)
        bias = rng.integers(-500, 500, size=wshape[0], dtype=np.int32)
        mult, shift = oracle.calculate_quantized_multipliers(0.02, rng.uniform(0.01, 0.1, wshape[0]), 1.1)
        announce("conv beyond few channels", shape, wshape)
        got, name = run_conv(src, w, bias, 5, 0, mult, shift, -5, -128, 127, (1, 1), (4, 4, 4, 4))
        assert name.startswith("implicit_pp"), name
        np.testing.assert_array_equal(
            got, oracle.conv_nhwc_direct(src, w, bias, 5, 0, mult, shift, -5, -128, 127, (1, 1), (4, 4, 4, 4), (1, 1)))


def test_conv_few_output_channels_large_images_band_form():
    """With more than 4 tiles of 32 output pixels per compute unit (and C a power of two from 64 on) the kernel above
    gives way to the form in which one workgroup stages the window of input rows under a band of output rows in LDS -
    padding included - and every tap is an LDS address: bands that do not divide the image height, a last tile of
    a few pixels, signed and unsigned sources (non-zero padding values), asymmetric padding, strides, dilation, 40 and
    33 output channels, C = 64 / 128 / 256, a 1 x 1 kernel whose K ends before its batch of k blocks does, weights with an
    offset (row sums of the patches), requantisation constants outside the short form, and the F32 destination."""
    rng = np.random.default_rng(707)
    cases = [
        # (src shape, weights shape, stride, pad, dilation, src dtype, weights dtype, weights zero point)
        ((8, 72, 72, 64), (64, 3, 3, 64), (1, 1), (1, 1, 1, 1), (1, 1), np.int8, np.int8, 0),
        ((2, 150, 150, 64), (40, 3, 3, 64), (1, 1), (1, 0, 2, 1), (1, 1), np.uint8, np.int8, 0),
        ((4, 200, 190, 64), (64, 3, 3, 64), (2, 2), (1, 1, 1, 1), (1, 1), np.int8, np.int8, 0),
        ((2, 140, 140, 64), (33, 3, 3, 64), (1, 1), (2, 2, 2, 2), (2, 2), np.uint8, np.int8, 0),
        ((2, 132, 132, 128), (64, 3, 3, 128), (1, 1), (1, 1, 1, 1), (1, 1), np.int8, np.int8, 0),
        ((1, 190, 190, 256), (64, 1, 1, 256), (1, 1), (0, 0, 0, 0), (1, 1), np.int8, np.int8, 0),
        ((1, 420, 170, 64), (64, 2, 3, 64), (1, 2), (0, 1, 1, 0), (1, 1), np.uint8, np.uint8, 131),
    ]
    for (shape, wshape, stride, pad, dil, dt, w_dt, w_zp) in cases:
        src = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max + 1, size=shape).astype(dt)
        w = rng.integers(np.iinfo(w_dt).min + 1, np.iinfo(w_dt).max + 1, size=wshape).astype(w_dt)
        bias = rng.integers(-500, 500, size=wshape[0], dtype=np.int32)
        K = wshape[1] * wshape[2] * wshape[3]
        zp = 5 if dt == np.int8 else 131
        lo, hi, ozp = (-128, 127, -5) if dt == np.int8 else (0, 255, 9)
        for per_channel in (True, False):
            reals = rng.uniform(0.5, 2.0, wshape[0] if per_channel else 1) * 40.0 / (K ** 0.5 * 74.0 * 74.0)
            mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
            if per_channel and shape[0] == 2:
                mult[1], shift[1] = 1 << 29, -1   # a multiplier below 2^30 and a left shift: not the short form
            want = oracle.conv_nhwc_direct(src, w, bias, zp, w_zp, mult, shift, ozp, lo, hi, stride, pad, dil)
            assert 0.1 < ((want > lo) & (want < hi)).mean()
            announce("conv band form", shape, wshape, stride, pad, dil, dt.__name__, w_dt.__name__, w_zp, "per_channel", per_channel)
            got, name = run_conv(src, w, bias, zp, w_zp, mult, shift, ozp, lo, hi, stride, pad, dil)
            assert name == "implicit_band_32x64", name
            np.testing.assert_array_equal(got, want)
    # a result offset beyond what the 16-bit tail of the short form takes: the general short form, same bits
    src = rng.integers(-128, 128, size=(8, 72, 72, 64), dtype=np.int8)
    w = rng.integers(-127, 128, size=(64, 3, 3, 64), dtype=np.int8)
    bias = rng.integers(-500, 500, size=64, dtype=np.int32)
    mult, shift = oracle.calculate_quantized_multipliers(1.0, np.full(64, 40.0 / (24.0 * 74.0 * 74.0)), 1.0)
    import torch
    rq = capi.requant(0, 0, 3000, -32768, 32767, True)
    cv = capi.Conv(capi.conv_desc(8, 72, 72, 64, 64, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), capi.S8, capi.S8, capi.S8, -5, 0, 5, rq))
    sd, wd, od = to_dev(src), to_dev(w), to_dev(np.zeros((8, 72, 72, 64), np.int8))
    keep = [to_dev(bias), to_dev(mult), to_dev(shift)]
    cv.prepare(wd, *keep)
    announce("conv band form, large result offset", cv.kernel_name)
    cv.run(sd, od)
    torch.cuda.synchronize()
    assert cv.kernel_name == "implicit_band_32x64", cv.kernel_name
    np.testing.assert_array_equal(od.cpu().numpy(),
                                  oracle.conv_nhwc_direct(src, w, bias, 5, 0, mult, shift, 3000, -128, 127, (1, 1), (1, 1, 1, 1), (1, 1)))
    cv.close()
    # F32 destination
    src = rng.integers(-128, 128, size=(2, 140, 130, 64), dtype=np.int8)
    w = rng.integers(-127, 128, size=(48, 3, 3, 64), dtype=np.int8)
    bias_f = rng.normal(0.0, 2.0, size=48).astype(np.float32)
    scale = float(np.float32(0.02) * np.float32(0.005))
    cols = oracle.im2col_nhwc(src, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 4)
    want = oracle.gemmlowp_f32(cols, oracle.weights_reshape(w), bias_f, -4, 0, scale, 0.0, 6.0, act_twice=False)
    cv = capi.Conv(capi.conv_desc(2, 140, 130, 64, 48, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), capi.S8, capi.S8, capi.F32, -4, 0, 4,
                                  scale=scale, act=(0.0, 6.0)))
    sd, wd, od, bd = to_dev(src), to_dev(w), to_dev(np.zeros((2, 140, 130, 48), np.float32)), to_dev(bias_f)
    cv.prepare(wd, bd)
    announce("conv band form, F32 destination", cv.kernel_name)
    cv.run(sd, od)
    torch.cuda.synchronize()
    assert cv.kernel_name == "implicit_band_32x64", cv.kernel_name
    assert np.array_equal(od.cpu().numpy().reshape(-1, 48).view(np.uint32), want.view(np.uint32))
    cv.close()


def test_conv_band_form_several_column_panels():
    """Pointwise and small-patch convolutions of large images with more than 64 output channels and K <= 192: the band form
    keeps up to four panels of 64 columns in LDS and takes a wave's 32 pixels through one after the other. 256, 192, 130
    and 100 output channels (a ragged last panel, a channel count that is no multiple of 4), C = 64 and 128, a 1 x 3 patch
    with padding, stride 2, both source signs, weights with an offset, per-channel and per-tensor requantisation,
    constants outside the short form, and the F32 destination."""
    rng = np.random.default_rng(2560)
    cases = [
        # (src shape, weights shape, stride, pad, dilation, src dtype, weights dtype, weights zero point)
        ((4, 100, 100, 64), (256, 1, 1, 64), (1, 1), (0, 0, 0, 0), (1, 1), np.int8, np.int8, 0),
        ((2, 150, 140, 128), (192, 1, 1, 128), (1, 1), (0, 0, 0, 0), (1, 1), np.uint8, np.int8, 0),
        ((2, 400, 300, 64), (130, 1, 1, 64), (2, 2), (0, 0, 0, 0), (1, 1), np.int8, np.int8, 0),
        ((2, 160, 150, 64), (100, 1, 3, 64), (1, 1), (1, 1, 0, 0), (1, 1), np.uint8, np.uint8, 131),
    ]
    for (shape, wshape, stride, pad, dil, dt, w_dt, w_zp) in cases:
        src = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max + 1, size=shape).astype(dt)
        w = rng.integers(np.iinfo(w_dt).min + 1, np.iinfo(w_dt).max + 1, size=wshape).astype(w_dt)
        bias = rng.integers(-500, 500, size=wshape[0], dtype=np.int32)
        K = wshape[1] * wshape[2] * wshape[3]
        zp = 5 if dt == np.int8 else 131
        lo, hi, ozp = (-128, 127, -5) if dt == np.int8 else (0, 255, 9)
        for per_channel in (True, False):
            reals = rng.uniform(0.5, 2.0, wshape[0] if per_channel else 1) * 40.0 / (K ** 0.5 * 74.0 * 74.0)
            mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
            if per_channel and shape[0] == 2:
                mult[70], shift[70] = 1 << 29, -1   # a multiplier below 2^30 and a left shift: not the short form
            want = oracle.conv_nhwc_direct(src, w, bias, zp, w_zp, mult, shift, ozp, lo, hi, stride, pad, dil)
            assert 0.1 < ((want > lo) & (want < hi)).mean()
            announce("conv band form, several panels", shape, wshape, stride, pad, dil, dt.__name__, w_dt.__name__, w_zp, "per_channel", per_channel)
            got, name = run_conv(src, w, bias, zp, w_zp, mult, shift, ozp, lo, hi, stride, pad, dil)
            assert name == "implicit_band_32x64", name
            np.testing.assert_array_equal(got, want)
    # F32 destination, 160 channels
    import torch
    src = rng.integers(-128, 128, size=(2, 140, 130, 64), dtype=np.int8)
    w = rng.integers(-127, 128, size=(160, 1, 1, 64), dtype=np.int8)
    bias_f = rng.normal(0.0, 2.0, size=160).astype(np.float32)
    scale = float(np.float32(0.02) * np.float32(0.005))
    cols = oracle.im2col_nhwc(src, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), 4)
    want = oracle.gemmlowp_f32(cols, oracle.weights_reshape(w), bias_f, -4, 0, scale, 0.0, 6.0, act_twice=False)
    cv = capi.Conv(capi.conv_desc(2, 140, 130, 64, 160, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), capi.S8, capi.S8, capi.F32, -4, 0, 4,
                                  scale=scale, act=(0.0, 6.0)))
    sd, wd, od, bd = to_dev(src), to_dev(w), to_dev(np.zeros((2, 140, 130, 160), np.float32)), to_dev(bias_f)
    cv.prepare(wd, bd)
    announce("conv band form, several panels, F32 destination", cv.kernel_name)
    cv.run(sd, od)
    torch.cuda.synchronize()
    assert cv.kernel_name == "implicit_band_32x64", cv.kernel_name
    assert np.array_equal(od.cpu().numpy().reshape(-1, 160).view(np.uint32), want.view(np.uint32))
    cv.close()


def test_conv_deep_patches_under_few_tiles_run_as_k_slices():
    """Few output tiles under a deep patch (the last 3 x 3 layers of a classifier: 14 x 14 or 7 x 7 pixels, 512 channels):
    the K range of the on-the-fly loader runs as slices along the grid of one S32 launch and a second kernel sums the
    planes and applies the epilogue, as for a dense product: strides, padding, dilation, both source signs, weights with
    an offset (row sums of the patches), per-channel and per-tensor requantisation; the explicit lowering (patches
    written out, then the dense product with its own slices) gives the same bits."""
    rng = np.random.default_rng(4608)
    for (shape, wshape, stride, pad, dil, dt, w_dt, w_zp) in [
            ((1, 14, 14, 512), (96, 3, 3, 512), (1, 1), (1, 1, 1, 1), (1, 1), np.int8, np.int8, 0),
            ((2, 9, 7, 256), (130, 3, 3, 256), (1, 1), (2, 2, 2, 2), (2, 2), np.uint8, np.int8, 0),
            ((1, 15, 15, 512), (200, 2, 2, 512), (2, 2), (0, 1, 1, 0), (1, 1), np.uint8, np.uint8, 131),
            ((3, 7, 7, 2048), (80, 1, 1, 2048), (1, 1), (0, 0, 0, 0), (1, 1), np.int8, np.int8, 0)]:
        src = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max + 1, size=shape).astype(dt)
        w = rng.integers(np.iinfo(w_dt).min + 1, np.iinfo(w_dt).max + 1, size=wshape).astype(w_dt)
        bias = rng.integers(-500, 500, size=wshape[0], dtype=np.int32)
        K = wshape[1] * wshape[2] * wshape[3]
        zp = 5 if dt == np.int8 else 131
        lo, hi, ozp = (-128, 127, -5) if dt == np.int8 else (0, 255, 9)
        for per_channel in (True, False):
            reals = rng.uniform(0.5, 2.0, wshape[0] if per_channel else 1) * 40.0 / (K ** 0.5 * 74.0 * 74.0)
            mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
            want = oracle.conv_nhwc_direct(src, w, bias, zp, w_zp, mult, shift, ozp, lo, hi, stride, pad, dil)
            assert 0.1 < ((want > lo) & (want < hi)).mean()
            for path in (capi.CONV_AUTO, capi.CONV_EXPLICIT):
                announce("conv k slices", shape, wshape, stride, pad, dil, dt.__name__, w_dt.__name__, w_zp, "per_channel", per_channel,
                         "path", path)
                got, name = run_conv(src, w, bias, zp, w_zp, mult, shift, ozp, lo, hi, stride, pad, dil, path=path)
                assert "_splitk" in name and name.startswith("implicit" if path == capi.CONV_AUTO else "im2col"), name
                np.testing.assert_array_equal(got, want)
    # the dequantising (F32) destination through the same slices
    import torch
    src = rng.integers(-128, 128, size=(1, 14, 14, 512), dtype=np.int8)
    w = rng.integers(-127, 128, size=(96, 3, 3, 512), dtype=np.int8)
    bias_f = rng.normal(0.0, 2.0, size=96).astype(np.float32)
    scale = float(np.float32(0.02) * np.float32(0.005))
    cols = oracle.im2col_nhwc(src, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 4)
    want = oracle.gemmlowp_f32(cols, oracle.weights_reshape(w), bias_f, -4, 0, scale, 0.0, 6.0, act_twice=False)
    cv = capi.Conv(capi.conv_desc(1, 14, 14, 512, 96, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), capi.S8, capi.S8, capi.F32, -4, 0, 4,
                                  scale=scale, act=(0.0, 6.0)))
    sd, wd, od, bd = to_dev(src), to_dev(w), to_dev(np.zeros((1, 14, 14, 96), np.float32)), to_dev(bias_f)
    cv.prepare(wd, bd)
    announce("conv k slices, F32 destination", cv.kernel_name)
    cv.run(sd, od)
    torch.cuda.synchronize()
    assert "_splitk" in cv.kernel_name, cv.kernel_name
    assert np.array_equal(od.cpu().numpy().reshape(-1, 96).view(np.uint32), want.view(np.uint32))
    cv.close()


def test_conv_channel_counts_padded_to_16():
    """A channel count that is not a multiple of 16: pixels and taps are copied with the channels padded to the next
    multiple of 16 and the fast implicit kernels run (never the byte-wise fallback), with identical results - the RGB of
    a first layer (7 x 7 stride 2, 3 x 3 stride 2), 1, 4, 5, 8, 24 and 40 channels, few and many output channels, both
    source signs with non-zero source offsets and padding values, symmetric weights and weights with an offset (the row
    sums of the patches then come from the unpadded source and the constant term from the unpadded K), asymmetric
    padding, dilation, both layouts, per-channel and per-tensor requantisation, a later change of both offsets. With the
    padding switched off the byte-wise loader gives the same bits."""
    rng = np.random.default_rng(99)
    cases = [
        # (src shape, weights shape, stride, pad, dilation, src dtype, weights dtype, weights zero point, layout)
        ((2, 30, 28, 3), (64, 7, 7, 3), (2, 2), (3, 3, 3, 3), (1, 1), np.uint8, np.int8, 0, capi.NHWC),
        ((1, 17, 19, 3), (32, 3, 3, 3), (2, 2), (1, 1, 1, 1), (1, 1), np.int8, np.uint8, 128, capi.NHWC),
        ((2, 9, 9, 1), (5, 3, 3, 1), (1, 1), (1, 0, 1, 2), (1, 1), np.uint8, np.int8, 0, capi.NHWC),
        ((1, 12, 10, 4), (70, 5, 5, 4), (1, 2), (2, 2, 2, 2), (1, 1), np.int8, np.int8, 0, capi.NCHW),
        ((2, 8, 8, 8), (16, 3, 3, 8), (1, 1), (2, 2, 2, 2), (2, 2), np.uint8, np.uint8, 128, capi.NHWC),
        ((1, 14, 14, 24), (64, 3, 3, 24), (1, 1), (1, 1, 1, 1), (1, 1), np.int8, np.int8, 0, capi.NHWC),
        ((3, 7, 7, 40), (120, 1, 1, 40), (1, 1), (0, 0, 0, 0), (1, 1), np.uint8, np.int8, 0, capi.NCHW),
        ((3, 6, 6, 5), (9, 1, 1, 5), (1, 1), (0, 0, 0, 0), (1, 1), np.uint8, np.uint8, 7, capi.NHWC),
        ((2, 9, 8, 3), (20, 3, 3, 3), (1, 1), (1, 1, 1, 1), (1, 1), np.int8, np.int8, -4, capi.NHWC),
        ((1, 11, 9, 20), (70, 2, 3, 20), (1, 2), (0, 1, 1, 0), (2, 1), np.uint8, np.uint8, 131, capi.NCHW),
    ]
    for (shape, wshape, stride, pad, dil, dt, w_dt, w_zp, layout) in cases:
        src = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max + 1, size=shape).astype(dt)
        w = rng.integers(np.iinfo(w_dt).min + 1, np.iinfo(w_dt).max + 1, size=wshape).astype(w_dt)
        bias = rng.integers(-500, 500, size=wshape[0], dtype=np.int32)
        K = wshape[1] * wshape[2] * wshape[3]
        zp = 5 if dt == np.int8 else 131
        lo, hi, ozp = (-128, 127, -5) if dt == np.int8 else (0, 255, 9)
        for per_channel in (True, False):
            reals = rng.uniform(0.5, 2.0, wshape[0] if per_channel else 1) * 40.0 / (K ** 0.5 * 74.0 * 74.0)
            mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
            want = oracle.conv_nhwc_direct(src, w, bias, zp, w_zp, mult, shift, ozp, lo, hi, stride, pad, dil)
            assert 0.1 < ((want > lo) & (want < hi)).mean()
            announce("conv padded channels", shape, wshape, stride, pad, dil, dt.__name__, w_dt.__name__, "w_zp", w_zp, "layout", layout,
                     per_channel)
            got, name = run_conv(src, w, bias, zp, w_zp, mult, shift, ozp, lo, hi, stride, pad, dil, layout=layout)
            assert name.startswith("implicit_") and "mfma" not in name, name
            np.testing.assert_array_equal(got, want)
    # the byte-wise loader instead (the convolution on the caller's channel count, no padded copy): the same bits
    for (shape, wshape, stride, pad, dil, dt, w_dt, w_zp, layout) in cases[:2] + cases[7:9]:
        src = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max + 1, size=shape).astype(dt)
        w = rng.integers(np.iinfo(w_dt).min + 1, np.iinfo(w_dt).max + 1, size=wshape).astype(w_dt)
        bias = rng.integers(-500, 500, size=wshape[0], dtype=np.int32)
        mult, shift = oracle.calculate_quantized_multiplier(float(40.0 / ((wshape[1] * wshape[2] * wshape[3]) ** 0.5 * 74.0 * 74.0)))
        zp = 5 if dt == np.int8 else 131
        lo, hi, ozp = (-128, 127, -5) if dt == np.int8 else (0, 255, 9)
        want = oracle.conv_nhwc_direct(src, w, bias, zp, w_zp, [mult], [shift], ozp, lo, hi, stride, pad, dil)
        announce("conv byte-wise loader", shape, wshape)
        got, name = run_conv(src, w, bias, zp, w_zp, [mult], [shift], ozp, lo, hi, stride, pad, dil, layout=layout,
                             path=capi.CONV_IN_PLACE)
        assert name.startswith("implicit_mfma"), name
        np.testing.assert_array_equal(got, want)
    # a handle that pads, after a change of both offsets and of the padding value
    src = rng.integers(-128, 128, size=(2, 7, 6, 3), dtype=np.int8)
    w = rng.integers(-127, 128, size=(8, 3, 3, 3), dtype=np.int8)
    bias = rng.integers(-500, 500, size=8, dtype=np.int32)
    mult, shift = oracle.calculate_quantized_multiplier(float(40.0 / (27 ** 0.5 * 74.0 * 74.0)))
    cv = capi.Conv(capi.conv_desc(2, 7, 6, 3, 8, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), capi.S8, capi.S8, capi.S8, -2, 0, 2,
                                  capi.requant(mult, shift, 1, -128, 127)))
    sd, wd, od = to_dev(src), to_dev(w), to_dev(np.zeros((2, 7, 6, 8), np.int8))
    keep = to_dev(bias)
    cv.prepare(wd, keep)
    for (in_zp, w_zp) in ((2, 0), (-6, 9)):
        if w_zp:
            cv.update_quant(-in_zp, -w_zp, in_zp, capi.requant(mult, shift, 1, -128, 127))
        cv.run(sd, od)
        import torch
        torch.cuda.synchronize()
        announce("conv padded channels, offsets", in_zp, w_zp, cv.kernel_name)
        np.testing.assert_array_equal(od.cpu().numpy(), oracle.conv_nhwc_direct(src, w, bias, in_zp, w_zp, [mult], [shift], 1, -128, 127,
                                                                                  (1, 1), (1, 1, 1, 1), (1, 1)))
    cv.close()


def test_conv_weights_offset_and_odd_channels_on_the_fly():
    """QASYMM8 weights with a non-zero offset need the row sums of the patch matrix (a pass over the source, padding
    included); channel counts that are not a multiple of 16 run with their channels padded (the test above): neither
    materialises the patches.
    Few and many output channels (both kernels), unsigned and signed sources."""
    rng = np.random.default_rng(88)
    for (shape, wshape, stride, pad, dil, dt, w_zp) in [
            ((2, 9, 8, 16), (24, 3, 3, 16), (1, 1), (1, 1, 1, 1), (1, 1), np.uint8, 131),
            ((1, 12, 11, 64), (80, 3, 3, 64), (2, 1), (1, 0, 1, 2), (1, 1), np.uint8, 120),
            ((2, 7, 7, 3), (8, 3, 3, 3), (1, 1), (1, 1, 1, 1), (1, 1), np.uint8, 128),
            ((1, 10, 9, 20), (70, 2, 3, 20), (1, 2), (0, 1, 1, 0), (2, 1), np.int8, 0),
            ((3, 6, 6, 5), (9, 1, 1, 5), (1, 1), (0, 0, 0, 0), (1, 1), np.uint8, 7)]:
        src = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max + 1, size=shape).astype(dt)
        w_dt = np.uint8 if w_zp else np.int8
        w = rng.integers(np.iinfo(w_dt).min + (0 if w_zp else 1), np.iinfo(w_dt).max + 1, size=wshape).astype(w_dt)
        bias = rng.integers(-500, 500, size=wshape[0], dtype=np.int32)
        K = wshape[1] * wshape[2] * wshape[3]
        mult, shift = oracle.calculate_quantized_multiplier(float(40.0 / (K ** 0.5 * 74.0 * 74.0)))
        zp = 5 if dt == np.int8 else 131
        lo, hi, ozp = (-128, 127, -5) if dt == np.int8 else (0, 255, 9)
        want = oracle.conv_nhwc_direct(src, w, bias, zp, w_zp, [mult], [shift], ozp, lo, hi, stride, pad, dil)
        assert 0.1 < ((want > lo) & (want < hi)).mean()
        for device in (True, False):
            announce("conv offsets / odd channels", shape, wshape, stride, pad, dil, dt.__name__, "w_zp", w_zp, "device", device)
            got, name = run_conv(src, w, bias, zp, w_zp, [mult], [shift], ozp, lo, hi, stride, pad, dil, device=device)
            assert name.startswith("implicit_"), name
            np.testing.assert_array_equal(got, want)


def test_conv_nchw_fixture(golden):
    """The reference oracle's outputs (tests/golden/conv_nhwc.npz) with every tensor handed over channel-planar"""
    g = golden("conv_nhwc.npz")
    for n in range(int(g["count"])):
        sx, sy, pl, pt, pr, pb, in_zp, w_zp, out_zp, pc = (int(x) for x in g["p%d" % n])
        src, w, bias, want = g["src%d" % n], g["w%d" % n], g["bias%d" % n], g["dst%d" % n]
        in_scale, out_scale = g["scales%d" % n]
        mult, shift = oracle.calculate_quantized_multipliers(in_scale, g["wscale%d" % n], out_scale)
        lo, hi = (-128, 127) if src.dtype == np.int8 else (0, 255)
        announce("conv NCHW fixture", n, src.shape, w.shape)
        got, _ = run_conv(src, w, bias, in_zp, w_zp, mult, shift, out_zp, lo, hi, (sx, sy), (pl, pt, pr, pb),
                          layout=capi.NCHW)
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("device", [True, False])
def test_conv_tensors_padded_along_channels(device):
    """src, weights and dst with padding between pixels, as the reference's convolution fixture hands them over
    (add_padding_x, tests/validation/Helpers.cpp:335-357): same result, padding bytes of dst untouched."""
    import torch
    rng = np.random.default_rng(61)
    for (B_, H, W, C, OFM, KH, KW, sp, wp, dp) in [(2, 9, 8, 16, 24, 3, 3, 16 + 5, 16 + 9, 24 + 3),
                                                   (1, 7, 7, 6, 10, 3, 2, 6 + 16, 6 + 1, 10 + 7),
                                                   (2, 6, 6, 32, 32, 1, 1, 32 + 2, 32, 32 + 16)]:
        src = rng.integers(-128, 128, size=(B_, H, W, C), dtype=np.int8)
        w = rng.integers(-127, 128, size=(OFM, KH, KW, C), dtype=np.int8)
        bias = rng.integers(-500, 500, size=OFM, dtype=np.int32)
        mult, shift = oracle.calculate_quantized_multipliers(0.02, rng.uniform(0.01, 1, OFM), 1.1)
        pad = (1, 1, 1, 1) if KH == 3 else (0, 0, 0, 0)
        want = oracle.conv_nhwc_direct(src, w, bias, 4, 0, mult, shift, -5, -128, 127, (1, 1), pad, (1, 1))
        OH, OW = want.shape[1], want.shape[2]
        src_p = np.full((B_, H, W, sp), 99, dtype=np.int8)
        src_p[..., :C] = src
        w_p = np.full((OFM, KH, KW, wp), 77, dtype=np.int8)
        w_p[..., :C] = w
        dst_p = np.full((B_, OH, OW, dp), 55, dtype=np.int8)
        rq = capi.requant(0, 0, -5, -128, 127, True)
        d = capi.conv_desc(B_, H, W, C, OFM, KH, KW, (1, 1), pad, (1, 1), capi.S8, capi.S8, capi.S8, -4, 0, 4, rq, 0,
                           capi.NHWC, (sp, wp, dp))
        cv = capi.Conv(d)
        announce("conv padded", (B_, H, W, C, OFM, KH, KW), (sp, wp, dp), "device", device)
        m, sh = np.ascontiguousarray(mult, dtype=np.int32), np.ascontiguousarray(shift, dtype=np.int32)
        if device:
            sd, wd, od = to_dev(src_p), to_dev(w_p), to_dev(dst_p)
            keep = [to_dev(bias), to_dev(m), to_dev(sh)]
            cv.prepare(wd, *keep)
            cv.run(sd, od)
            torch.cuda.synchronize()
            got = od.cpu().numpy()
        else:
            cv.prepare(w_p, bias, m, sh)
            got = dst_p.copy()
            cv.run(src_p, got)
        cv.close()
        np.testing.assert_array_equal(got[..., :OFM], want)
        assert (got[..., OFM:] == 55).all(), "padding bytes of the destination were overwritten"
    with pytest.raises(capi.Mi355Error, match="stride is smaller"):
        capi.Conv(capi.conv_desc(1, 4, 4, 16, 8, 1, 1, pixel_strides=(8, 0, 0)))


def _padded_view(rng, dense, pads, fill):
    """A buffer of `fill` bytes holding `dense` (4 dimensions, the last one contiguous) with pads[i] extra elements
    after dimension i of each of the last three dimensions' rows / planes / images; returns (buffer, view on the
    valid elements, byte strides of dimensions 1, 2 and 3 in the reference's order: innermost first)."""
    n3, n2, n1, n0 = dense.shape
    big = np.full((n3, n2 + pads[2], n1 + pads[1], n0 + pads[0]), fill, dtype=dense.dtype)
    view = big[:, :n2, :n1, :n0]
    view[...] = dense
    e = dense.dtype.itemsize
    s1 = (n0 + pads[0]) * e
    s2 = s1 * (n1 + pads[1])
    s3 = s2 * (n2 + pads[2])
    return big, view, (s1, s2, s3)


@pytest.mark.parametrize("layout", ["nhwc", "nchw"])
@pytest.mark.parametrize("device", [True, False])
def test_conv_tensors_padded_in_every_dimension(layout, device):
    """Padding after every dimension of src, weights and dst (ITensorInfo::strides_in_bytes()[1..3] all larger than
    dense, arm_compute/core/ITensorInfo.h:81-334), both layouts: same integers, padding of dst untouched. Strides
    given at create for the first case and through mi355_conv_set_strides_nd after create for the second."""
    import torch
    rng = np.random.default_rng(67)
    nchw = layout == "nchw"
    for case, (B_, H, W, C, OFM, KH, KW, pads_s, pads_w, pads_d) in enumerate(
            [(2, 9, 8, 16, 24, 3, 3, (5, 2, 1), (9, 1, 2), (3, 1, 2)),
             (3, 7, 6, 5, 10, 2, 3, (0, 3, 0), (0, 0, 4), (0, 2, 1))]):
        src = rng.integers(-128, 128, size=(B_, H, W, C), dtype=np.int8)
        w = rng.integers(-127, 128, size=(OFM, KH, KW, C), dtype=np.int8)
        bias = rng.integers(-500, 500, size=OFM, dtype=np.int32)
        mult, shift = oracle.calculate_quantized_multipliers(0.02, rng.uniform(0.01, 1, OFM), 1.1)
        pad = (1, 1, 1, 1) if KH == 3 else (0, 1, 1, 0)
        want = oracle.conv_nhwc_direct(src, w, bias, 4, 0, mult, shift, -5, -128, 127, (1, 1), pad, (1, 1))
        to_layout = (lambda a: np.ascontiguousarray(a.transpose(0, 3, 1, 2))) if nchw else (lambda a: a)
        src_b, _, ss = _padded_view(rng, to_layout(src), pads_s, 99)
        w_b, _, ws = _padded_view(rng, to_layout(w), pads_w, 77)
        dst_b, dst_v, ds = _padded_view(rng, np.zeros_like(to_layout(want)), pads_d, 55)
        dst_v[...] = 11
        rq = capi.requant(0, 0, -5, -128, 127, True)
        lay = capi.NCHW if nchw else capi.NHWC
        if case == 0:
            d = capi.conv_desc(B_, H, W, C, OFM, KH, KW, (1, 1), pad, (1, 1), capi.S8, capi.S8, capi.S8, -4, 0, 4, rq, 0,
                               lay, (ss[0], ws[0], ds[0]), outer_strides=(ss[1:], ws[1:], ds[1:]))
            cv = capi.Conv(d)
        else:
            cv = capi.Conv(capi.conv_desc(B_, H, W, C, OFM, KH, KW, (1, 1), pad, (1, 1), capi.S8, capi.S8, capi.S8, -4,
                                          0, 4, rq, 0, lay))
            cv.set_strides_nd(ss, ws, ds)
        announce("conv padded in every dimension", layout, (B_, H, W, C, OFM, KH, KW), ss, ws, ds, "device", device)
        m, sh = np.ascontiguousarray(mult, dtype=np.int32), np.ascontiguousarray(shift, dtype=np.int32)
        if device:
            sd, wd, od = to_dev(src_b), to_dev(w_b), to_dev(dst_b)
            keep = [to_dev(bias), to_dev(m), to_dev(sh)]
            cv.prepare(wd, *keep)
            cv.run(sd, od)
            torch.cuda.synchronize()
            got = od.cpu().numpy()
        else:
            cv.prepare(w_b, bias, m, sh)
            got = dst_b.copy()
            cv.run(src_b, got)
        cv.close()
        n3, n2, n1, n0 = to_layout(want).shape
        np.testing.assert_array_equal(got[:, :n2, :n1, :n0], to_layout(want))
        mask = np.ones(got.shape, dtype=bool)
        mask[:, :n2, :n1, :n0] = False
        assert (got[mask] == 55).all(), "padding bytes of the destination were overwritten"


def test_conv_f32_destination_padded():
    """The dequantising convolution into an NHWC float tensor with padding after pixels and rows"""
    import torch
    rng = np.random.default_rng(68)
    B_, H, W, C, OFM = 2, 6, 7, 16, 12
    src = rng.integers(-128, 128, size=(B_, H, W, C), dtype=np.int8)
    w = rng.integers(-127, 128, size=(OFM, 3, 3, C), dtype=np.int8)
    dense = capi.Conv(capi.conv_desc(B_, H, W, C, OFM, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), capi.S8, capi.S8, capi.F32, -3,
                                     0, 3, None, 0, capi.NHWC, scale=0.0123))
    dense.prepare(to_dev(w))
    want_d = torch.zeros((B_, H, W, OFM), dtype=torch.float32, device="cuda")
    dense.run(to_dev(src), want_d)
    torch.cuda.synchronize()
    want = want_d.cpu().numpy()
    dense.close()
    dst_b, _, ds = _padded_view(rng, np.zeros_like(want), (3, 2, 0), 7.5)
    announce("conv F32 padded destination", ds)
    cv = capi.Conv(capi.conv_desc(B_, H, W, C, OFM, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), capi.S8, capi.S8, capi.F32, -3, 0,
                                  3, None, 0, capi.NHWC, (0, 0, ds[0]), scale=0.0123, outer_strides=((0, 0), (0, 0), ds[1:])))
    od = to_dev(dst_b)
    cv.prepare(to_dev(w))
    cv.run(to_dev(src), od)
    torch.cuda.synchronize()
    got = od.cpu().numpy()
    cv.close()
    np.testing.assert_array_equal(got[:, :H, :W, :OFM].view(np.uint32), want.view(np.uint32))
    mask = np.ones(got.shape, dtype=bool)
    mask[:, :H, :W, :OFM] = False
    assert (got[mask] == 7.5).all(), "padding of the destination was overwritten"


def test_conv_band_form_random_geometry_sweep():
    """10 seeded geometries on images large enough for the band form: kernel sizes, strides, asymmetric padding,
    dilation, 64 / 128 channels, 1 to 64 output channels, both source signs, weights with and without an offset"""
    rng = np.random.default_rng(1777)
    done, bands = 0, 0
    while done < 10:
        C = int(rng.choice([64, 64, 128]))
        KH, KW = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        if KH * KW * C > 1152:
            continue
        stride = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        dil = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        pad = tuple(int(x) for x in rng.integers(0, 3, size=4))
        B_ = int(rng.integers(1, 4))
        # about 36000 output pixels
        OW = int(rng.integers(40, 180))
        OH = max(8, 36000 // (B_ * OW) + int(rng.integers(0, 9)))
        W = (OW - 1) * stride[0] + dil[0] * (KW - 1) + 1 - pad[0] - pad[2]
        H = (OH - 1) * stride[1] + dil[1] * (KH - 1) + 1 - pad[1] - pad[3] + int(rng.integers(0, stride[1]))
        if B_ * OH * OW <= 4 * 256 * 32 or W < 1 or H < 1:
            continue
        OFM = int(rng.choice([1, 7, 24, 40, 64, 64]))
        dt = np.int8 if rng.integers(2) else np.uint8
        w_dt = np.int8 if (dt == np.int8 or rng.integers(2)) else np.uint8
        src = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max + 1, size=(B_, H, W, C)).astype(dt)
        w = rng.integers(np.iinfo(w_dt).min + (1 if w_dt == np.int8 else 0), np.iinfo(w_dt).max + 1, size=(OFM, KH, KW, C)).astype(w_dt)
        bias = rng.integers(-800, 800, size=OFM, dtype=np.int32)
        in_zp = int(rng.integers(-10, 10)) if dt == np.int8 else int(rng.integers(100, 150))
        w_zp = 0 if w_dt == np.int8 else int(rng.integers(100, 150))
        K = KH * KW * C
        reals = rng.uniform(0.5, 2.0, OFM) * 40.0 / (K ** 0.5 * 74.0 * 74.0)
        mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
        lo, hi, ozp = (-128, 127, -5) if dt == np.int8 else (0, 255, 9)
        want = oracle.conv_nhwc_direct(src, w, bias, in_zp, w_zp, mult, shift, ozp, lo, hi, stride, pad, dil)
        announce("conv band sweep", done, src.shape, w.shape, stride, pad, dil, dt.__name__, w_dt.__name__, in_zp, w_zp)
        got, name = run_conv(src, w, bias, in_zp, w_zp, mult, shift, ozp, lo, hi, stride, pad, dil)
        np.testing.assert_array_equal(got, want)
        bands += name == "implicit_band_32x64"
        done += 1
    assert bands >= 6, bands  # (an output row of more than 512 pixels or a window beyond LDS takes the other form)


def test_conv_random_geometry_sweep():
    """40 seeded geometries: kernel sizes, strides, asymmetric padding, dilation, channel counts on and off the implicit
    loader's 16-byte granularity, both layouts, both signs, per-tensor and per-channel weights"""
    rng = np.random.default_rng(777)
    done = 0
    while done < 40:
        B_ = int(rng.integers(1, 4))
        H, W = int(rng.integers(3, 15)), int(rng.integers(3, 15))
        C = int(rng.choice([3, 8, 16, 16, 32, 48, 64, 20]))
        OFM = int(rng.choice([1, 7, 16, 24, 64, 65]))
        KH, KW = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        stride = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        dil = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        pad = tuple(int(x) for x in rng.integers(0, 3, size=4))
        if H + pad[1] + pad[3] < dil[1] * (KH - 1) + 1 or W + pad[0] + pad[2] < dil[0] * (KW - 1) + 1:
            continue
        dt = np.int8 if rng.integers(2) else np.uint8
        per_channel = bool(rng.integers(2))
        w_dt = np.int8 if (per_channel or dt == np.int8) else np.uint8
        src = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max + 1, size=(B_, H, W, C)).astype(dt)
        w = rng.integers(np.iinfo(w_dt).min + (1 if w_dt == np.int8 else 0), np.iinfo(w_dt).max + 1,
                         size=(OFM, KH, KW, C)).astype(w_dt)
        bias = rng.integers(-800, 800, size=OFM, dtype=np.int32)
        in_zp = int(rng.integers(-10, 10)) if dt == np.int8 else int(rng.integers(100, 150))
        w_zp = 0 if (per_channel or w_dt == np.int8) else int(rng.integers(100, 150))
        out_zp = -5 if dt == np.int8 else 9
        reals = rng.uniform(0.2, 2.0, size=OFM if per_channel else 1) * 60.0 / (74.0 * 74.0 * np.sqrt(KH * KW * C))
        mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
        lo, hi = (-128, 127) if dt == np.int8 else (0, 255)
        want = oracle.conv_nhwc_direct(src, w, bias, in_zp, w_zp, mult, shift, out_zp, lo, hi, stride, pad, dil)
        layout = capi.NCHW if rng.integers(3) == 0 else capi.NHWC
        path = int(rng.integers(2))
        device = bool(rng.integers(2))
        announce("conv sweep", done, src.shape, w.shape, stride, pad, dil, dt.__name__, "pc", per_channel, "layout", layout,
                 "path", path, "dev", device)
        got, name = run_conv(src, w, bias, in_zp, w_zp, mult, shift, out_zp, lo, hi, stride, pad, dil, path=path, device=device,
                             layout=layout)
        # the patch matrix only exists on request: channel counts off the 16-byte granularity and weights with an offset
        # (row sums of the patches) run on the on-the-fly loaders too
        assert name.startswith("implicit_" if path == 0 else "im2col+"), name
        np.testing.assert_array_equal(got, want, err_msg="case %d" % done)
        done += 1


@pytest.mark.parametrize("device", [True, False])
def test_conv_with_f32_destination(device):
    """QASYMM8_SIGNED input and weights, F32 destination (src/cpu/operators/CpuGemmConv2d.cpp:297-305 of the reference):
    the same on-the-fly lowering as the 8-bit destination with the dequantising epilogue (few output channels: the
    LDS-resident-weights kernel; 5 input channels under a weights offset: the byte-wise loader and row sums of the patches;
    3 input channels under symmetric weights: channels padded to 16);
    checked against the oracle's im2col + F32 GEMM, identical bits"""
    import torch
    rng = np.random.default_rng(91)
    for (B_, H, W, C, OFM, KH, KW, stride, pad, in_zp, w_zp, act, twice) in [
            (2, 9, 8, 16, 24, 3, 3, (1, 1), (1, 1, 1, 1), 4, 0, (-np.inf, np.inf), False),
            (1, 7, 6, 5, 9, 3, 2, (2, 1), (0, 1, 1, 0), -3, 6, (0.0, np.inf), True),
            (3, 5, 5, 32, 64, 1, 1, (1, 1), (0, 0, 0, 0), 0, 0, (0.0, 6.0), True),
            (2, 8, 7, 3, 12, 3, 3, (1, 1), (1, 1, 1, 1), 5, 0, (-np.inf, np.inf), False)]:
        src = rng.integers(-128, 128, size=(B_, H, W, C), dtype=np.int8)
        w = rng.integers(-127, 128, size=(OFM, KH, KW, C), dtype=np.int8)
        bias = rng.normal(0.0, 2.0, size=OFM).astype(np.float32)
        scale = float(np.float32(0.02) * np.float32(0.005))
        cols = oracle.im2col_nhwc(src, KH, KW, stride, pad, (1, 1), in_zp)
        want = oracle.gemmlowp_f32(cols, oracle.weights_reshape(w), bias, -in_zp, -w_zp, scale, act[0], act[1],
                                   act_twice=twice)
        d = capi.conv_desc(B_, H, W, C, OFM, KH, KW, stride, pad, (1, 1), capi.S8, capi.S8, capi.F32, -in_zp, -w_zp, in_zp,
                           scale=scale, act=act, flags=capi.GEMM_ACT_TWICE if twice else 0)
        cv = capi.Conv(d)
        OH, OW = cv.out_dims()
        out = np.zeros((B_, OH, OW, OFM), dtype=np.float32)
        announce("conv f32", (B_, H, W, C, OFM, KH, KW), stride, pad, in_zp, w_zp, act, "device", device, cv.kernel_name)
        if device:
            sd, wd, od, bd = to_dev(src), to_dev(w), to_dev(out), to_dev(bias)
            cv.prepare(wd, bd)
            cv.run(sd, od)
            torch.cuda.synchronize()
            out = od.cpu().numpy()
        else:
            cv.prepare(w, bias)
            cv.run(src, out)
        assert cv.kernel_name.startswith("implicit_"), cv.kernel_name
        cv.close()
        assert np.array_equal(out.reshape(-1, OFM).view(np.uint32), want.view(np.uint32))
