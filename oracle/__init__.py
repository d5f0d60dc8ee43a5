"""TEST INFRASTRUCTURE ONLY — numpy-facing wrappers over oracle/liboracle.so (the C restatement of the
reference's quantized-GEMM arithmetic) and, when it has been built, oracle/_ref/libaclref.so (the
reference's own portable test oracle).  Imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py; never by the library.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libaclref.so")

I32P = C.POINTER(C.c_int32)


def build(with_ref=True):
    """Compile liboracle.so (and _ref when the reference checkout is present)."""
    subprocess.check_call(["make", "-s", "-B", "liboracle.so"], cwd=_HERE)
    if with_ref:
        subprocess.check_call(["make", "-s", "ref"], cwd=_HERE)


def _load():
    if not os.path.exists(_LIB_PATH):
        build(with_ref=False)
    lib = C.CDLL(_LIB_PATH)
    lib.orc_f32_to_f16.restype = C.c_uint16
    lib.orc_f32_to_f16.argtypes = [C.c_float]
    lib.orc_f16_to_f32.restype = C.c_float
    lib.orc_f16_to_f32.argtypes = [C.c_uint16]
    lib.orc_sqdmulh.restype = C.c_int32
    lib.orc_sqdmulh.argtypes = [C.c_int32, C.c_int32]
    lib.orc_rounding_shift_right.restype = C.c_int32
    lib.orc_rounding_shift_right.argtypes = [C.c_int32, C.c_int32]
    lib.orc_requant_s32.restype = C.c_int32
    lib.orc_requant_s32.argtypes = [C.c_int32] * 4
    lib.orc_requant_scale_s32.restype = C.c_int32
    lib.orc_requant_scale_s32.argtypes = [C.c_int32] * 4
    lib.orc_sqrdmulh_s32.restype = C.c_int32
    lib.orc_sqrdmulh_s32.argtypes = [C.c_int32, C.c_int32]
    lib.orc_requant_fixedpoint_s16.restype = C.c_int16
    lib.orc_requant_fixedpoint_s16.argtypes = [C.c_int32] * 5
    lib.orc_narrow_clamp.restype = C.c_int32
    lib.orc_narrow_clamp.argtypes = [C.c_int32, C.c_int, C.c_int32, C.c_int32]
    lib.orc_calculate_quantized_multiplier.restype = C.c_int
    lib.orc_calculate_quantized_multiplier.argtypes = [C.c_float, I32P, I32P]
    lib.orc_fast_prepare.restype = C.c_void_p
    lib.orc_fast_prepare.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_int]
    lib.orc_fast_destroy.argtypes = [C.c_void_p]
    lib.orc_fast_threads.restype = C.c_int
    return lib


lib = _load()


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _signed(a):
    assert a.dtype in (np.int8, np.uint8), a.dtype
    return 1 if a.dtype == np.int8 else 0


def _qparams(mult, shift):
    m = np.ascontiguousarray(np.atleast_1d(mult), dtype=np.int32)
    s = np.ascontiguousarray(np.atleast_1d(shift), dtype=np.int32)
    assert m.shape == s.shape
    return m, s, int(m.shape[0])


def sqdmulh(a, b):
    return lib.orc_sqdmulh(int(a), int(b))


def rounding_shift_right(x, e):
    return lib.orc_rounding_shift_right(int(x), int(e))


def requant_s32(v, mult, shift, offset):
    return lib.orc_requant_s32(int(v), int(mult), int(shift), int(offset))


def calculate_quantized_multiplier(real):
    """-> (multiplier, shift); raises ValueError where the reference returns an error Status."""
    m, s = C.c_int32(0), C.c_int32(0)
    if lib.orc_calculate_quantized_multiplier(C.c_float(real), C.byref(m), C.byref(s)) != 0:
        raise ValueError("multiplier %r rejected" % (real,))
    return m.value, s.value


def calculate_quantized_multipliers(in_scale, w_scales, out_scale):
    """Per-channel (mult[], shift[]) as src/core/utils/quantization/AsymmHelpers.cpp:137-145 (float arithmetic)."""
    w = np.atleast_1d(np.asarray(w_scales, dtype=np.float32))
    real = (np.float32(in_scale) * w) / np.float32(out_scale)
    pairs = [calculate_quantized_multiplier(float(r)) for r in real]
    return (np.array([p[0] for p in pairs], dtype=np.int32), np.array([p[1] for p in pairs], dtype=np.int32))


def gemmlowp_s32(A, B, a_offset=0, b_offset=0):
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    out = np.empty((M, N), dtype=np.int32)
    lib.orc_gemmlowp_s32(_p(A), _signed(A), C.c_int64(K), _p(B), _signed(B), C.c_int64(N), _p(out), C.c_int64(N),
                         M, N, K, C.c_int32(a_offset), C.c_int32(b_offset))
    return out


def output_stage_fixedpoint(src, bias, mult, shift, result_offset, min_bound, max_bound, dst_dtype):
    src = np.ascontiguousarray(src, dtype=np.int32)
    M, N = src.shape
    m, s, n = _qparams(mult, shift)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    out = np.empty((M, N), dtype=dst_dtype)
    lib.orc_output_stage_fixedpoint(_p(src), C.c_int64(N), _p(bias), _p(out), C.c_int64(N), _signed(out), M, N,
                                    _p(m), _p(s), n, C.c_int32(result_offset), C.c_int32(min_bound),
                                    C.c_int32(max_bound))
    return out


def gemmlowp_fixedpoint(A, B, bias, a_offset, b_offset, mult, shift, result_offset, min_bound, max_bound, dst_dtype):
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    M, K = A.shape
    _, N = B.shape
    m, s, n = _qparams(mult, shift)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    out = np.empty((M, N), dtype=dst_dtype)
    lib.orc_gemmlowp_fixedpoint(_p(A), _signed(A), C.c_int64(K), _p(B), _signed(B), C.c_int64(N), _p(bias), _p(out),
                                C.c_int64(N), _signed(out), M, N, K, C.c_int32(a_offset), C.c_int32(b_offset),
                                _p(m), _p(s), n, C.c_int32(result_offset), C.c_int32(min_bound),
                                C.c_int32(max_bound))
    return out


def output_stage_scale(src, bias, mult, shift, result_offset, min_bound, max_bound, dst_dtype):
    """QUANTIZE_DOWN with an integer multiplier: ((v + bias + result_offset) * mult) >> shift"""
    src = np.ascontiguousarray(src, dtype=np.int32)
    M, N = src.shape
    m, s, n = _qparams(mult, shift)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    out = np.empty((M, N), dtype=dst_dtype)
    lib.orc_output_stage_scale(_p(src), C.c_int64(N), _p(bias), _p(out), C.c_int64(N), _signed(out), M, N, _p(m), _p(s), n,
                               C.c_int32(result_offset), C.c_int32(min_bound), C.c_int32(max_bound))
    return out


def output_stage_fixedpoint_s16(src, bias, mult, shift, min_bound=-32768, max_bound=32767):
    """int32 -> QSYMM16 (rounding doubling high multiply, rounding shift, no offset)"""
    src = np.ascontiguousarray(src, dtype=np.int32)
    M, N = src.shape
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    out = np.empty((M, N), dtype=np.int16)
    lib.orc_output_stage_fixedpoint_s16(_p(src), C.c_int64(N), _p(bias), _p(out), C.c_int64(N), M, N, C.c_int32(mult),
                                        C.c_int32(shift), C.c_int32(min_bound), C.c_int32(max_bound))
    return out


def gemmlowp_scale(A, B, bias, a_offset, b_offset, mult, shift, result_offset, min_bound, max_bound, dst_dtype):
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    M, K = A.shape
    _, N = B.shape
    m, s, n = _qparams(mult, shift)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    out = np.empty((M, N), dtype=dst_dtype)
    lib.orc_gemmlowp_scale(_p(A), _signed(A), C.c_int64(K), _p(B), _signed(B), C.c_int64(N), _p(bias), _p(out),
                           C.c_int64(N), _signed(out), M, N, K, C.c_int32(a_offset), C.c_int32(b_offset), _p(m), _p(s), n,
                           C.c_int32(result_offset), C.c_int32(min_bound), C.c_int32(max_bound))
    return out


def gemmlowp_f32(A, B, bias, a_offset, b_offset, scale, act_min=-np.inf, act_max=np.inf, prev=None, act_twice=False):
    """prev: previous destination values to accumulate into (GEMMInfo::accumulate), or None"""
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    M, K = A.shape
    _, N = B.shape
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    out = np.empty((M, N), dtype=np.float32) if prev is None else np.array(prev, dtype=np.float32, order="C")
    assert out.shape == (M, N)
    lib.orc_gemmlowp_f32(_p(A), _signed(A), C.c_int64(K), _p(B), _signed(B), C.c_int64(N), _p(bias), _p(out),
                         C.c_int64(N), M, N, K, C.c_int32(a_offset), C.c_int32(b_offset), C.c_float(scale),
                         C.c_float(act_min), C.c_float(act_max), 1 if prev is not None else 0, 1 if act_twice else 0)
    return out


def gemmlowp_f16(A, B, bias, a_offset, b_offset, scale, act_min=-np.inf, act_max=np.inf, prev=None, act_twice=False):
    """F16 destination: the float result (previous half values widened when accumulating) rounded to half once"""
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    M, K = A.shape
    _, N = B.shape
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    out = np.empty((M, N), dtype=np.float16) if prev is None else np.array(prev, dtype=np.float16, order="C")
    assert out.shape == (M, N)
    lib.orc_gemmlowp_f16(_p(A), _signed(A), C.c_int64(K), _p(B), _signed(B), C.c_int64(N), _p(bias), _p(out),
                         C.c_int64(N), M, N, K, C.c_int32(a_offset), C.c_int32(b_offset), C.c_float(scale),
                         C.c_float(act_min), C.c_float(act_max), 1 if prev is not None else 0, 1 if act_twice else 0)
    return out


def f32_to_f16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    return np.array([lib.orc_f32_to_f16(C.c_float(v)) for v in x.ravel()], dtype=np.uint16).reshape(x.shape)


def f16_bits_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    return np.array([lib.orc_f16_to_f32(int(v)) for v in h.ravel()], dtype=np.float32).reshape(h.shape)


def conv_out_dims(H, W, KH, KW, stride=(1, 1), pad=(0, 0, 0, 0), dilation=(1, 1)):
    """stride = (sx, sy); pad = (left, top, right, bottom); dilation = (dx, dy) -> (OH, OW)"""
    oh, ow = C.c_int(0), C.c_int(0)
    lib.orc_conv_out_dims(H, W, KH, KW, stride[0], stride[1], pad[0], pad[1], pad[2], pad[3], dilation[0],
                          dilation[1], C.byref(oh), C.byref(ow))
    return oh.value, ow.value


def im2col_nhwc(src, KH, KW, stride=(1, 1), pad=(0, 0, 0, 0), dilation=(1, 1), pad_value=0):
    src = np.ascontiguousarray(src)
    B_, H, W, Cc = src.shape
    OH, OW = conv_out_dims(H, W, KH, KW, stride, pad, dilation)
    out = np.empty((B_ * OH * OW, KH * KW * Cc), dtype=src.dtype)
    lib.orc_im2col_nhwc(_p(src), _p(out), B_, H, W, Cc, KH, KW, stride[0], stride[1], pad[0], pad[1], pad[2],
                        pad[3], dilation[0], dilation[1], int(pad_value) & 0xFF)
    return out


def weights_reshape(w):
    """[OFM][KH][KW][C] -> B[K][OFM]"""
    w = np.ascontiguousarray(w)
    OFM, KH, KW, Cc = w.shape
    out = np.empty((KH * KW * Cc, OFM), dtype=w.dtype)
    lib.orc_weights_reshape(_p(w), _p(out), OFM, KH, KW, Cc)
    return out


def conv_nhwc_direct(src, w, bias, src_zp, w_zp, mult, shift, result_offset, min_bound, max_bound, stride=(1, 1),
                     pad=(0, 0, 0, 0), dilation=(1, 1)):
    src = np.ascontiguousarray(src)
    w = np.ascontiguousarray(w)
    B_, H, W, Cc = src.shape
    OFM, KH, KW, C2 = w.shape
    assert Cc == C2
    OH, OW = conv_out_dims(H, W, KH, KW, stride, pad, dilation)
    m, s, n = _qparams(mult, shift)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    out = np.empty((B_, OH, OW, OFM), dtype=src.dtype)
    lib.orc_conv_nhwc_direct(_p(src), _signed(src), _p(w), _signed(w), _p(bias), _p(out), _signed(out), B_, H, W,
                             Cc, OFM, KH, KW, stride[0], stride[1], pad[0], pad[1], pad[2], pad[3], dilation[0],
                             dilation[1], C.c_int32(src_zp), C.c_int32(w_zp), _p(m), _p(s), n,
                             C.c_int32(result_offset), C.c_int32(min_bound), C.c_int32(max_bound))
    return out


def conv_nhwc_gemm(src, w, bias, src_zp, w_zp, mult, shift, result_offset, min_bound, max_bound, stride=(1, 1),
                   pad=(0, 0, 0, 0), dilation=(1, 1)):
    """The reference's lowering: im2col (pad with zero point) + weight flatten + gemmlowp with negated offsets
    (src/cpu/operators/CpuGemmConv2d.cpp:243-332)."""
    src = np.ascontiguousarray(src)
    B_, H, W, Cc = src.shape
    OFM, KH, KW, _ = w.shape
    OH, OW = conv_out_dims(H, W, KH, KW, stride, pad, dilation)
    cols = im2col_nhwc(src, KH, KW, stride, pad, dilation, pad_value=src_zp)
    bm = weights_reshape(w)
    out = gemmlowp_fixedpoint(cols, bm, bias, -src_zp, -w_zp, mult, shift, result_offset, min_bound, max_bound,
                              src.dtype)
    return out.reshape(B_, OH, OW, OFM)


class FastGemm:
    """Timed CPU baseline: B packed once, fused offset + fixed-point epilogue, OpenMP + SIMD."""

    def __init__(self, B):
        B = np.ascontiguousarray(B)
        self.K, self.N = B.shape
        self._h = lib.orc_fast_prepare(_p(B), _signed(B), C.c_int64(self.N), self.N, self.K)
        self.level = None

    def run(self, A, bias, a_offset, b_offset, mult, shift, result_offset, min_bound, max_bound, dst_dtype):
        A = np.ascontiguousarray(A)
        M, K = A.shape
        assert K == self.K
        m, s, n = _qparams(mult, shift)
        bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
        out = np.empty((M, self.N), dtype=dst_dtype)
        self.level = lib.orc_fast_gemmlowp_fixedpoint(
            C.c_void_p(self._h), _p(A), _signed(A), C.c_int64(K), _p(bias), _p(out), C.c_int64(self.N), _signed(out),
            M, C.c_int32(a_offset), C.c_int32(b_offset), _p(m), _p(s), n, C.c_int32(result_offset),
            C.c_int32(min_bound), C.c_int32(max_bound))
        return out

    def close(self):
        if self._h:
            lib.orc_fast_destroy(C.c_void_p(self._h))
            self._h = None

    def __del__(self):
        self.close()


def fast_threads():
    return lib.orc_fast_threads()


# ---------------------------------------------------------------------------------------------------------------
# The reference's own oracle (only where oracle/_ref has been built; it cannot be built without /root/reference)
# ---------------------------------------------------------------------------------------------------------------
def ref_available():
    return os.path.exists(_REF_PATH)


_ref = None


def ref():
    global _ref
    if _ref is None:
        r = C.CDLL(_REF_PATH)
        r.ref_asymm_int_mult.restype = C.c_int32
        r.ref_asymm_int_mult.argtypes = [C.c_int32, C.c_int32]
        r.ref_asymm_rounding_divide_by_pow2.restype = C.c_int32
        r.ref_asymm_rounding_divide_by_pow2.argtypes = [C.c_int32, C.c_int]
        r.ref_quantize_down_scalar.restype = C.c_int32
        r.ref_quantize_down_scalar.argtypes = [C.c_int32] * 6
        r.ref_calculate_quantized_multiplier.restype = C.c_int
        r.ref_calculate_quantized_multiplier.argtypes = [C.c_float, I32P, I32P]
        _ref = r
    return _ref


def ref_calculate_quantized_multiplier(real):
    m, s = C.c_int32(0), C.c_int32(0)
    if ref().ref_calculate_quantized_multiplier(C.c_float(real), C.byref(m), C.byref(s)) != 0:
        raise ValueError("multiplier %r rejected" % (real,))
    return m.value, s.value


def ref_gemmlowp_core(A, B, a_offset, b_offset):
    """A [batch?][M][K], B [K][N] or [batch][K][N]; both uint8 or both int8."""
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    assert A.dtype == B.dtype
    A3 = A if A.ndim == 3 else A[None]
    batch, M, K = A3.shape
    N = B.shape[-1]
    out = np.empty((batch, M, N), dtype=np.int32)
    ref().ref_gemmlowp_core(_p(A3), _p(B), _signed(A), M, N, K, batch, 1 if B.ndim == 3 else 0,
                            C.c_int32(a_offset), C.c_int32(b_offset), _p(out))
    return out if A.ndim == 3 else out[0]


def ref_gemmlowp_u8s8(A, B):
    A = np.ascontiguousarray(A, dtype=np.uint8)
    B = np.ascontiguousarray(B, dtype=np.int8)
    M, K = A.shape
    N = B.shape[1]
    out = np.empty((M, N), dtype=np.int32)
    ref().ref_gemmlowp_u8s8(_p(A), _p(B), M, N, K, _p(out))
    return out


def ref_quantize_down_fixedpoint(src, bias, mult, shift, result_offset, lo, hi, dst_dtype):
    src = np.ascontiguousarray(src, dtype=np.int32)
    M, N = src.shape
    m, s, n = _qparams(mult, shift)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    out = np.empty((M, N), dtype=dst_dtype)
    ref().ref_quantize_down_fixedpoint(_p(src), _p(bias), M, N, _p(m), _p(s), n, C.c_int32(result_offset),
                                       C.c_int32(lo), C.c_int32(hi), _signed(out), _p(out))
    return out


def ref_quantize_down_scale(src, bias, mult, shift, result_offset, lo, hi, dst_dtype):
    src = np.ascontiguousarray(src, dtype=np.int32)
    M, N = src.shape
    m, s, n = _qparams(mult, shift)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    out = np.empty((M, N), dtype=dst_dtype)
    ref().ref_quantize_down_scale(_p(src), _p(bias), M, N, _p(m), _p(s), n, C.c_int32(result_offset), C.c_int32(lo),
                                  C.c_int32(hi), _signed(out), _p(out))
    return out


def ref_quantize_down_fixedpoint_s16(src, bias, mult, shift, lo, hi):
    src = np.ascontiguousarray(src, dtype=np.int32)
    M, N = src.shape
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    out = np.empty((M, N), dtype=np.int16)
    ref().ref_quantize_down_fixedpoint_s16(_p(src), _p(bias), M, N, C.c_int32(mult), C.c_int32(shift), C.c_int32(lo),
                                           C.c_int32(hi), _p(out))
    return out


def ref_dequantize_s32(src, scale):
    src = np.ascontiguousarray(src, dtype=np.int32)
    out = np.empty(src.shape, dtype=np.float32)
    ref().ref_dequantize_s32(_p(src), int(src.size), C.c_float(scale), _p(out))
    return out


def ref_dequantize_s32_f16(src, scale, prev=None):
    src = np.ascontiguousarray(src, dtype=np.int32)
    out = np.empty(src.shape, dtype=np.float16)
    prev = None if prev is None else np.ascontiguousarray(prev, dtype=np.float16)
    ref().ref_dequantize_s32_f16(_p(src), int(src.size), C.c_float(scale), _p(prev), _p(out))
    return out


def ref_im2col_nhwc(src, KH, KW, stride, pad, zero_point):
    src = np.ascontiguousarray(src)
    B_, H, W, Cc = src.shape
    OH, OW = conv_out_dims(H, W, KH, KW, stride, pad)
    out = np.empty((B_ * OH * OW, KH * KW * Cc), dtype=np.uint8)
    ref().ref_im2col_nhwc(_p(src.view(np.uint8)), _p(out), B_, H, W, Cc, KH, KW, stride[0], stride[1], pad[0],
                          pad[1], pad[2], pad[3], OH, OW, int(zero_point))
    return out.view(src.dtype)


def ref_conv_nhwc_quantized(src, w, bias, in_scale, in_zp, w_scales, w_zp, out_scale, out_zp, stride=(1, 1),
                            pad=(0, 0, 0, 0), dilation=(1, 1), per_channel=False):
    """NHWC in / out at this boundary; permuted to the NCHW the reference's conv oracle works in."""
    src = np.ascontiguousarray(src)
    w = np.ascontiguousarray(w)
    B_, H, W, Cc = src.shape
    OFM, KH, KW, _ = w.shape
    OH, OW = conv_out_dims(H, W, KH, KW, stride, pad, dilation)
    s_nchw = np.ascontiguousarray(src.transpose(0, 3, 1, 2))
    w_nchw = np.ascontiguousarray(w.transpose(0, 3, 1, 2))
    ws = np.ascontiguousarray(np.atleast_1d(w_scales), dtype=np.float32)
    bias = np.ascontiguousarray(bias, dtype=np.int32)
    out = np.empty((B_, OFM, OH, OW), dtype=src.dtype)
    ref().ref_conv_nchw_quantized(_p(s_nchw), _p(w_nchw), _p(bias), _p(out), _signed(src), 1 if per_channel else 0,
                                  B_, Cc, H, W, OFM, KH, KW, OH, OW, stride[0], stride[1], pad[0], pad[1],
                                  dilation[0], dilation[1], C.c_float(in_scale), C.c_int32(in_zp), _p(ws),
                                  int(ws.shape[0]), C.c_int32(w_zp), C.c_float(out_scale), C.c_int32(out_zp))
    return np.ascontiguousarray(out.transpose(0, 2, 3, 1))
