"""ctypes binding of include/mi355_gemmlowp.h for tests and bench.py. Accepts numpy arrays (host pointers) and
torch CUDA tensors (device pointers) interchangeably; no computation happens here."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmi355gemmlowp.so")

U8, S8, S32, F32, S16, F16 = 0, 1, 2, 3, 4, 5
EPI_S32, EPI_FIXEDPOINT, EPI_F32 = 0, 1, 2
PATH_AUTO, PATH_SIMPLE, PATH_MFMA, PATH_SKINNY = 0, 1, 2, 3
PATH_TILE = 16  # + n: the pipelined kernel's n-th tile configuration
CONV_AUTO, CONV_EXPLICIT, CONV_IN_PLACE = 0, 1, 2
GEMM_ACCUMULATE, GEMM_ACT_TWICE = 1, 2
NHWC, NCHW = 0, 1

EXPORTS = [
    "mi355_gemmlowp_create", "mi355_gemmlowp_prepare", "mi355_gemmlowp_update_quant", "mi355_gemmlowp_set_strides", "mi355_gemmlowp_set_strides_3d",
    "mi355_gemmlowp_run", "mi355_gemmlowp_run_noalloc", "mi355_gemmlowp_noalloc_workspace_bytes",
    "mi355_gemmlowp_destroy", "mi355_gemmlowp_kernel_name", "mi355_output_stage_run", "mi355_conv_create",
    "mi355_conv_prepare", "mi355_conv_update_quant", "mi355_conv_set_strides", "mi355_conv_set_strides_nd", "mi355_conv_run", "mi355_conv_out_dims", "mi355_conv_destroy", "mi355_conv_kernel_name",
    "mi355_im2col_nhwc_run", "mi355_last_error", "mi355_device_info",
]


class Requant(C.Structure):
    _fields_ = [("per_channel", C.c_int32), ("multiplier", C.c_int32), ("shift", C.c_int32),
                ("result_offset", C.c_int32), ("min_bound", C.c_int32), ("max_bound", C.c_int32),
                ("stage", C.c_int32)]


class GemmDesc(C.Structure):
    _fields_ = [("M", C.c_int32), ("N", C.c_int32), ("K", C.c_int32), ("batch", C.c_int32),
                ("a_dtype", C.c_int32), ("b_dtype", C.c_int32), ("dst_dtype", C.c_int32), ("epilogue", C.c_int32),
                ("lda", C.c_int64), ("ldb", C.c_int64), ("ldd", C.c_int64),
                ("a_batch_stride", C.c_int64), ("b_batch_stride", C.c_int64), ("d_batch_stride", C.c_int64),
                ("a_offset", C.c_int32), ("b_offset", C.c_int32), ("requant", Requant),
                ("scale", C.c_float), ("act_min", C.c_float), ("act_max", C.c_float),
                ("path", C.c_int32), ("b_transposed", C.c_int32), ("b_k_interleave", C.c_int32),
                ("flags", C.c_int32), ("a_plane_rows", C.c_int32), ("d_plane_rows", C.c_int32),
                ("a_plane_stride", C.c_int64), ("d_plane_stride", C.c_int64)]


class OutputStageDesc(C.Structure):
    _fields_ = [("M", C.c_int32), ("N", C.c_int32), ("ld_src", C.c_int64), ("ld_dst", C.c_int64),
                ("dst_dtype", C.c_int32), ("requant", Requant)]


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("batch", "H", "W", "C", "OFM", "KH", "KW", "stride_x", "stride_y", "pad_left", "pad_top",
                 "pad_right", "pad_bottom", "dilation_x", "dilation_y", "src_dtype", "weights_dtype", "dst_dtype",
                 "src_offset", "weights_offset", "pad_value")] + [("requant", Requant), ("path", C.c_int32),
                                                                  ("layout", C.c_int32),
                                                                  ("src_pixel_stride", C.c_int64),
                                                                  ("weights_pixel_stride", C.c_int64),
                                                                  ("dst_pixel_stride", C.c_int64),
                                                                  ("scale", C.c_float), ("act_min", C.c_float),
                                                                  ("act_max", C.c_float), ("flags", C.c_int32)] + [
                                                                      (n, C.c_int64) for n in
                                                                      ("src_stride2", "src_stride3", "weights_stride2",
                                                                       "weights_stride3", "dst_stride2", "dst_stride3")]


_lib = None


def lib():
    """The loaded shared library. Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: run `python -m computelibrary_amd.build`" % LIB_PATH)
        # A process may hold only one HIP runtime. PyTorch ships its own copy with the same soname as ROCm's, and
        # whichever is loaded first serves both: load torch's first so device tensors and this library share it.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        l = C.CDLL(LIB_PATH)
        vp, i32p, f32p = C.c_void_p, C.c_void_p, C.c_void_p
        l.mi355_gemmlowp_create.argtypes = [C.POINTER(GemmDesc), C.POINTER(vp)]
        l.mi355_gemmlowp_prepare.argtypes = [vp, vp, i32p, i32p, i32p, vp]
        l.mi355_gemmlowp_update_quant.argtypes = [vp, C.c_int32, C.c_int32, C.POINTER(Requant), C.c_float, vp]
        l.mi355_gemmlowp_set_strides.argtypes = [vp] + [C.c_int64] * 6
        l.mi355_gemmlowp_set_strides_3d.argtypes = [vp] + [C.c_int64] * 8
        l.mi355_gemmlowp_run.argtypes = [vp, vp, f32p, vp, vp]
        l.mi355_gemmlowp_run_noalloc.argtypes = [vp, vp, f32p, vp, vp]
        l.mi355_gemmlowp_noalloc_workspace_bytes.argtypes = []
        l.mi355_gemmlowp_noalloc_workspace_bytes.restype = C.c_size_t
        l.mi355_gemmlowp_destroy.argtypes = [vp]
        l.mi355_gemmlowp_destroy.restype = None
        l.mi355_gemmlowp_kernel_name.argtypes = [vp]
        l.mi355_gemmlowp_kernel_name.restype = C.c_char_p
        l.mi355_output_stage_run.argtypes = [C.POINTER(OutputStageDesc), vp, i32p, vp, vp]
        l.mi355_conv_create.argtypes = [C.POINTER(ConvDesc), C.POINTER(vp)]
        l.mi355_conv_prepare.argtypes = [vp, vp, i32p, i32p, i32p, vp]
        l.mi355_conv_run.argtypes = [vp, vp, vp, vp]
        l.mi355_conv_set_strides.argtypes = [vp, C.c_int64, C.c_int64, C.c_int64]
        l.mi355_conv_set_strides_nd.argtypes = [vp, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
        l.mi355_conv_update_quant.argtypes = [vp, C.c_int32, C.c_int32, C.c_int32, C.POINTER(Requant), i32p, i32p, vp]
        l.mi355_conv_out_dims.argtypes = [C.POINTER(ConvDesc), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
        l.mi355_conv_out_dims.restype = None
        l.mi355_conv_destroy.argtypes = [vp]
        l.mi355_conv_destroy.restype = None
        l.mi355_conv_kernel_name.argtypes = [vp]
        l.mi355_conv_kernel_name.restype = C.c_char_p
        l.mi355_im2col_nhwc_run.argtypes = [C.POINTER(ConvDesc), vp, vp, vp]
        l.mi355_last_error.restype = C.c_char_p
        l.mi355_device_info.argtypes = [C.c_char_p, C.c_size_t]
        _lib = l
    return _lib


class Mi355Error(RuntimeError):
    pass


def _check(rc):
    if rc != 0:
        raise Mi355Error(lib().mi355_last_error().decode())


def ptr(x):
    """host pointer of a numpy array / device pointer of a torch tensor / None"""
    if x is None:
        return None
    if isinstance(x, np.ndarray):
        return x.ctypes.data
    return x.data_ptr()


def dtype_code(x):
    name = str(x.dtype).replace("torch.", "")
    return {"uint8": U8, "int8": S8, "int32": S32, "float32": F32, "int16": S16, "float16": F16}[name]


STAGE_FIXEDPOINT, STAGE_SCALE = 0, 1


def requant(mult=0, shift=0, offset=0, lo=-(1 << 31), hi=(1 << 31) - 1, per_channel=False, stage=STAGE_FIXEDPOINT):
    return Requant(1 if per_channel else 0, int(mult), int(shift), int(offset), int(lo), int(hi), int(stage))


def device_info():
    buf = C.create_string_buffer(64)
    cus = lib().mi355_device_info(buf, 64)
    return buf.value.decode(), cus


class Gemm:
    """create -> prepare -> run, for row-major contiguous (or explicitly strided) operands"""

    def __init__(self, M, N, K, a_dtype, b_dtype, dst_dtype, epilogue, a_offset=0, b_offset=0, rq=None, scale=1.0,
                 act_min=-np.inf, act_max=np.inf, batch=1, b_batched=False, lda=None, ldb=None, ldd=None,
                 path=PATH_AUTO, b_transposed=False, b_k_interleave=0, flags=0, a_planes=None, d_planes=None,
                 a_batch_stride=None, d_batch_stride=None):
        """a_planes / d_planes: (rows per plane, plane stride) of matrices whose rows come as planes with gaps between
        them (A: bytes, D: elements); the batch strides then have to be given too."""
        lda, ldb, ldd = lda or K, ldb or (K if b_transposed else N), ldd or N
        b_rows = N if b_transposed else K
        ap, dp = a_planes or (0, 0), d_planes or (0, 0)
        self.desc = GemmDesc(M, N, K, batch, a_dtype, b_dtype, dst_dtype, epilogue, lda, ldb, ldd,
                             a_batch_stride or M * lda, b_rows * ldb if b_batched else 0, d_batch_stride or M * ldd,
                             a_offset, b_offset, rq or requant(), scale, act_min, act_max, path,
                             1 if b_transposed else 0, b_k_interleave, flags, ap[0], dp[0], ap[1], dp[1])
        self._h = C.c_void_p()
        _check(lib().mi355_gemmlowp_create(C.byref(self.desc), C.byref(self._h)))

    @property
    def kernel_name(self):
        return lib().mi355_gemmlowp_kernel_name(self._h).decode()

    def prepare(self, B, bias=None, mult=None, shift=None, stream=None):
        _check(lib().mi355_gemmlowp_prepare(self._h, ptr(B), ptr(bias), ptr(mult), ptr(shift), stream))

    def set_strides_3d(self, lda, ldb, ldd, a_batch_stride, b_batch_stride, d_batch_stride, a_plane_stride, d_plane_stride):
        _check(lib().mi355_gemmlowp_set_strides_3d(self._h, lda, ldb, ldd, a_batch_stride, b_batch_stride, d_batch_stride,
                                                   a_plane_stride, d_plane_stride))
        d = self.desc
        d.lda, d.ldb, d.ldd, d.a_batch_stride, d.b_batch_stride, d.d_batch_stride = lda, ldb, ldd, a_batch_stride, b_batch_stride, d_batch_stride
        d.a_plane_stride, d.d_plane_stride = a_plane_stride, d_plane_stride

    def update_quant(self, a_offset, b_offset, rq, scale=1.0, stream=None):
        _check(lib().mi355_gemmlowp_update_quant(self._h, a_offset, b_offset, C.byref(rq) if rq else None, scale,
                                                 stream))

    def set_strides(self, lda, ldb, ldd, a_batch_stride=None, b_batch_stride=None, d_batch_stride=None):
        d = self.desc
        a_bs = d.M * lda if a_batch_stride is None else a_batch_stride
        d_bs = d.M * ldd if d_batch_stride is None else d_batch_stride
        b_bs = ((d.N if d.b_transposed else d.K) * ldb if d.b_batch_stride else 0) if b_batch_stride is None \
            else b_batch_stride
        _check(lib().mi355_gemmlowp_set_strides(self._h, lda, ldb, ldd, a_bs, b_bs, d_bs))
        d.lda, d.ldb, d.ldd, d.a_batch_stride, d.b_batch_stride, d.d_batch_stride = lda, ldb, ldd, a_bs, b_bs, d_bs
        d.a_plane_stride, d.d_plane_stride = d.a_plane_rows * lda, d.d_plane_rows * ldd  # the library closes the gaps

    def run(self, A, D, bias_f32=None, stream=None):
        _check(lib().mi355_gemmlowp_run(self._h, ptr(A), ptr(bias_f32), ptr(D), stream))

    def run_noalloc(self, A, D, bias_f32=None, stream=None):
        _check(lib().mi355_gemmlowp_run_noalloc(self._h, ptr(A), ptr(bias_f32), ptr(D), stream))

    def close(self):
        if self._h:
            lib().mi355_gemmlowp_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def output_stage(src, bias, dst, rq, stream=None, ld_src=None, ld_dst=None):
    M, N = src.shape[0], src.shape[1]
    d = OutputStageDesc(M, N, ld_src or N, ld_dst or N, dtype_code(dst), rq)
    _check(lib().mi355_output_stage_run(C.byref(d), ptr(src), ptr(bias), ptr(dst), stream))


def conv_desc(batch, H, W, Cc, OFM, KH, KW, stride=(1, 1), pad=(0, 0, 0, 0), dilation=(1, 1), src_dtype=S8,
              weights_dtype=S8, dst_dtype=S8, src_offset=0, weights_offset=0, pad_value=0, rq=None, path=0, layout=0, pixel_strides=(0, 0, 0), scale=1.0,
              act=(-np.inf, np.inf), flags=0, outer_strides=((0, 0), (0, 0), (0, 0))):
    """pixel_strides: strides_in_bytes()[1] of src, weights and dst; outer_strides: their ([2], [3]); 0 = no gap."""
    return ConvDesc(batch, H, W, Cc, OFM, KH, KW, stride[0], stride[1], pad[0], pad[1], pad[2], pad[3], dilation[0],
                    dilation[1], src_dtype, weights_dtype, dst_dtype, src_offset, weights_offset, pad_value,
                    rq or requant(), path, layout, pixel_strides[0], pixel_strides[1], pixel_strides[2], scale,
                    act[0], act[1], flags, outer_strides[0][0], outer_strides[0][1], outer_strides[1][0],
                    outer_strides[1][1], outer_strides[2][0], outer_strides[2][1])


class Conv:
    def __init__(self, desc):
        self.desc = desc
        self._h = C.c_void_p()
        _check(lib().mi355_conv_create(C.byref(self.desc), C.byref(self._h)))

    @property
    def kernel_name(self):
        return lib().mi355_conv_kernel_name(self._h).decode()

    def out_dims(self):
        oh, ow = C.c_int32(0), C.c_int32(0)
        lib().mi355_conv_out_dims(C.byref(self.desc), C.byref(oh), C.byref(ow))
        return oh.value, ow.value

    def prepare(self, weights, bias=None, mult=None, shift=None, stream=None):
        _check(lib().mi355_conv_prepare(self._h, ptr(weights), ptr(bias), ptr(mult), ptr(shift), stream))

    def update_quant(self, src_offset, weights_offset, pad_value, rq, mult=None, shift=None, stream=None):
        _check(lib().mi355_conv_update_quant(self._h, src_offset, weights_offset, pad_value, C.byref(rq), ptr(mult),
                                             ptr(shift), stream))

    def set_strides(self, src_pixel_stride, weights_pixel_stride, dst_pixel_stride):
        _check(lib().mi355_conv_set_strides(self._h, src_pixel_stride, weights_pixel_stride, dst_pixel_stride))

    def set_strides_nd(self, src, weights, dst):
        """Each argument: (strides_in_bytes()[1], [2], [3]) of that tensor, 0 = no gap."""
        a3 = C.c_int64 * 3
        _check(lib().mi355_conv_set_strides_nd(self._h, a3(*src), a3(*weights), a3(*dst)))

    def run(self, src, dst, stream=None):
        _check(lib().mi355_conv_run(self._h, ptr(src), ptr(dst), stream))

    def close(self):
        if self._h:
            lib().mi355_conv_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def im2col_nhwc(desc, src, dst, stream=None):
    _check(lib().mi355_im2col_nhwc_run(C.byref(desc), ptr(src), ptr(dst), stream))
