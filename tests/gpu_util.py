"""Helpers shared by the GPU parity tests: drive the C ABI with host (numpy) or device (torch) buffers."""
import numpy as np

from computelibrary_amd import capi

CODE = {np.dtype(np.uint8): capi.U8, np.dtype(np.int8): capi.S8}


def torch_dev():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    return torch


def to_dev(x):
    torch = torch_dev()
    if x is None:
        return None
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def announce(*what):
    print("[case]", *what, flush=True)


def run_gemm(A, B, epilogue, dst_dtype, a_offset=0, b_offset=0, bias=None, mult=None, shift=None, result_offset=0,
             lo=-(1 << 31), hi=(1 << 31) - 1, scale=1.0, bias_f32=None, act=(-np.inf, np.inf), path=capi.PATH_AUTO,
             device=False, lda=None, ldd=None, stage=0, prev=None, flags=0):
    """A [M][K] or [batch][M][K]; B [K][N] or [batch][K][N]. prev: what the destination holds before the call (for
    GEMM_ACCUMULATE). Returns (numpy result, kernel name)."""
    A3 = A if A.ndim == 3 else A[None]
    batch, M, K = A3.shape
    N = B.shape[-1]
    per_channel = mult is not None and np.ndim(mult) > 0 and len(mult) > 1
    rq = capi.requant(0 if per_channel or mult is None else int(np.atleast_1d(mult)[0]),
                      0 if per_channel or shift is None else int(np.atleast_1d(shift)[0]), result_offset, lo, hi,
                      per_channel, stage)
    dcode = {np.dtype(np.uint8): capi.U8, np.dtype(np.int8): capi.S8, np.dtype(np.int32): capi.S32,
             np.dtype(np.float32): capi.F32, np.dtype(np.float16): capi.F16}[np.dtype(dst_dtype)]
    lda = lda or K
    ldd = ldd or N
    g = capi.Gemm(M, N, K, CODE[A.dtype], CODE[B.dtype], dcode, epilogue, a_offset, b_offset, rq, scale, act[0],
                  act[1], batch=batch, b_batched=(B.ndim == 3), lda=lda, ldd=ldd, path=path, flags=flags)
    Ah = np.zeros((batch, M, lda), dtype=A.dtype)
    Ah[:, :, :K] = A3
    Dh = np.full((batch, M, ldd), 77, dtype=dst_dtype)
    if prev is not None:
        Dh[:, :, :N] = prev if prev.ndim == 3 else prev[None]
    mult_a = None if not per_channel else np.ascontiguousarray(mult, dtype=np.int32)
    shift_a = None if not per_channel else np.ascontiguousarray(shift, dtype=np.int32)
    bias_a = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    bf_a = None if bias_f32 is None else np.ascontiguousarray(bias_f32, dtype=np.float32)
    Bc = np.ascontiguousarray(B)
    if device:
        torch = torch_dev()
        Ad, Bd, Dd = to_dev(Ah), to_dev(Bc), to_dev(Dh)
        keep = [to_dev(bias_a), to_dev(mult_a), to_dev(shift_a), to_dev(bf_a)]
        g.prepare(Bd, keep[0], keep[1], keep[2])
        g.run(Ad, Dd, keep[3])
        torch.cuda.synchronize()
        Dh = Dd.cpu().numpy()
    else:
        g.prepare(Bc, bias_a, mult_a, shift_a)
        g.run(Ah, Dh, bf_a)
    name = g.kernel_name  # (the kernel the run took: a launch may refine what create() announced)
    g.close()
    if ldd != N:
        assert (Dh[:, :, N:] == 77).all(), "padding columns of the destination were overwritten"
    out = Dh[:, :, :N]
    return (out if A.ndim == 3 else out[0]), name
