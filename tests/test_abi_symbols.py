"""The C-ABI library loads without a GPU and exports every function include/mi355_gemmlowp.h declares."""
import ctypes
import os
import re

from computelibrary_amd import capi

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "mi355_gemmlowp.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", text)))


def test_header_functions_are_exported():
    names = declared_functions()
    assert len(names) >= 16
    lib = ctypes.CDLL(capi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(capi.EXPORTS) == names


def test_descriptor_struct_sizes_match_header_layout():
    # 4 + 4 ints, 6 int64, 2 ints, 6-int requant, 3 floats, 2 ints
    assert ctypes.sizeof(capi.Requant) == 24
    assert ctypes.sizeof(capi.GemmDesc) == 32 + 48 + 8 + 24 + 12 + 8 + 4  # + tail padding to 8
    assert ctypes.sizeof(capi.OutputStageDesc) == 8 + 16 + 4 + 24 + 4
    assert ctypes.sizeof(capi.ConvDesc) == 21 * 4 + 24 + 8


def test_create_rejects_bad_descriptors_without_a_gpu():
    rq = capi.requant(1 << 30, 1, 0, 0, 255)
    with __import__("pytest").raises(capi.Mi355Error):
        capi.Gemm(0, 4, 4, capi.U8, capi.U8, capi.S32, capi.EPI_S32)
    with __import__("pytest").raises(capi.Mi355Error):
        capi.Gemm(4, 4, 4, capi.U8, capi.U8, capi.U8, capi.EPI_S32)  # S32 epilogue needs S32 dst
    with __import__("pytest").raises(capi.Mi355Error):
        capi.Gemm(4, 4, 4, capi.U8, capi.U8, capi.U8, capi.EPI_FIXEDPOINT, rq=capi.requant(1, 1, 0, 10, 5))
    with __import__("pytest").raises(capi.Mi355Error):
        capi.Gemm(4, 4, 4, capi.U8, capi.U8, capi.S32, capi.EPI_S32, lda=2)
    with __import__("pytest").raises(capi.Mi355Error):
        capi.Gemm(40, 4, 4, capi.U8, capi.U8, capi.S32, capi.EPI_S32, path=capi.PATH_SKINNY)
    g = capi.Gemm(4, 4, 4, capi.U8, capi.U8, capi.U8, capi.EPI_FIXEDPOINT, rq=rq)
    assert g.kernel_name.startswith("skinny")
    g.close()
