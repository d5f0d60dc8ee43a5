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


def test_descriptor_struct_layouts_match_the_header(tmp_path):
    """sizeof and the offset of every field, as the C compiler lays out include/mi355_gemmlowp.h, against the ctypes
    mirrors in computelibrary_amd/capi.py."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    structs = {"mi355_requant": capi.Requant, "mi355_gemm_desc": capi.GemmDesc,
               "mi355_output_stage_desc": capi.OutputStageDesc, "mi355_conv_desc": capi.ConvDesc}
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "mi355_gemmlowp.h"', 'int main(void) {']
    for cname, ct in structs.items():
        lines.append('printf("%s %%zu\\n", sizeof(%s));' % (cname, cname))
        for fname, _ in ct._fields_:
            lines.append('printf("%s.%s %%zu\\n", offsetof(%s, %s));' % (cname, fname, cname, fname))
    lines += ['return 0; }']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-I", os.path.join(root, "include"), "-o", str(exe), str(src)])
    out = dict(l.split() for l in subprocess.check_output([str(exe)], text=True).splitlines())
    for cname, ct in structs.items():
        assert int(out[cname]) == ctypes.sizeof(ct), cname
        for fname, _ in ct._fields_:
            assert int(out["%s.%s" % (cname, fname)]) == getattr(ct, fname).offset, (cname, fname)


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
        capi.Gemm(80, 4, 4, capi.U8, capi.U8, capi.S32, capi.EPI_S32, path=capi.PATH_SKINNY)
    g = capi.Gemm(4, 4, 4, capi.U8, capi.U8, capi.U8, capi.EPI_FIXEDPOINT, rq=rq)
    assert g.kernel_name.startswith("skinny")
    g.close()
