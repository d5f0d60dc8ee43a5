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


def test_clamp_bounds_partly_outside_the_output_type_are_rejected():
    """Bounds inside the 8-bit range clamp, bounds that cover it saturate; one end in and one end out is refused, for the
    fused GEMM, the convolution and a later update alike (the reference's own kernels disagree on such bounds)."""
    import pytest
    for dt, bad, good in ((capi.U8, [(-5, 200), (10, 300), (-1, 254)], [(0, 255), (3, 250), (-(1 << 31), (1 << 31) - 1), (-9, 999)]),
                          (capi.S8, [(-129, 0), (0, 128), (-200, 100)], [(-128, 127), (-100, 5), (-128, 200), (-500, 127)])):
        for lo, hi in bad:
            with pytest.raises(capi.Mi355Error, match="partly outside"):
                capi.Gemm(4, 4, 4, dt, dt, dt, capi.EPI_FIXEDPOINT, rq=capi.requant(1 << 30, 1, 0, lo, hi))
            with pytest.raises(capi.Mi355Error, match="partly outside"):
                capi.Conv(capi.conv_desc(1, 4, 4, 16, 8, 3, 3, src_dtype=dt, weights_dtype=dt, dst_dtype=dt,
                                         rq=capi.requant(1 << 30, 1, 0, lo, hi)))
        for lo, hi in good:
            g = capi.Gemm(4, 4, 4, dt, dt, dt, capi.EPI_FIXEDPOINT, rq=capi.requant(1 << 30, 1, 0, lo, hi))
            with pytest.raises(capi.Mi355Error, match="partly outside"):
                g.update_quant(0, 0, capi.requant(1 << 30, 1, 0, bad[0][0], bad[0][1]))
            g.close()


def test_set_strides_checks_what_create_checks():
    import pytest
    g = capi.Gemm(8, 12, 16, capi.S8, capi.S8, capi.S32, capi.EPI_S32, batch=2)
    g.set_strides(20, 12, 16)
    assert (g.desc.lda, g.desc.ldd, g.desc.a_batch_stride, g.desc.d_batch_stride) == (20, 16, 160, 128)
    with pytest.raises(capi.Mi355Error, match="row stride"):
        g.set_strides(15, 12, 16)
    with pytest.raises(capi.Mi355Error, match="batch stride"):
        g.set_strides(20, 12, 16, a_batch_stride=100)
    with pytest.raises(capi.Mi355Error, match="shared"):
        g.set_strides(20, 12, 16, b_batch_stride=16 * 12)
    g.close()
    c = capi.Conv(capi.conv_desc(1, 4, 4, 16, 8, 3, 3))
    c.set_strides(24, 16, 8)
    with pytest.raises(capi.Mi355Error, match="stride is smaller"):
        c.set_strides(8, 16, 8)
    c.close()


def test_strides_of_outer_dimensions_are_checked_without_a_gpu():
    """Strides of dimensions 2 and 3 of convolution tensors and the plane strides of 3D-reinterpreted GEMM matrices: every
    stride has to step over what lies below it, at create and when set later; 0 stands for 'no gap'."""
    import pytest
    # NHWC 1x6x5x16 -> 8 channels, 3x3 pad 1: src rows of 5 pixels x 20 bytes = 100, images of 6 rows
    ok = capi.conv_desc(1, 6, 5, 16, 8, 3, 3, pad=(1, 1, 1, 1), pixel_strides=(20, 0, 0), outer_strides=((120, 900), (0, 0), (0, 0)))
    capi.Conv(ok).close()
    for bad in (((99, 0), (0, 0), (0, 0)),       # src row stride below 5 pixels x 20 bytes
                ((120, 700), (0, 0), (0, 0)),    # src image stride below 6 rows x 120 bytes
                ((0, 0), (40, 0), (0, 0)),       # weights: a row of 3 taps x 16 bytes needs 48
                ((0, 0), (0, 0), (39, 0))):      # dst: a row of 5 pixels x 8 bytes needs 40
        with pytest.raises(capi.Mi355Error, match="stride is smaller"):
            capi.Conv(capi.conv_desc(1, 6, 5, 16, 8, 3, 3, pad=(1, 1, 1, 1), pixel_strides=(20, 0, 0), outer_strides=bad))
    c = capi.Conv(capi.conv_desc(2, 6, 5, 16, 8, 3, 3, pad=(1, 1, 1, 1), layout=capi.NCHW))
    c.set_strides_nd((7, 50, 900), (0, 0, 0), (5, 30, 0))   # NCHW: rows of 5 (+2), planes of 6 rows (+8 bytes), images of 16 planes
    with pytest.raises(capi.Mi355Error, match="stride is smaller"):
        c.set_strides_nd((4, 0, 0), (0, 0, 0), (0, 0, 0))
    with pytest.raises(capi.Mi355Error, match="stride is smaller"):
        c.set_strides_nd((7, 41, 0), (0, 0, 0), (0, 0, 0))
    c.close()
    # GEMM: 12 rows as 3 planes of 4 rows
    g = capi.Gemm(12, 8, 16, capi.S8, capi.S8, capi.S32, capi.EPI_S32, batch=2, lda=20, ldd=8, a_planes=(4, 100), d_planes=(4, 40),
                  a_batch_stride=300, d_batch_stride=120)
    g.set_strides_3d(24, 8, 9, 400, 0, 200, 120, 50)
    assert (g.desc.a_plane_stride, g.desc.d_plane_stride) == (120, 50)
    g.set_strides(20, 8, 8, a_batch_stride=240, d_batch_stride=96)  # planes without a gap again
    assert (g.desc.a_plane_stride, g.desc.d_plane_stride) == (80, 32)
    with pytest.raises(capi.Mi355Error, match="plane stride"):
        g.set_strides_3d(24, 8, 9, 400, 0, 200, 80, 50)     # 3 rows x 24 + 16 bytes do not fit 80
    with pytest.raises(capi.Mi355Error, match="batch stride"):
        g.set_strides_3d(24, 8, 9, 300, 0, 200, 120, 50)    # 2 planes x 120 + 3 x 24 + 16 > 300
    g.close()
    with pytest.raises(capi.Mi355Error, match="plane_rows"):
        capi.Gemm(12, 8, 16, capi.S8, capi.S8, capi.S32, capi.EPI_S32, a_planes=(5, 100), a_batch_stride=400)
