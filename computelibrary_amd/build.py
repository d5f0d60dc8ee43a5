"""Builds libmi355gemmlowp.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m computelibrary_amd.build            # the product library and the measurement-only kernels
    python -m computelibrary_amd.build --phases   # also the instrumented build for `bench.py --phase-clocks`
The shared library lands in computelibrary_amd/lib/ (git-ignored; it travels with the tree to the GPU box).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")
LIB = os.path.join(LIBDIR, "libmi355gemmlowp.so")
# measurement-only kernels for `bench.py --ceilings`: a library of their own, never linked into the product library
CEILINGS_LIB = os.path.join(LIBDIR, "libmi355ceilings.so")
CEILINGS_SOURCES = ["ceilings.hip"]
# the product library once more with the pipelined kernel compiled to leave clock readings at the ends of its parts
# (`bench.py --phase-clocks`); also a library of its own
PHASES_LIB = os.path.join(LIBDIR, "libmi355phases.so")
SOURCES = ["gemm_dma.hip", "gemm_mfma.hip", "gemm_skinny.hip", "gemm_narrow.hip", "kernels_aux.hip", "capi.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


# per file: the narrow-N convolution kernels' file asks for the first 3 dwords of a kernel's arguments to be preloaded into
# scalar registers when a wave is launched (see conv_halo_kernel)
FILE_FLAGS = {"gemm_narrow.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=3"]}


def _compile(src, extra=(), suffix=""):
    obj = os.path.join(OBJDIR, src.replace(".hip", suffix + ".o"))
    cmd = [HIPCC] + FLAGS + FILE_FLAGS.get(src, []) + list(extra) + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    if out.strip():
        print(out)
    return obj


def _link(lib, members, verbose):
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + members
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    if verbose:
        print("built", lib)


def build(verbose=True):
    """The product library and the measurement-only kernels (a library of their own)."""
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(_compile, SOURCES + CEILINGS_SOURCES))
    _link(LIB, objs[:len(SOURCES)], verbose)
    _link(CEILINGS_LIB, objs[len(SOURCES):], verbose)
    return LIB


def build_phases(verbose=True):
    """The instrumented build `bench.py --phase-clocks` runs on: only made when that is asked for."""
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as ex:
        instrumented = ("gemm_dma.hip", "gemm_narrow.hip")
        phases = [ex.submit(_compile, src, ("-DMI355_PHASE_CLOCKS",), "_phases") for src in instrumented]
        objs = list(ex.map(_compile, [x for x in SOURCES if x not in instrumented]))
        objs += [f.result() for f in phases]
    _link(PHASES_LIB, objs, verbose)
    return PHASES_LIB


if __name__ == "__main__":
    build()
    if "--phases" in sys.argv[1:]:
        build_phases()
    sys.exit(0)
