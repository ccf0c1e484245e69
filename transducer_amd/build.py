"""In-tree build of the native libraries (no torch, no cmake):

  transducer_amd/librnnt_hip.so    HIP kernels + extern "C" interface (hipcc, gfx950)
  transducer_amd/libtransducer.so  the reference's C++ interface (transducer.h) on top of it
  transducer_amd/_transducer*.so   pybind11 module with the reference's function names

Run as ``python -m transducer_amd.build``.
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")

HIP_SOURCES = ["rnnt_capi.hip", "rnnt_dp.hip", "rnnt_gemm.hip", "rnnt_grads.hip", "rnnt_lse.hip"]

# -ffp-contract=off: the lattice recursions must round like the reference's scalar code.
# packed-fp32 instructions are disabled for the device pass (the host pass does not know the
# feature and says so; that warning is expected).
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def hip_library_path():
    return os.path.join(HERE, "librnnt_hip.so")


def build_hip(verbose=True):
    objs = []
    for src in HIP_SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        _run(["hipcc"] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
        objs.append(obj)
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", hip_library_path()] + objs)


def build_cxx():
    lib = os.path.join(HERE, "libtransducer.so")
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-I", INCLUDE,
          os.path.join(CSRC, "transducer.cpp"), "-o", lib,
          "-L", HERE, "-lrnnt_hip", "-Wl,-rpath,$ORIGIN"])


def build_pybind():
    import pybind11
    ext = sysconfig.get_config_var("EXT_SUFFIX")
    out = os.path.join(HERE, "_transducer" + ext)
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
          "-I", INCLUDE, "-I", pybind11.get_include(), "-I", sysconfig.get_paths()["include"],
          os.path.join(CSRC, "_transducer.cpp"), "-o", out,
          "-L", HERE, "-ltransducer", "-lrnnt_hip", "-Wl,-rpath,$ORIGIN"])


def build_all():
    build_hip()
    build_cxx()
    build_pybind()


if __name__ == "__main__":
    build_all()
    sys.exit(0)
