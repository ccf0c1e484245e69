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

# (source, extra flags, object name).  The gradient kernels are by far the longest compile: the
# file comes in six parts (egrads, pgrads x fp32, bf16, fp16 scores) that are compiled side by side.
HIP_SOURCES = [("rnnt_grads.hip", ["-DRNNT_GRADS_PART=%d" % part], "rnnt_grads_%d.o" % part)
               for part in range(6)] + \
              [(src, [], src.replace(".hip", ".o"))
               for src in ("rnnt_dp.hip", "rnnt_capi.hip", "rnnt_lse.hip", "rnnt_cand.hip",
                           "rnnt_fused.hip", "rnnt_prep.hip")]

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


def hip_library_path(out_dir=HERE):
    return os.path.join(out_dir, "librnnt_hip.so")


def build_hip(out_dir=HERE, obj_dir=CSRC):
    """The translation units are compiled side by side (a handful of hipcc processes), then
    linked."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(obj_dir, exist_ok=True)
    jobs = []
    for src, extra, name in HIP_SOURCES:
        obj = os.path.join(obj_dir, name)
        jobs.append((["hipcc"] + HIPCC_FLAGS + extra + ["-c", os.path.join(CSRC, src), "-o", obj],
                     obj))
    workers = max(1, min(len(jobs), (os.cpu_count() or 2) - 1))
    with ThreadPoolExecutor(workers) as pool:
        list(pool.map(lambda job: _run(job[0]), jobs))
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", hip_library_path(out_dir)] +
         [obj for _, obj in jobs])


def build_cxx(out_dir=HERE):
    lib = os.path.join(out_dir, "libtransducer.so")
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-I", INCLUDE,
          os.path.join(CSRC, "transducer.cpp"), "-o", lib,
          "-L", out_dir, "-lrnnt_hip", "-Wl,-rpath,$ORIGIN"])


def build_pybind(out_dir=HERE):
    import pybind11
    ext = sysconfig.get_config_var("EXT_SUFFIX")
    out = os.path.join(out_dir, "_transducer" + ext)
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
          "-I", INCLUDE, "-I", pybind11.get_include(), "-I", sysconfig.get_paths()["include"],
          os.path.join(CSRC, "_transducer.cpp"), "-o", out,
          "-L", out_dir, "-ltransducer", "-lrnnt_hip", "-Wl,-rpath,$ORIGIN"])


def build_all(out_dir=HERE, obj_dir=CSRC):
    """out_dir: where the three libraries go (default: next to the sources, where the package
    loads them from); obj_dir: where the object files go."""
    os.makedirs(out_dir, exist_ok=True)
    build_hip(out_dir, obj_dir)
    build_cxx(out_dir)
    build_pybind(out_dir)


if __name__ == "__main__":
    build_all()
    sys.exit(0)
