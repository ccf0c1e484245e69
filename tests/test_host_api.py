"""Host-side checks that need no GPU: the shared libraries load, export what the headers
declare, reject bad arguments before touching the device, and the Python front end keeps the
reference's checks and messages (transducer/torch_binding.py:180-229)."""
import ctypes
import os
import re
import subprocess

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "transducer_amd")


def test_c_interface_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "rnnt_hip.h")).read()
    declared = sorted(set(re.findall(r"\b(rnnt_hip_\w+)\s*\(", header)))
    assert len(declared) >= 14
    lib = ctypes.CDLL(os.path.join(PKG, "librnnt_hip.so"))
    for name in declared:
        assert hasattr(lib, name), name
    from transducer_amd import capi
    assert sorted(capi.SIGNATURES) == declared


def test_cxx_interface_exports_the_three_reference_functions():
    out = subprocess.check_output(["nm", "-DC", os.path.join(PKG, "libtransducer.so")], text=True)
    sig = r"float const\*, float const\*"
    assert re.search(r" T forward\(" + sig, out)
    assert re.search(r" T backward\(" + sig, out)
    assert re.search(r" T viterbi\(" + sig, out)
    # and with exactly the reference's parameter lists (transducer/transducer.h:3-49)
    assert ("forward(float const*, float const*, float*, float*, float const*, int const*, "
            "int const*, int const*, int, int, int, int, int, bool)") in out
    assert ("backward(float const*, float const*, float*, float*, float*, float const*, "
            "float const*, int const*, int const*, int const*, int, int, int, int, int, bool)") in out
    assert ("viterbi(float const*, float const*, float const*, int*, int const*, int const*, "
            "int, int, int, int, int, bool)") in out


def test_bad_sizes_are_rejected_before_any_device_work():
    from transducer_amd import capi
    lib = capi.load()
    assert lib.rnnt_hip_forward(None, None, None, None, None, None, None, None,
                                -1, 1, 1, 1, 0, None) == 1
    assert b"negative size" in lib.rnnt_hip_last_error()
    assert lib.rnnt_hip_log_norms(None, None, None, None, None, 1, 70000, 2, 70000, None) == 1
    assert b"2^31" in lib.rnnt_hip_last_error()
    with pytest.raises(capi.RnntHipError):
        capi.call("rnnt_hip_backward", None, None, None, None, None, None, None, None, None, None,
                  1, 1, -3, 1, 0, None)
    # empty batch: nothing to do, no device needed
    assert lib.rnnt_hip_forward(None, None, None, None, None, None, None, None,
                                0, 5, 3, 4, 0, None) == 0
    # far below one [B,T,V] array (2.56 GB at this shape)
    assert lib.rnnt_hip_loss_workspace_bytes(32, 2000, 101, 10000) < 600 * 2**20


def test_blank_outside_the_vocabulary_is_refused_by_every_entry_point_that_takes_one():
    """The reference indexes rows with `blank` unchecked (transducer_cpu.cpp:46,96); here a blank
    outside [0, V) is an argument error, reported before any pointer is looked at."""
    from transducer_amd import capi
    lib = capi.load()
    n = None
    for blank in (-1, 7, 1 << 20):
        calls = [
            lib.rnnt_hip_forward(n, n, n, n, n, n, n, n, 2, 5, 3, 7, blank, n),
            lib.rnnt_hip_backward(n, n, n, n, n, n, n, n, n, n, 2, 5, 3, 7, blank, n),
            lib.rnnt_hip_viterbi(n, n, n, n, n, n, 2, 5, 3, 7, blank, n),
            lib.rnnt_hip_loss_forward(n, n, n, n, n, n, n, 0, 2, 5, 3, 7, blank, n),
            lib.rnnt_hip_loss_backward(n, n, n, n, n, n, n, n, n, 0, 2, 5, 3, 7, blank, n),
            lib.rnnt_hip_viterbi_decode(n, n, n, n, n, 2, 5, 3, 7, blank, n),
            lib.rnnt_hip_loss_forward_bf16(n, n, n, n, n, n, n, 0, 2, 5, 3, 7, blank, n),
            lib.rnnt_hip_loss_backward_f16(n, n, n, n, n, n, n, n, n, 0, 2, 5, 3, 7, blank, n),
            lib.rnnt_hip_viterbi_decode_bf16(n, n, n, n, n, 2, 5, 3, 7, blank, n),
        ]
        assert calls == [1] * len(calls), (blank, calls)
        assert b"blank index" in lib.rnnt_hip_last_error()
    # the last valid index passes this check (and then fails on the null pointers instead)
    assert lib.rnnt_hip_forward(n, n, n, n, n, n, n, n, 2, 5, 3, 7, 6, n) == 1
    assert b"blank index" not in lib.rnnt_hip_last_error()


def test_front_end_refuses_a_blank_outside_the_vocabulary():
    from transducer_amd import torch_binding
    with pytest.raises(ValueError, match="blank must lie in"):
        torch_binding._check_blank(5, 5)
    with pytest.raises(ValueError, match="blank must lie in"):
        torch_binding._check_blank(-1, 5)
    torch_binding._check_blank(4, 5)


def test_workspace_has_no_BTV_or_BTUV_term():
    """O(B*T*U) lattice planes plus one O(B*U*V) entry (the pieces of exp(P - mP), 6 bytes per
    element of predictions with U rounded up to 32): growing V by dV adds exactly that much, for
    any T.  Small problems (at most 256 workgroups after splitting a tile's frames) add a bounded
    scratch for the partial sums of pgrads: at most 256 x 64 KB."""
    from transducer_amd import capi
    lib = capi.load()
    f = lib.rnnt_hip_loss_workspace_bytes
    y_bytes = lambda v0, v1: 8 * 128 * (v1 - v0) * 6
    per_v_short = f(8, 500, 101, 10016) - f(8, 500, 101, 4096)
    per_v_long = f(8, 2000, 101, 10016) - f(8, 2000, 101, 4096)
    assert per_v_short == per_v_long == y_bytes(4096, 10016)
    for T in (500, 2000):
        extra = f(8, T, 101, 32) - (f(8, T, 101, 4096) - y_bytes(32, 4096))
        assert 0 < extra <= 256 * 64 * 1024 + 4096

def test_pybind_module_has_the_reference_keyword_names():
    from transducer_amd import _transducer
    doc = _transducer.forward.__doc__
    for kw in ("emissions", "predictions", "costs", "alphas", "logNorms", "labels",
               "input_lengths", "label_lengths", "batch_size", "max_input_length",
               "max_label_length", "alphabet_size", "blank", "use_cuda"):
        assert kw + ":" in doc
    assert "log_norms:" in _transducer.viterbi.__doc__  # the reference spells it differently here
    assert "lngrads:" in _transducer.backward.__doc__
    assert isinstance(_transducer.__version__, str)


def test_host_pointers_raise_like_a_backend_that_was_not_built():
    from transducer_amd import _transducer
    with pytest.raises(ValueError, match="not built with the CPU backend"):
        _transducer.forward(0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 2, 0, False)
    with pytest.raises(ValueError, match="not built with the CPU backend"):
        _transducer.backward(0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 2, 0, False)
    with pytest.raises(ValueError, match="not built with the CPU backend"):
        _transducer.viterbi(0, 0, 0, 0, 0, 0, 1, 1, 1, 2, 0, False)


def _inputs(B=2, T=5, U=3, V=4):
    E = torch.rand(B, T, V)
    P = torch.rand(B, U, V)
    labels = torch.randint(1, V, (B, U - 1), dtype=torch.int32)
    il = torch.full((B,), T, dtype=torch.int32)
    ll = torch.full((B,), U - 1, dtype=torch.int32)
    return E, P, labels, il, ll


def test_certify_inputs_messages():
    from transducer_amd.torch_binding import certify_inputs
    E, P, labels, il, ll = _inputs()
    certify_inputs(E, P, labels, il, ll)
    with pytest.raises(TypeError, match="emissions must be torch.float32"):
        certify_inputs(E.double(), P, labels, il, ll)
    with pytest.raises(TypeError, match="labels must be torch.int32"):
        certify_inputs(E, P, labels.long(), il, ll)
    with pytest.raises(TypeError, match="input_lengths must be torch.int32"):
        certify_inputs(E, P, labels, il.long(), ll)
    with pytest.raises(ValueError, match="labels must be contiguous"):
        certify_inputs(E, P, labels.t().contiguous().t(), il, ll)
    with pytest.raises(ValueError, match="vocab size mismatch."):
        certify_inputs(E, P[:, :, :3].contiguous(), labels, il, ll)
    with pytest.raises(ValueError, match="must have a length per example."):
        certify_inputs(E, P, labels, il[:1], ll)
    with pytest.raises(ValueError, match="must have a label length per example."):
        certify_inputs(E, P, labels, il, ll[:1])
    with pytest.raises(ValueError, match="must have a label per example."):
        certify_inputs(E, P, labels[:1], il, ll)
    with pytest.raises(ValueError, match="labels must be padded to maximum label length."):
        certify_inputs(E, P, labels[:, :1].contiguous(), il, ll)
    with pytest.raises(ValueError, match="Input length mismatch"):
        certify_inputs(E, P, labels, il + 1, ll)
    with pytest.raises(ValueError, match="Output length mismatch"):
        certify_inputs(E, P, labels, il, ll + 1)


def test_loss_on_host_tensors_fails_loudly():
    from transducer_amd import TransducerLoss
    E, P, labels, il, ll = _inputs()
    with pytest.raises(ValueError, match="not built with the CPU backend"):
        TransducerLoss()(E, P, labels, il, ll)
    with pytest.raises(ValueError, match="not built with the CPU backend"):
        TransducerLoss().viterbi(E, P, il, ll)
    assert TransducerLoss(blank=3).blank == 3


def test_setup_script_names_the_package_and_builds_through_the_in_tree_build():
    """setup.py stands in for the reference's CMake-driven one (setup.py:23-73): it must name
    the package and route build_ext to transducer_amd/build.py (not run here: the build check
    compiles everything already)."""
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.check_output([sys.executable, "setup.py", "--name", "--version"], cwd=root,
                                  stderr=subprocess.DEVNULL).decode().split()
    assert out[0] == "transducer_amd" and out[1][0].isdigit()
    text = open(os.path.join(root, "setup.py")).read()
    assert "build_all()" in text and "check_call" not in text  # no cmake / network step of its own


def test_a_cxx_caller_of_the_reference_header_compiles_links_and_sees_its_exceptions(tmp_path):
    """A translation unit written against the reference's transducer.h (three free functions,
    C++ linkage, transducer/transducer.h:3-49) builds against include/transducer.h and
    libtransducer.so with a plain g++ line; the backend that is not built reports
    std::invalid_argument as transducer/transducer.cpp:41,97,147 do (no device is touched)."""
    src = tmp_path / "caller.cpp"
    src.write_text(r'''
#include <cstdio>
#include <stdexcept>
#include <string>
#include "transducer.h"
template <typename F> static int refused(F f) {
  try { f(); } catch (const std::invalid_argument& e) {
    return std::string(e.what()).find("not built") != std::string::npos ? 1 : 0;
  }
  return 0;
}
int main() {
  float x[8] = {0}; int n[2] = {1, 0}; int lab[2] = {0, 0};
  int ok = 0;
  ok += refused([&] { forward(x, x, x, x, x, lab, n, n + 1, 1, 1, 1, 2, 0, false); });
  ok += refused([&] { backward(x, x, x, x, x, x, x, lab, n, n + 1, 1, 1, 1, 2, 0, false); });
  ok += refused([&] { viterbi(x, x, x, lab, n, n + 1, 1, 1, 1, 2, 0, false); });
  std::printf("%d\n", ok);
  return ok == 3 ? 0 : 1;
}
''')
    exe = tmp_path / "caller"
    subprocess.check_call(["g++", "-std=c++11", "-I", os.path.join(ROOT, "include"), str(src),
                           "-o", str(exe), "-L", PKG, "-ltransducer", "-lrnnt_hip",
                           "-Wl,-rpath," + PKG])
    assert subprocess.check_output([str(exe)], text=True).strip() == "3"


def test_setup_py_builds_an_importable_package_outside_the_source_tree(tmp_path):
    """The counterpart of the reference's setup.py:23-73 (build_ext through CMake and a pybind11
    fetched from the network): here build_ext drives hipcc and g++ directly.  A non-inplace
    build must leave a package that imports and exports the C interface from its own copy of
    the libraries, without touching the ones in the source tree."""
    lib, tmp = str(tmp_path / "lib"), str(tmp_path / "tmp")
    before = os.path.getmtime(os.path.join(PKG, "librnnt_hip.so"))
    subprocess.check_call(
        ["python", os.path.join(ROOT, "setup.py"), "-q", "build_py", "--build-lib", lib,
         "build_ext", "--build-lib", lib, "--build-temp", tmp], cwd=ROOT,
        stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    assert os.path.getmtime(os.path.join(PKG, "librnnt_hip.so")) == before
    built = os.listdir(os.path.join(lib, "transducer_amd"))
    assert "librnnt_hip.so" in built and "libtransducer.so" in built
    assert any(f.startswith("_transducer") and f.endswith(".so") for f in built)
    code = ("import os, transducer_amd; from transducer_amd import capi, _transducer; "
            "assert os.path.dirname(capi.LIB_PATH) == os.path.dirname(transducer_amd.__file__); "
            "print(capi.load().rnnt_hip_abi_version(), _transducer.__version__, "
            "transducer_amd.__file__)")
    env = dict(os.environ, PYTHONPATH=lib)
    out = subprocess.check_output(["python", "-c", code], cwd=str(tmp_path), env=env, text=True)
    assert out.split()[0] == "1" and lib in out.split()[2]


def test_the_build_module_imports_without_the_built_libraries():
    # `python -m transducer_amd.build` must work in a tree that holds no .so yet (or a stale
    # one): importing the package or its build module loads no native library; asking for
    # TransducerLoss does.
    import subprocess
    import sys
    code = ("import sys, transducer_amd, transducer_amd.build; "
            "assert 'transducer_amd._transducer' not in sys.modules; "
            "assert 'transducer_amd.torch_binding' not in sys.modules; "
            "from transducer_amd import TransducerLoss; "
            "assert 'transducer_amd._transducer' in sys.modules")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    subprocess.check_call([sys.executable, "-c", code], cwd=root)


def test_maxplus_mode_setter_and_query():
    from transducer_amd import capi
    lib = capi.load()
    try:
        capi.call("rnnt_hip_set_maxplus_mode", 1)
        assert lib.rnnt_hip_maxplus_tries_lists(32, 2000, 101, 10000) == 0
        capi.call("rnnt_hip_set_maxplus_mode", 2)
        assert lib.rnnt_hip_maxplus_tries_lists(2, 10, 5, 64) == 1
        assert lib.rnnt_hip_maxplus_tries_lists(2, 10, 5, 17408) == 1
        assert lib.rnnt_hip_maxplus_tries_lists(2, 10, 5, 17409) == 0  # a row longer than a wavefront keeps
        capi.call("rnnt_hip_set_maxplus_mode", 0)
        assert lib.rnnt_hip_maxplus_tries_lists(32, 2000, 101, 10000) == 1
        assert lib.rnnt_hip_maxplus_tries_lists(32, 2000, 101, 2000) == 0
        assert lib.rnnt_hip_maxplus_tries_lists(32, 2000, 101, 3000) == 1
        assert lib.rnnt_hip_maxplus_tries_lists(32, 2000, 51, 10000) == 1
        assert lib.rnnt_hip_maxplus_tries_lists(32, 2000, 17, 10000) == 0   # U x V too small to pay
        assert lib.rnnt_hip_maxplus_tries_lists(32, 2000, 33, 4000) == 0
        assert lib.rnnt_hip_maxplus_tries_lists(32, 2000, 101, 32000) == 0
        with pytest.raises(capi.RnntHipError):
            capi.call("rnnt_hip_set_maxplus_mode", 7)
    finally:
        capi.call("rnnt_hip_set_maxplus_mode", 0)
