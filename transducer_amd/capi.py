"""ctypes view of ``librnnt_hip.so`` (the C interface in ``include/rnnt_hip.h``) for callers
that hold raw device pointers, e.g. torch tensors' ``data_ptr()``.  Raises if the library is
missing or a call fails; there is no fallback."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "librnnt_hip.so")

_F = ctypes.c_void_p
_I = ctypes.c_int
_Z = ctypes.c_size_t

SIGNATURES = {
    "rnnt_hip_last_error": (ctypes.c_char_p, []),
    "rnnt_hip_abi_version": (_I, []),
    "rnnt_hip_forward": (_I, [_F] * 8 + [_I] * 5 + [_F]),
    "rnnt_hip_backward": (_I, [_F] * 10 + [_I] * 5 + [_F]),
    "rnnt_hip_viterbi": (_I, [_F] * 6 + [_I] * 5 + [_F]),
    "rnnt_hip_log_norms": (_I, [_F] * 5 + [_I] * 4 + [_F]),
    "rnnt_hip_dense_grads": (_I, [_F] * 9 + [_I] * 4 + [_F]),
    "rnnt_hip_loss_workspace_bytes": (_Z, [_I] * 4),
    "rnnt_hip_loss_forward": (_I, [_F] * 7 + [_Z] + [_I] * 5 + [_F]),
    "rnnt_hip_loss_backward": (_I, [_F] * 9 + [_Z] + [_I] * 5 + [_F]),
    "rnnt_hip_loss_forward_bf16": (_I, [_F] * 7 + [_Z] + [_I] * 5 + [_F]),
    "rnnt_hip_loss_backward_bf16": (_I, [_F] * 9 + [_Z] + [_I] * 5 + [_F]),
    "rnnt_hip_loss_forward_f16": (_I, [_F] * 7 + [_Z] + [_I] * 5 + [_F]),
    "rnnt_hip_loss_backward_f16": (_I, [_F] * 9 + [_Z] + [_I] * 5 + [_F]),
    "rnnt_hip_viterbi_decode": (_I, [_F] * 5 + [_I] * 5 + [_F]),
    "rnnt_hip_viterbi_decode_static": (_I, [_F] * 5 + [_I] * 5 + [_F]),
    "rnnt_hip_static_scratch_bytes": (_Z, []),
    "rnnt_hip_release_scratch": (_I, []),
    "rnnt_hip_viterbi_decode_bf16": (_I, [_F] * 5 + [_I] * 5 + [_F]),
    "rnnt_hip_viterbi_decode_f16": (_I, [_F] * 5 + [_I] * 5 + [_F]),
    "rnnt_hip_check_kernels": (_I, [_F]),
    "rnnt_hip_set_spin_limit": (_I, [_I]),
    "rnnt_hip_set_maxplus_mode": (_I, [_I]),
    "rnnt_hip_set_fused_grads": (_I, [_I]),
    "rnnt_hip_maxplus_tries_lists": (_I, [_I] * 4),
    "rnnt_hip_maxplus_table": (_I, [_F] * 6 + [_I] * 5 + [_F]),
    "rnnt_hip_chain_floor": (_I, [_I, _I, _F]),
    "rnnt_hip_lse_bound_check": (_I, [ctypes.c_uint, ctypes.c_uint, _F, _F]),
    "rnnt_hip_libm_probe": (_I, [_F, _F, _F, ctypes.c_long, _F]),
    "rnnt_hip_profile_enable": (_I, [_I]),
    "rnnt_hip_profile_stage_count": (_I, []),
    "rnnt_hip_profile_stage_name": (ctypes.c_char_p, [_I]),
    "rnnt_hip_profile_read": (_I, [_F, _F, _I]),
}

_lib = None


class RnntHipError(RuntimeError):
    pass


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RnntHipError(
                "librnnt_hip.so is not built; run `python -m transducer_amd.build`")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def call(name, *args):
    """Calls an int-returning entry point and raises on a non-zero status."""
    lib = load()
    status = getattr(lib, name)(*args)
    if status != 0:
        raise RnntHipError("{} failed ({}): {}".format(
            name, status, lib.rnnt_hip_last_error().decode()))


def profile_enable(on):
    call("rnnt_hip_profile_enable", 1 if on else 0)


def profile_read():
    """-> {stage name: (total milliseconds, launches)} since profiling was enabled / last read."""
    lib = load()
    n = lib.rnnt_hip_profile_stage_count()
    ms = (ctypes.c_double * n)()
    cnt = (ctypes.c_int * n)()
    call("rnnt_hip_profile_read", ctypes.cast(ms, _F), ctypes.cast(cnt, _F), n)
    return {lib.rnnt_hip_profile_stage_name(i).decode(): (ms[i], cnt[i]) for i in range(n)}
