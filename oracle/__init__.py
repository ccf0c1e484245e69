"""TEST INFRASTRUCTURE: numpy front end of the CPU oracle (``librnnt_oracle.so``) and, where it
was built, of the reference's own CPU sources (``_ref/libtransducer_ref.so``).

Only ``tests/``, the smoke check and the CPU-baseline leg of the benchmark import this module;
the product package never does.  Array conventions follow the reference
(``transducer/transducer.h:3-49``): ``E[B,T,V]``, ``P[B,U,V]`` with ``U`` = longest label + 1,
``labels[B,U-1]``, ``LN/alphas/lngrads[B,T,U]``, all C-contiguous.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librnnt_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libtransducer_ref.so")

_lib = None
_ref = None


def build(reference=True):
    """Compile the oracle (and the reference sources when their tree is present)."""
    subprocess.check_call(["make", "-C", _HERE, "librnnt_oracle.so"] + (["ref"] if reference else []))


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build(reference=False)
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def have_ref():
    return os.path.exists(_REF_PATH)


def ref():
    global _ref
    if _ref is None:
        _ref = ctypes.CDLL(_REF_PATH)
    return _ref


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _np(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


def _real(precision):
    return (np.float32, "_f32") if precision == "f32" else (np.float64, "_f64")


def _dims(E, P):
    B, T, V = E.shape
    U = P.shape[1]
    return B, T, U, V


def _full_lengths(E, P, input_lengths, label_lengths):
    B, T, U, _ = _dims(E, P)
    il = np.full(B, T, np.int32) if input_lengths is None else _np(input_lengths, np.int32)
    ll = np.full(B, U - 1, np.int32) if label_lengths is None else _np(label_lengths, np.int32)
    return il, ll


# ---------------------------------------------------------------- oracle (restatement)

def log_norms_naive(E, P, input_lengths=None, label_lengths=None, precision="f32"):
    dt, sfx = _real(precision)
    E, P = _np(E, dt), _np(P, dt)
    B, T, U, V = _dims(E, P)
    il, ll = _full_lengths(E, P, input_lengths, label_lengths)
    LN = np.empty((B, T, U), dt)
    getattr(lib(), "orc_log_norms_naive" + sfx)(_p(E), _p(P), _p(LN), _p(il), _p(ll), B, T, U, V)
    return LN


def log_norms_sep(E, P, precision="f32", return_sum=False, lanes=1):
    """Separable-max form (torch_binding.py:35-40).  lanes: partial sums of the inner sum (1 =
    index order; 8 = the order of a vectorised dot product; the reference leaves it to BLAS)."""
    dt, sfx = _real(precision)
    E, P = _np(E, dt), _np(P, dt)
    B, T, U, V = _dims(E, P)
    LN = np.empty((B, T, U), dt)
    S = np.empty((B, T, U), dt) if return_sum else None
    getattr(lib(), "orc_log_norms_sep_lanes" + sfx)(_p(E), _p(P), _p(LN), _p(S), B, T, U, V,
                                                    int(lanes))
    return (LN, S) if return_sum else LN


def log_norms_truth(E, P, input_lengths=None, label_lengths=None):
    """fp64 log-sum-exp of the fp32 inputs."""
    E, P = _np(E, np.float32), _np(P, np.float32)
    B, T, U, V = _dims(E, P)
    il = None if input_lengths is None else _np(input_lengths, np.int32)
    ll = None if label_lengths is None else _np(label_lengths, np.int32)
    LN = np.empty((B, T, U), np.float64)
    lib().orc_log_norms_truth(_p(E), _p(P), _p(LN), _p(il), _p(ll), B, T, U, V)
    return LN


def libm_expf(x):
    """expf of the host's C library, elementwise (what std::exp(float) is in the reference)."""
    x = _np(x, np.float32)
    y = np.empty_like(x)
    lib().orc_libm_expf(_p(x), _p(y), ctypes.c_long(x.size))
    return y


def libm_log1pf(x):
    """log1pf of the host's C library, elementwise."""
    x = _np(x, np.float32)
    y = np.empty_like(x)
    lib().orc_libm_log1pf(_p(x), _p(y), ctypes.c_long(x.size))
    return y


def forward(E, P, LN, labels, input_lengths, label_lengths, blank=0, precision="f32"):
    """-> costs[B], alphas[B,T,U] (cells outside the valid region hold NaN)."""
    dt, sfx = _real(precision)
    E, P, LN = _np(E, dt), _np(P, dt), _np(LN, dt)
    B, T, U, V = _dims(E, P)
    labels = _np(labels, np.int32).reshape(B, max(U - 1, 0))
    il, ll = _np(input_lengths, np.int32), _np(label_lengths, np.int32)
    costs = np.empty(B, dt)
    alphas = np.full((B, T, U), np.nan, dt)
    getattr(lib(), "orc_forward" + sfx)(_p(E), _p(P), _p(costs), _p(alphas), _p(LN), _p(labels),
                                        _p(il), _p(ll), B, T, U, V, blank)
    return costs, alphas


def backward(E, P, alphas, LN, labels, input_lengths, label_lengths, blank=0, precision="f32"):
    """-> sparse egrads[B,T,V], sparse pgrads[B,U,V], lngrads[B,T,U]."""
    dt, sfx = _real(precision)
    E, P, LN, alphas = _np(E, dt), _np(P, dt), _np(LN, dt), _np(alphas, dt)
    B, T, U, V = _dims(E, P)
    labels = _np(labels, np.int32).reshape(B, max(U - 1, 0))
    il, ll = _np(input_lengths, np.int32), _np(label_lengths, np.int32)
    eg, pg, lng = np.empty_like(E), np.empty_like(P), np.empty_like(LN)
    getattr(lib(), "orc_backward" + sfx)(_p(E), _p(P), _p(eg), _p(pg), _p(lng), _p(alphas), _p(LN),
                                         _p(labels), _p(il), _p(ll), B, T, U, V, blank)
    return eg, pg, lng


def viterbi(E, P, LN, input_lengths, label_lengths, blank=0, precision="f32"):
    """-> labels[B,U-1]; entries past label_lengths[b] are -1 (the reference leaves them unset)."""
    dt, sfx = _real(precision)
    E, P, LN = _np(E, dt), _np(P, dt), _np(LN, dt)
    B, T, U, V = _dims(E, P)
    il, ll = _np(input_lengths, np.int32), _np(label_lengths, np.int32)
    out = np.full((B, max(U - 1, 0)), -1, np.int32)
    getattr(lib(), "orc_viterbi" + sfx)(_p(E), _p(P), _p(LN), _p(out), _p(il), _p(ll), B, T, U, V,
                                        blank)
    return out


def accumulate_grads(E, P, egrads, pgrads, lngrads, LN, input_lengths, label_lengths,
                     precision="f32"):
    """Adds the dense softmax part into copies of egrads/pgrads and returns them."""
    dt, sfx = _real(precision)
    E, P, LN, lngrads = _np(E, dt), _np(P, dt), _np(LN, dt), _np(lngrads, dt)
    eg, pg = np.array(egrads, dt, order="C"), np.array(pgrads, dt, order="C")
    B, T, U, V = _dims(E, P)
    il, ll = _np(input_lengths, np.int32), _np(label_lengths, np.int32)
    getattr(lib(), "orc_accumulate_grads" + sfx)(_p(E), _p(P), _p(eg), _p(pg), _p(lngrads), _p(LN),
                                                 _p(il), _p(ll), B, T, U, V)
    return eg, pg


def dense_grads_sep(E, P, egrads, pgrads, lngrads, deltas, precision="f32"):
    dt, sfx = _real(precision)
    E, P, lngrads, deltas = _np(E, dt), _np(P, dt), _np(lngrads, dt), _np(deltas, dt)
    eg, pg = np.array(egrads, dt, order="C"), np.array(pgrads, dt, order="C")
    B, T, U, V = _dims(E, P)
    getattr(lib(), "orc_dense_grads_sep" + sfx)(_p(E), _p(P), _p(eg), _p(pg), _p(lngrads),
                                                _p(deltas), B, T, U, V)
    return eg, pg


def best_labels(E, P, input_lengths=None, label_lengths=None, blank=0):
    E, P = _np(E, np.float32), _np(P, np.float32)
    B, T, U, V = _dims(E, P)
    il = None if input_lengths is None else _np(input_lengths, np.int32)
    ll = None if label_lengths is None else _np(label_lengths, np.int32)
    best = np.zeros((B, T, U), np.float32)
    arg = np.zeros((B, T, U), np.int32)
    lib().orc_best_labels_f32_table(_p(E), _p(P), _p(best), _p(arg), _p(il), _p(ll), B, T, U, V,
                                    blank)
    return best, arg


def loss_and_grads(E, P, labels, input_lengths, label_lengths, blank=0, deltas=None,
                   precision="f32", lse="naive"):
    """The torch-free end-to-end path of the reference's C++ tests (transducer/test.cpp:7-90):
    log-normaliser -> forward -> backward -> dense gradient accumulation.
    ``lse``: "naive" (test.h:51-80), "sep" (torch_binding.py:35-40,85-89, with deltas; inner
    sums in index order) or "sep8" (the same with eight partial sums per inner sum)."""
    dt, _ = _real(precision)
    B = E.shape[0]
    if lse == "naive":
        LN = log_norms_naive(E, P, input_lengths, label_lengths, precision)
    elif lse == "sep8":
        LN = log_norms_sep(E, P, precision, lanes=8)
    else:
        LN = log_norms_sep(E, P, precision)
    costs, alphas = forward(E, P, LN, labels, input_lengths, label_lengths, blank, precision)
    eg, pg, lng = backward(E, P, alphas, LN, labels, input_lengths, label_lengths, blank, precision)
    d = np.ones(B, dt) if deltas is None else _np(deltas, dt)
    if lse == "naive":
        eg, pg = accumulate_grads(E, P, eg, pg, lng, LN, input_lengths, label_lengths, precision)
        eg *= d[:, None, None]
        pg *= d[:, None, None]
    else:
        eg, pg = dense_grads_sep(E, P, eg, pg, lng, d, precision)
    return dict(costs=costs, alphas=alphas, log_norms=LN, lngrads=lng, egrads=eg, pgrads=pg)


# ---------------------------------------------------------------- compiled reference

def ref_forward(E, P, LN, labels, input_lengths, label_lengths, blank=0):
    E, P, LN = _np(E, np.float32), _np(P, np.float32), _np(LN, np.float32)
    B, T, U, V = _dims(E, P)
    labels = _np(labels, np.int32).reshape(B, max(U - 1, 0))
    il, ll = _np(input_lengths, np.int32), _np(label_lengths, np.int32)
    costs = np.empty(B, np.float32)
    alphas = np.full((B, T, U), np.nan, np.float32)
    ref().ref_forward(_p(E), _p(P), _p(costs), _p(alphas), _p(LN), _p(labels), _p(il), _p(ll),
                      B, T, U, V, blank)
    return costs, alphas


def ref_backward(E, P, alphas, LN, labels, input_lengths, label_lengths, blank=0):
    E, P, LN, alphas = (_np(x, np.float32) for x in (E, P, LN, alphas))
    B, T, U, V = _dims(E, P)
    labels = _np(labels, np.int32).reshape(B, max(U - 1, 0))
    il, ll = _np(input_lengths, np.int32), _np(label_lengths, np.int32)
    eg, pg, lng = np.empty_like(E), np.empty_like(P), np.empty_like(LN)
    ref().ref_backward(_p(E), _p(P), _p(eg), _p(pg), _p(lng), _p(alphas), _p(LN), _p(labels),
                       _p(il), _p(ll), B, T, U, V, blank)
    return eg, pg, lng


def ref_viterbi(E, P, LN, input_lengths, label_lengths, blank=0):
    E, P, LN = _np(E, np.float32), _np(P, np.float32), _np(LN, np.float32)
    B, T, U, V = _dims(E, P)
    il, ll = _np(input_lengths, np.int32), _np(label_lengths, np.int32)
    out = np.full((B, max(U - 1, 0)), -1, np.int32)
    ref().ref_viterbi(_p(E), _p(P), _p(LN), _p(out), _p(il), _p(ll), B, T, U, V, blank)
    return out


def ref_log_norms(E, P, input_lengths, label_lengths):
    E, P = _np(E, np.float32), _np(P, np.float32)
    B, T, U, V = _dims(E, P)
    il, ll = _np(input_lengths, np.int32), _np(label_lengths, np.int32)
    LN = np.empty((B, T, U), np.float32)
    ref().ref_compute_log_norms(_p(E), _p(P), _p(LN), _p(il), _p(ll), B, T, U, V)
    return LN


def ref_accumulate_grads(E, P, egrads, pgrads, lngrads, LN, input_lengths, label_lengths):
    E, P, LN, lngrads = (_np(x, np.float32) for x in (E, P, LN, lngrads))
    eg, pg = np.array(egrads, np.float32, order="C"), np.array(pgrads, np.float32, order="C")
    B, T, U, V = _dims(E, P)
    il, ll = _np(input_lengths, np.int32), _np(label_lengths, np.int32)
    ref().ref_accumulate_grads(_p(E), _p(P), _p(eg), _p(pg), _p(lngrads), _p(LN), _p(il), _p(ll),
                               B, T, U, V)
    return eg, pg
