"""The diagnostics of the lattice walks: the bounded wait between the two wavefronts of a long
label axis (its give-up path is forced from the host with a trip bound of zero; the kernel still
runs to its end) and the chain-latency floor probe."""
import ctypes

import numpy as np
import pytest

from util import DeviceCase, gpu_backward, gpu_forward, gpu_viterbi

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
import oracle  # noqa: E402
from transducer_amd import capi  # noqa: E402
from transducer_amd.synthetic import make_inputs, small_config  # noqa: E402

KEYS = ("emissions", "predictions", "labels", "input_lengths", "label_lengths")


@pytest.mark.parametrize("U", [100, 400])
def test_a_wait_that_runs_out_raises_the_flag_and_the_kernel_still_finishes(U):
    """101 label positions: two wavefronts of one workgroup wait for each other; 401: the alpha
    walk also runs the two halves of the label axis as two workgroups side by side, the upper
    one waiting (with the same bound) for the scores the lower one writes to memory."""
    lib = capi.load()
    d = make_inputs(small_config(2, 300, U, 16, ragged=False), seed=9)
    E, P, labels, il, ll = (d[k] for k in KEYS)
    LN = oracle.log_norms_naive(E, P, il, ll)
    want_costs, _ = oracle.forward(E, P, LN, labels, il, ll)
    c = DeviceCase(E, P, labels, il, ll)
    assert lib.rnnt_hip_check_kernels(None) == 0
    before = lib.rnnt_hip_set_spin_limit(0)
    try:
        _, alphas = gpu_forward(c, LN)          # returns: the walk finishes on whatever it finds
        gpu_viterbi(c, LN)
        if U > 256:                             # the dalpha walk of two halves waits the same way
            assert lib.rnnt_hip_check_kernels(None) == 2
            gpu_backward(c, np.nan_to_num(alphas, posinf=0.0, neginf=0.0), LN)
        assert lib.rnnt_hip_check_kernels(None) == 2
        assert b"gave up waiting" in lib.rnnt_hip_last_error()
        assert lib.rnnt_hip_check_kernels(None) == 0   # reading the flag clears it
    finally:
        assert lib.rnnt_hip_set_spin_limit(before) == 0
    costs, _ = gpu_forward(c, LN)
    paths = gpu_viterbi(c, LN)
    assert lib.rnnt_hip_check_kernels(None) == 0
    assert np.allclose(costs, want_costs, rtol=1e-4, atol=1e-5)
    assert np.array_equal(paths, oracle.viterbi(E, P, LN, il, ll))


def probe(x):
    from util import dev, ptr
    dx = dev(x)
    e = torch.empty_like(dx)
    l = torch.empty_like(dx)
    capi.call("rnnt_hip_libm_probe", ptr(dx), ptr(e), ptr(l), x.size, None)
    torch.cuda.synchronize()
    return e.cpu().numpy(), l.cpu().numpy()


def same_bits(a, b):
    nan = np.isnan(a) & np.isnan(b)
    return (a.view(np.uint32) == b.view(np.uint32)) | nan


def test_device_expf_and_log1pf_carry_the_bits_of_the_hosts_c_library():
    """The lattice kernels' expf / log1pf restate glibc's algorithms operation for operation
    (the reference's std::exp / std::log1p on floats, transducer_cpu.cpp:16-24,124-135).  Held
    here to the host's library on every 97th float of expf's range [-104.5, 2] and of log1pf's
    range [0, 1] (22 + 11 million arguments), on the special values and on random draws."""
    def every(lo_bits, hi_bits, step):
        return np.arange(lo_bits, hi_bits + 1, step, dtype=np.uint32).view(np.float32)
    f32 = lambda v: int(np.float32(v).view(np.uint32))
    neg = every(0x80000000, f32(-104.5), 97)
    pos = every(0, f32(2.0), 97)
    special = np.array([0.0, -0.0, 1.0, -1.0, 88.0, 88.72, 88.73, 100.0, -87.3, -87.4, -88.0,
                        -103.0, -103.9, -103.97, -103.98, -104.0, -200.0, np.inf, -np.inf, np.nan,
                        2.0 ** -29, 2.0 ** -30, 2.0 ** -54, 2.0 ** -55, 1e-45, 0.41421354,
                        0.41421357, 0.4142136, 0.99999994, 0.9999999, 0.99999, 2.0 ** -149],
                       np.float32)
    rng = np.random.default_rng(7)
    rnd = (rng.random(1 << 20, dtype=np.float32) * np.float32(106.5) - np.float32(104.5))
    x = np.concatenate([neg, pos, special, rnd.astype(np.float32)])
    e, l = probe(x)
    ok = same_bits(e, oracle.libm_expf(x))
    assert ok.all(), "expf: %d of %d differ, first at x=%r" % ((~ok).sum(), x.size, x[~ok][:3])
    sel = (~np.signbit(x) & (x <= 1.0)) | np.isnan(x)   # log1pf is restated for [+0, 1] only
    ok = same_bits(l[sel], oracle.libm_log1pf(x[sel]))
    assert ok.all(), "log1pf: %d of %d differ, first at x=%r" % ((~ok).sum(), sel.sum(),
                                                                  x[sel][~ok][:3])


def test_the_bound_behind_the_fast_log_sum_exp_holds_for_every_float():
    """alpha_kernel keeps a log-sum-exp formed on the hardware exp/log units only where it can
    show that the C library's sum rounds to the same float; that proof uses a bound on the fast
    value's distance from log1pf(expf(d)).  Here the bound is checked for all 2,139,095,041
    floats d in [-inf, -0] (on the device; its library values are the ones the test above holds
    to the host's); the largest distance found stays a twentieth or more below the bound."""
    lib = capi.load()
    bad = ctypes.c_ulonglong(123)
    ratio = ctypes.c_float(-1.0)
    assert lib.rnnt_hip_lse_bound_check(0x80000000, 0xff800000, ctypes.byref(bad),
                                        ctypes.byref(ratio)) == 0
    print("fast log-sum-exp: %d floats outside the bound, largest distance / bound = %.3f"
          % (bad.value, ratio.value))
    assert bad.value == 0
    assert 0.0 < ratio.value <= 0.95
    assert lib.rnnt_hip_lse_bound_check(0x3f800000, 0x40000000, ctypes.byref(bad),
                                        ctypes.byref(ratio)) == 1   # positive floats: refused


def test_chain_latency_floor_is_a_plausible_number_of_nanoseconds():
    lib = capi.load()
    out = ctypes.c_double(0.0)
    for kind, lo, hi in ((0, 20.0, 200.0), (1, 2.0, 60.0), (2, 60.0, 500.0)):
        assert lib.rnnt_hip_chain_floor(kind, 20000, ctypes.byref(out)) == 0
        print("chain floor kind %d: %.1f ns per step" % (kind, out.value))
        assert lo < out.value < hi
    assert lib.rnnt_hip_chain_floor(3, 100, ctypes.byref(out)) == 1
    assert lib.rnnt_hip_chain_floor(0, 0, ctypes.byref(out)) == 1


def test_scratch_pool_can_be_released_between_calls():
    """The allocating entry points take their scratch from a pool that keeps freed blocks;
    rnnt_hip_release_scratch hands them back to the driver, and the next call allocates afresh
    with the same results."""
    from util import DeviceCase, gpu_forward, gpu_log_norms, gpu_viterbi
    rng = np.random.default_rng(3)
    B, T, U, V = 2, 40, 9, 50
    E = rng.standard_normal((B, T, V)).astype(np.float32)
    P = rng.standard_normal((B, U, V)).astype(np.float32)
    labels = rng.integers(1, V, (B, U - 1)).astype(np.int32)
    il, ll = np.array([T, T - 3], np.int32), np.array([U - 1, U - 2], np.int32)
    c = DeviceCase(E, P, labels, il, ll)
    lib = capi.load()
    LN = gpu_log_norms(c)
    costs, alphas = gpu_forward(c, LN)
    paths = gpu_viterbi(c, LN)
    assert lib.rnnt_hip_release_scratch() == 0
    assert lib.rnnt_hip_release_scratch() == 0   # nothing held: still fine
    costs2, alphas2 = gpu_forward(c, LN)
    assert np.array_equal(costs, costs2) and np.array_equal(np.nan_to_num(alphas), np.nan_to_num(alphas2))
    assert np.array_equal(paths, gpu_viterbi(c, LN))
