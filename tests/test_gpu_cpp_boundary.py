"""The reference's three C++ functions (transducer/transducer.h:3-49) as a caller of the
reference reaches them: the pybind module `_transducer` (transducer/_transducer.cpp:41-148) ->
libtransducer.so (include/transducer.h) -> the C interface -> the HIP kernels, with raw device
pointers and use_cuda=True.  The inputs and expected outputs are what the reference's compiled
CPU sources produced (tests/golden/ref_cases.npz) and the vectors its own tests hold
(transducer/test.cpp:92-226,259-308)."""
import numpy as np
import pytest

from util import (DeviceCase, assert_close, check_close_reference, gpu_backward, gpu_forward,
                  ref_cases, reference_vectors, vector_case)

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
import oracle  # noqa: E402
from transducer_amd import _transducer  # noqa: E402

CASES = ref_cases()
VEC = reference_vectors()


def p(t):
    return t.data_ptr() if t is not None else 0


def module_forward(c, LN, blank=0):
    B, T, U, V = c.dims
    costs = torch.full((B,), float("nan"), device="cuda:0")
    alphas = torch.full((B, T, U), float("nan"), device="cuda:0")
    d_LN = torch.tensor(LN, device="cuda:0")
    _transducer.forward(emissions=p(c.E), predictions=p(c.P), costs=p(costs), alphas=p(alphas),
                        logNorms=p(d_LN), labels=p(c.labels), input_lengths=p(c.il),
                        label_lengths=p(c.ll), batch_size=B, max_input_length=T,
                        max_label_length=U, alphabet_size=V, blank=blank, use_cuda=True)
    torch.cuda.synchronize()
    return costs.cpu().numpy(), alphas.cpu().numpy()


def module_backward(c, alphas, LN, blank=0):
    B, T, U, V = c.dims
    eg = torch.full_like(c.E, float("nan"))   # the library clears the outputs itself
    pg = torch.full_like(c.P, float("nan"))   # (transducer_cuda.cu:326-331)
    lng = torch.full((B, T, U), float("nan"), device="cuda:0")
    d_alphas = torch.tensor(np.nan_to_num(alphas), device="cuda:0")
    d_LN = torch.tensor(LN, device="cuda:0")
    _transducer.backward(emissions=p(c.E), predictions=p(c.P), egrads=p(eg), pgrads=p(pg),
                         lngrads=p(lng), alphas=p(d_alphas), logNorms=p(d_LN),
                         labels=p(c.labels), input_lengths=p(c.il), label_lengths=p(c.ll),
                         batch_size=B, max_input_length=T, max_label_length=U,
                         alphabet_size=V, blank=blank, use_cuda=True)
    torch.cuda.synchronize()
    return eg.cpu().numpy(), pg.cpu().numpy(), lng.cpu().numpy()


def module_viterbi(c, LN, blank=0):
    B, T, U, V = c.dims
    out = torch.full((B, max(U - 1, 0)), -1, dtype=torch.int32, device="cuda:0")
    d_LN = torch.tensor(LN, device="cuda:0")
    _transducer.viterbi(emissions=p(c.E), predictions=p(c.P), log_norms=p(d_LN),
                        labels=p(out) if U > 1 else 0, input_lengths=p(c.il),
                        label_lengths=p(c.ll), batch_size=B, max_input_length=T,
                        max_label_length=U, alphabet_size=V, blank=blank, use_cuda=True)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("name", sorted(CASES))
def test_the_three_functions_against_the_reference_fixture(name):
    f = CASES[name]
    c = DeviceCase(f["emissions"], f["predictions"], f["labels"], f["input_lengths"],
                   f["label_lengths"])
    LN = f["log_norms"]
    costs, alphas = module_forward(c, LN)
    assert np.array_equal(np.isinf(costs), np.isinf(f["costs"]))
    assert_close(costs, f["costs"], what="costs")
    assert np.array_equal(np.isnan(alphas), np.isnan(f["alphas"])), "cells outside stay untouched"
    assert_close(alphas, f["alphas"], what="alphas")
    eg, pg, lng = module_backward(c, f["alphas"], LN)
    assert_close(lng, f["lngrads"], what="lngrads")
    assert_close(eg, f["egrads_sparse"], what="egrads (sparse)")
    assert_close(pg, f["pgrads_sparse"], what="pgrads (sparse)")
    if "viterbi" in f:
        assert np.array_equal(module_viterbi(c, LN), f["viterbi"])
    # the same kernels as behind the C interface called directly: the same bits
    c_costs, c_alphas = gpu_forward(c, LN)
    assert np.array_equal(costs, c_costs) and np.array_equal(alphas, c_alphas, equal_nan=True)
    c_eg, c_pg, c_lng = gpu_backward(c, f["alphas"], LN)
    assert np.array_equal(eg, c_eg) and np.array_equal(pg, c_pg) and np.array_equal(lng, c_lng)


@pytest.mark.parametrize("name", ["small", "big"])
def test_vectors_of_the_reference_tests_through_the_module(name):
    """transducer/test.cpp:132-226: forward, backward and the torch-free dense accumulation of
    transducer/test.h:82-113 (the oracle's), compared with the costs and gradients the test holds."""
    v = VEC[name]
    E, P, labels, il, ll = vector_case(v)
    c = DeviceCase(E, P, labels, il, ll)
    LN = oracle.log_norms_naive(E, P, il, ll)
    costs, alphas = module_forward(c, LN)
    np.testing.assert_allclose(costs, np.array(v["costs"], np.float32), rtol=1e-6, atol=1e-5)
    eg, pg, lng = module_backward(c, alphas, LN)
    # the test's own next step (test.cpp:40-47): add the dense terms to the sparse gradients
    eg, pg = oracle.accumulate_grads(E, P, eg, pg, lng, LN, il, ll)
    check_close_reference(eg, v["egrads"])
    check_close_reference(pg, v["pgrads"])


@pytest.mark.parametrize("name", ["viterbi_no_blanks", "viterbi_bigger"])
def test_viterbi_vectors_of_the_reference_tests_through_the_module(name):
    v = VEC[name]
    E, P, labels, il, ll = vector_case(v)
    c = DeviceCase(E, P, labels, il, ll)
    LN = oracle.log_norms_naive(E, P, il, ll)
    assert np.array_equal(module_viterbi(c, LN), np.array(v["labels"], np.int32))


def test_failures_surface_as_the_reference_exception_types():
    """transducer.cpp:41 (std::invalid_argument -> ValueError) for the backend that is not built;
    a status of the C interface for bad sizes becomes ValueError as well."""
    with pytest.raises(ValueError):
        _transducer.forward(0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 2, 0, False)
    x = torch.zeros(16, device="cuda:0")
    with pytest.raises(ValueError):
        _transducer.forward(p(x), p(x), p(x), p(x), p(x), p(x), p(x), p(x), -1, 1, 1, 2, 0, True)
