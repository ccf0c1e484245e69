"""Pins the CPU oracle (oracle/) before anything is compared with it: the reference's own
golden vectors and closed form, the reference's compiled sources (bit for bit, via the committed
fixtures and -- where it was built -- oracle/_ref directly), brute-force path enumeration,
finite differences and the invariants of the lattice."""
import itertools
import math

import numpy as np
import pytest

import oracle
from transducer_amd.synthetic import CONFIGS, make_inputs, small_config
from util import check_close_reference, ref_cases, reference_vectors, vector_case

VEC = reference_vectors()


def full_path(E, P, labels, il, ll, precision="f32"):
    return oracle.loss_and_grads(E, P, labels, il, ll, precision=precision)


# ------------------------------------------------------------------ the reference's own vectors
def test_tiny_closed_form():
    # transducer/test.cpp:92-130: T=2, no labels, V=2 -- two forced blank moves
    E, P, labels, il, ll = vector_case(VEC["tiny"])
    e, p = E.astype(np.float64).ravel(), P.astype(np.float64).ravel()
    ln1 = math.log(math.exp(e[0] + p[0]) + math.exp(e[1] + p[1]))
    ln2 = math.log(math.exp(e[2] + p[0]) + math.exp(e[3] + p[1]))
    cost = -(e[0] + p[0] - ln1 + e[2] + p[0] - ln2)
    eg = [math.exp(e[0] + p[0] - ln1) - 1, math.exp(e[1] + p[1] - ln1),
          math.exp(e[2] + p[0] - ln2) - 1, math.exp(e[3] + p[1] - ln2)]
    pg = [eg[0] + eg[2], eg[1] + eg[3]]
    r = full_path(E, P, labels, il, ll)
    check_close_reference(r["costs"], [cost])
    check_close_reference(r["egrads"], eg)
    check_close_reference(r["pgrads"], pg)


@pytest.mark.parametrize("name", ["small", "big"])
@pytest.mark.parametrize("lse", ["naive", "sep"])
def test_golden_loss_and_grads(name, lse):
    v = VEC[name]
    E, P, labels, il, ll = vector_case(v)
    r = oracle.loss_and_grads(E, P, labels, il, ll, lse=lse)
    check_close_reference(r["costs"], v["costs"])
    check_close_reference(r["egrads"], v["egrads"])
    check_close_reference(r["pgrads"], v["pgrads"])


@pytest.mark.parametrize("name", ["viterbi_no_blanks", "viterbi_bigger"])
def test_golden_viterbi(name):
    v = VEC[name]
    E, P, _, il, ll = vector_case(v)
    LN = oracle.log_norms_naive(E, P, il, ll)
    got = oracle.viterbi(E, P, LN, il, ll)
    assert np.array_equal(got, np.array(v["labels"], np.int32))


def test_viterbi_empty_cases():
    # transducer/test.cpp:229-257: T=0 with nothing to read, and an empty transcript
    out = oracle.viterbi(np.zeros((1, 0, 2), np.float32), np.zeros((1, 1, 2), np.float32),
                         np.zeros((1, 0, 1), np.float32), [0], [0])
    assert out.shape == (1, 0)
    E, P, _, il, ll = vector_case(VEC["viterbi_empty_transcript"])
    LN = oracle.log_norms_naive(E, P, il, ll)
    assert oracle.viterbi(E, P, LN, il, ll).shape == (1, 0)


# ------------------------------------------------------------------ against the compiled reference
CASES = ref_cases()


@pytest.mark.parametrize("name", sorted(CASES))
def test_bit_exact_with_reference_fixture(name):
    c = CASES[name]
    E, P, labels, il, ll = (c[k] for k in ("emissions", "predictions", "labels", "input_lengths",
                                           "label_lengths"))
    LN = oracle.log_norms_naive(E, P, il, ll)
    assert np.array_equal(LN, c["log_norms"])
    costs, alphas = oracle.forward(E, P, LN, labels, il, ll)
    assert np.array_equal(costs, c["costs"])
    assert np.array_equal(alphas, c["alphas"], equal_nan=True)
    eg, pg, lng = oracle.backward(E, P, np.nan_to_num(alphas), LN, labels, il, ll)
    assert np.array_equal(eg, c["egrads_sparse"])
    assert np.array_equal(pg, c["pgrads_sparse"])
    assert np.array_equal(lng, c["lngrads"])
    eg2, pg2 = oracle.accumulate_grads(E, P, eg, pg, lng, LN, il, ll)
    assert np.array_equal(eg2, c["egrads"])
    assert np.array_equal(pg2, c["pgrads"])
    if "viterbi" in c:
        assert np.array_equal(oracle.viterbi(E, P, LN, il, ll), c["viterbi"])


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built (needs /root/reference)")
@pytest.mark.parametrize("shape", [(2, 300, 40, 50), (3, 64, 101, 17), (1, 2000, 20, 8)])
def test_bit_exact_with_reference_live(shape):
    d = make_inputs(small_config(*shape), seed=11)
    E, P, labels, il, ll = (d[k] for k in ("emissions", "predictions", "labels", "input_lengths",
                                           "label_lengths"))
    LN = oracle.log_norms_naive(E, P, il, ll)
    assert np.array_equal(LN, oracle.ref_log_norms(E, P, il, ll))
    costs, alphas = oracle.forward(E, P, LN, labels, il, ll)
    rc, ra = oracle.ref_forward(E, P, LN, labels, il, ll)
    assert np.array_equal(costs, rc) and np.array_equal(alphas, ra, equal_nan=True)
    a0 = np.nan_to_num(alphas)
    for mine, theirs in zip(oracle.backward(E, P, a0, LN, labels, il, ll),
                            oracle.ref_backward(E, P, a0, LN, labels, il, ll)):
        assert np.array_equal(mine, theirs)
    assert np.array_equal(oracle.viterbi(E, P, LN, il, ll), oracle.ref_viterbi(E, P, LN, il, ll))


# ------------------------------------------------------------------ what the mathematics fixes
def brute_force(E, P, labels, T, U, blank=0):
    """-log of the sum over every alignment (all interleavings of T blank moves and U-1 label
    moves whose last move is the final blank), in fp64, straight from the definition."""
    E, P = E.astype(np.float64), P.astype(np.float64)
    logp = E[:, None, :] + P[None, :, :]
    logp = logp - np.log(np.exp(logp).sum(-1, keepdims=True))
    total = 0.0
    for ups in itertools.combinations(range(T - 1 + U - 1), U - 1):
        t = u = 0
        lp = 0.0
        for step in range(T - 1 + U - 1):
            if step in ups:
                lp += logp[t, u, labels[u]]
                u += 1
            else:
                lp += logp[t, u, blank]
                t += 1
        lp += logp[T - 1, U - 1, blank]
        total += math.exp(lp)
    return -math.log(total)


@pytest.mark.parametrize("T,U,V", [(1, 1, 3), (1, 4, 5), (5, 1, 4), (4, 3, 5), (6, 4, 3)])
def test_cost_equals_sum_over_alignments(T, U, V):
    rng = np.random.default_rng(T * 100 + U * 10 + V)
    E = rng.standard_normal((1, T, V)).astype(np.float32)
    P = rng.standard_normal((1, U, V)).astype(np.float32)
    labels = rng.integers(1, V, (1, max(U - 1, 0))).astype(np.int32)
    want = brute_force(E[0], P[0], labels[0], T, U)
    for precision, tol in (("f64", 1e-12), ("f32", 2e-6)):
        r = oracle.loss_and_grads(E, P, labels, [T], [U - 1], precision=precision)
        assert abs(float(r["costs"][0]) - want) <= tol * max(1.0, abs(want))


def brute_force_viterbi(E, P, LN, T, U, blank=0):
    """Best total score over every alignment and every label choice, fp64; returns the score."""
    E, P, LN = E.astype(np.float64), P.astype(np.float64), LN.astype(np.float64)
    V = E.shape[1]
    best = -np.inf
    nb = [v for v in range(V) if v != blank]
    for ups in itertools.combinations(range(T - 1 + U - 1), U - 1):
        t = u = 0
        score = 0.0
        for step in range(T - 1 + U - 1):
            if step in ups:
                score += max(E[t, v] + P[u, v] for v in nb) - LN[t, u]
                u += 1
            else:
                score += E[t, blank] + P[u, blank] - LN[t, u]
                t += 1
        best = max(best, score)
    return best


def path_score(E, P, LN, labels, T, U, blank=0):
    """fp64 score of the best alignment that emits exactly `labels` (small DP over (t,u))."""
    E, P, LN = E.astype(np.float64), P.astype(np.float64), LN.astype(np.float64)
    s = np.full((T, U), -np.inf)
    s[0, 0] = 0.0
    for t in range(T):
        for u in range(U):
            if t > 0:
                s[t, u] = max(s[t, u], s[t - 1, u] + E[t - 1, blank] + P[u, blank] - LN[t - 1, u])
            if u > 0:
                l = labels[u - 1]
                s[t, u] = max(s[t, u], s[t, u - 1] + E[t, l] + P[u - 1, l] - LN[t, u - 1])
    return s[T - 1, U - 1]


@pytest.mark.parametrize("T,U,V", [(3, 3, 4), (5, 3, 6), (4, 4, 3)])
def test_viterbi_reaches_the_best_score(T, U, V):
    rng = np.random.default_rng(T * 100 + U * 10 + V)
    E = rng.standard_normal((1, T, V)).astype(np.float32)
    P = rng.standard_normal((1, U, V)).astype(np.float32)
    LN = oracle.log_norms_naive(E, P, [T], [U - 1])
    got = oracle.viterbi(E, P, LN, [T], [U - 1])[0]
    assert (got != 0).all()
    want = brute_force_viterbi(E[0], P[0], LN[0], T, U)
    assert abs(path_score(E[0], P[0], LN[0], got, T, U) - want) < 1e-5


def test_gradients_match_finite_differences():
    # the reference's recipe (torch_test.py:209-269) in fp64 with a tighter step
    d = make_inputs(small_config(3, 6, 2, 4), seed=3)
    E, P, labels, il, ll = (d[k] for k in ("emissions", "predictions", "labels", "input_lengths",
                                           "label_lengths"))
    E64, P64 = E.astype(np.float64), P.astype(np.float64)
    r = oracle.loss_and_grads(E64, P64, labels, il, ll, precision="f64")
    eps = 1e-6

    def total(Ex, Px):
        return oracle.loss_and_grads(Ex, Px, labels, il, ll, precision="f64")["costs"].sum()

    for arr, grad, is_e in ((E64, r["egrads"], True), (P64, r["pgrads"], False)):
        for idx in np.ndindex(arr.shape):
            up, dn = arr.copy(), arr.copy()
            up[idx] += eps
            dn[idx] -= eps
            num = (total(up, P64) - total(dn, P64)) if is_e else (total(E64, up) - total(E64, dn))
            assert abs(num / (2 * eps) - grad[idx]) < 1e-6, (is_e, idx)


def test_lattice_invariants():
    d = make_inputs(CONFIGS["cfg1"], seed=5)
    E, P, labels, il, ll = (d[k] for k in ("emissions", "predictions", "labels", "input_lengths",
                                           "label_lengths"))
    r = oracle.loss_and_grads(E, P, labels, il, ll, precision="f64")
    B, T, V = E.shape
    for b in range(B):
        Tb, Ub = il[b], ll[b] + 1
        # rows of a softmax-minus-target gradient sum to zero; padded rows are exactly zero
        assert np.abs(r["egrads"][b, :Tb].sum(-1)).max() < 1e-12
        assert np.abs(r["pgrads"][b, :Ub].sum(-1)).max() < 1e-12
        assert not r["egrads"][b, Tb:].any() and not r["pgrads"][b, Ub:].any()
        # every path crosses each anti-diagonal once: occupancies on a diagonal sum to one
        g = r["lngrads"][b]
        assert abs(g[0, 0] - 1.0) < 1e-12
        for s in range(Tb + Ub - 1):
            tot = sum(g[t, s - t] for t in range(Tb) if 0 <= s - t < Ub)
            assert abs(tot - 1.0) < 1e-10
        assert not g[Tb:].any() and not g[:, Ub:].any()


def test_separable_forms_agree_with_naive_forms():
    d = make_inputs(small_config(2, 20, 6, 40, sigma=2.0), seed=9)
    E, P, labels, il, ll = (d[k] for k in ("emissions", "predictions", "labels", "input_lengths",
                                           "label_lengths"))
    truth = oracle.log_norms_truth(E, P)
    assert np.abs(oracle.log_norms_sep(E, P, "f64") - truth).max() < 1e-12
    assert np.abs(oracle.log_norms_naive(E, P, precision="f64") - truth).max() < 1e-12
    assert np.abs(oracle.log_norms_sep(E, P) - truth).max() < 4e-6
    deltas = np.array([0.5, 2.0])
    a = oracle.loss_and_grads(E, P, labels, il, ll, deltas=deltas, precision="f64", lse="naive")
    b = oracle.loss_and_grads(E, P, labels, il, ll, deltas=deltas, precision="f64", lse="sep")
    assert np.abs(a["egrads"] - b["egrads"]).max() < 1e-12
    assert np.abs(a["pgrads"] - b["pgrads"]).max() < 1e-12


def test_empty_utterance_costs_infinity_and_zero_grads():
    # transducer/transducer_cpu.cpp:39-41, 92-94
    d = make_inputs(small_config(3, 5, 2, 4), seed=1)
    E, P, labels, il, ll = (d[k] for k in ("emissions", "predictions", "labels", "input_lengths",
                                           "label_lengths"))
    il = il.copy()
    il[1] = 0
    r = oracle.loss_and_grads(E, P, labels, il, ll)
    assert np.isposinf(r["costs"][1]) and np.isfinite(r["costs"][[0, 2]]).all()
    assert not r["egrads"][1].any() and not r["pgrads"][1].any() and not r["lngrads"][1].any()


def test_separable_log_norms_with_partial_sums_is_the_same_mathematics():
    """log_norms_sep(lanes=8) only re-orders the inner sum (eight partial sums, as a vectorised
    dot product forms them): the fp64 instance agrees with index order to fp64 rounding, the fp32
    instance to a few fp32 spacings, and the two are not bit-identical (else it would measure
    nothing)."""
    rng = np.random.default_rng(3)
    E = rng.standard_normal((2, 9, 301)).astype(np.float32)
    P = rng.standard_normal((2, 5, 301)).astype(np.float32)
    a64 = oracle.log_norms_sep(E, P, precision="f64")
    b64 = oracle.log_norms_sep(E, P, precision="f64", lanes=8)
    assert np.abs(a64 - b64).max() < 1e-13
    a32 = oracle.log_norms_sep(E, P)
    b32 = oracle.log_norms_sep(E, P, lanes=8)
    assert np.abs(a32 - a64).max() < 4e-6 and np.abs(b32 - a64).max() < 4e-6
    assert not np.array_equal(a32, b32)
    assert np.array_equal(oracle.log_norms_sep(E, P, lanes=1), a32)
