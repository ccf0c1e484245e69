"""Parity of the HIP path with the CPU oracle, through the C interface of librnnt_hip.so.

Boundary tests feed both sides the same log_norms (the contract of transducer.h: the
normaliser is an input there), so the lattice recursions are compared on their own; the
log-normaliser and the dense gradient kernels are gated separately; end-to-end runs close the
loop.  Tolerance for costs and gradients: rel 1e-4 / abs 1e-5 in fp32; viterbi paths exact."""
import numpy as np
import pytest

import oracle
from transducer_amd.synthetic import CONFIGS, make_inputs, small_config
from util import (DeviceCase, assert_close, assert_same_bits, check_close_reference, gpu_backward, gpu_dense_grads,
                  gpu_forward, gpu_log_norms, gpu_loss, gpu_viterbi, ref_cases, reference_vectors,
                  vector_case, violations)

pytestmark = pytest.mark.gpu

VEC = reference_vectors()
CASES = ref_cases()
KEYS = ("emissions", "predictions", "labels", "input_lengths", "label_lengths")


def unpack(d):
    return tuple(d[k] for k in KEYS)


# ------------------------------------------------------------------ reference-held vectors
@pytest.mark.parametrize("name", ["small", "big"])
def test_golden_vectors_whole_loss(name):
    v = VEC[name]
    E, P, labels, il, ll = vector_case(v)
    costs, eg, pg = gpu_loss(DeviceCase(E, P, labels, il, ll))
    # the reference's own bar for these vectors (transducer/test.cpp:51,86-87)
    check_close_reference(costs, v["costs"])
    check_close_reference(eg, v["egrads"])
    check_close_reference(pg, v["pgrads"])


def test_tiny_closed_form_whole_loss():
    E, P, labels, il, ll = vector_case(VEC["tiny"])
    want = oracle.loss_and_grads(E, P, labels, il, ll, precision="f64")
    costs, eg, pg = gpu_loss(DeviceCase(E, P, labels, il, ll))
    check_close_reference(costs, want["costs"])
    check_close_reference(eg, want["egrads"])
    check_close_reference(pg, want["pgrads"])


@pytest.mark.parametrize("name", ["viterbi_no_blanks", "viterbi_bigger"])
def test_golden_viterbi(name):
    v = VEC[name]
    E, P, labels, il, ll = vector_case(v)
    c = DeviceCase(E, P, labels, il, ll)
    LN = oracle.log_norms_naive(E, P, il, ll)
    assert np.array_equal(gpu_viterbi(c, LN), np.array(v["labels"], np.int32))


def test_viterbi_empty_inputs_are_accepted():
    # transducer/test.cpp:229-257
    from transducer_amd import capi
    from util import dev, ptr
    il, ll = dev(np.array([0], np.int32)), dev(np.array([0], np.int32))
    capi.call("rnnt_hip_viterbi", None, None, None, None, ptr(il), ptr(ll), 1, 0, 1, 2, 0, None)
    E, P, labels, il, ll = vector_case(VEC["viterbi_empty_transcript"])
    c = DeviceCase(E, P, labels, il, ll)
    LN = oracle.log_norms_naive(E, P, il, ll)
    assert gpu_viterbi(c, LN).shape == (1, 0)


# ------------------------------------------------------------------ transducer.h boundary
@pytest.mark.parametrize("name", sorted(CASES))
def test_boundary_against_reference_fixture(name):
    """forward / backward / viterbi with the fixture's log_norms against what the reference's
    compiled CPU sources produced (ragged lengths, empty utterances, empty labels, ties)."""
    f = CASES[name]
    E, P, labels, il, ll = unpack(f)
    c = DeviceCase(E, P, labels, il, ll)
    LN = f["log_norms"]
    costs, alphas = gpu_forward(c, LN)
    assert np.array_equal(np.isinf(costs), np.isinf(f["costs"]))
    assert_close(costs, f["costs"], what="costs")
    assert np.array_equal(np.isnan(alphas), np.isnan(f["alphas"])), "cells outside must be untouched"
    # The lattice kernels use the C library's own expf / log1pf and the reference's order of
    # operations: with the same log_norms every alpha, every dalpha and every blank / label
    # term carries the bits the reference's compiled CPU sources produced.
    assert_same_bits(costs, f["costs"], what="costs")
    assert_same_bits(alphas, f["alphas"], what="alphas")
    eg, pg, lng = gpu_backward(c, alphas, LN)
    assert_same_bits(lng, f["lngrads"], what="lngrads")
    assert_same_bits(eg, f["egrads_sparse"], what="egrads (sparse)")
    assert_same_bits(pg, f["pgrads_sparse"], what="pgrads (sparse)")
    if "viterbi" in f:
        got = gpu_viterbi(c, LN)
        assert np.array_equal(got, f["viterbi"])


def long_case(B, V, seed, sigma=1.0, ragged=True, T=2000, U=100):
    cfg = small_config(B, T, U, V, sigma=sigma, ragged=ragged)
    return unpack(make_inputs(cfg, seed=seed))


@pytest.mark.parametrize("B", [1, 10])
@pytest.mark.parametrize("T", [1, 10, 100])
def test_reference_stress_grid(B, T):
    """The grid of the reference's CPU-against-GPU stress test at its own sizes
    (transducer/test_cuda.cu:323-378: uniform [0,1) scores, input lengths in [0,T], label
    lengths in [0,U-1], host-computed log_norms, forward + backward + dense accumulation), at
    this build's tolerance instead of the reference's 1e-3 / 1e-4 where both sides are given the
    same log_norms."""
    rng = np.random.Generator(np.random.Philox(key=1000 * B + T))
    for U in (1, 10, 100):
        for V in (8, 20, 32, 101, 128):
            print("stress case B=%d T=%d U=%d V=%d" % (B, T, U, V), flush=True)
            E = rng.random((B, T, V), dtype=np.float32)
            P = rng.random((B, U, V), dtype=np.float32)
            il = rng.integers(0, T + 1, B).astype(np.int32)
            ll = rng.integers(0, U, B).astype(np.int32)
            labels = rng.integers(1, V, (B, U - 1)).astype(np.int32)
            LN = oracle.log_norms_naive(E, P, il, ll)
            costs_o, alphas_o = oracle.forward(E, P, LN, labels, il, ll)
            eg_o, pg_o, lng_o = oracle.backward(E, P, np.nan_to_num(alphas_o), LN, labels, il, ll)
            ed_o, pd_o = oracle.accumulate_grads(E, P, eg_o, pg_o, lng_o, LN, il, ll)
            c = DeviceCase(E, P, labels, il, ll)
            costs, alphas = gpu_forward(c, LN)
            assert np.array_equal(np.isinf(costs), np.isinf(costs_o))
            assert_close(costs, costs_o, what="costs")
            eg, pg, lng = gpu_backward(c, alphas, LN)
            assert_close(lng, lng_o, what="lngrads")
            ed, pd = gpu_dense_grads(c, eg, pg, lng, LN)
            assert_close(ed, ed_o, what="egrads")
            assert_close(pd, pd_o, what="pgrads")
            # and the fused path, which computes log_norms itself (a last-bit difference there
            # moves a rounding in alpha, ~6e-5 at |alpha| ~ 1e3): held to the reference's own
            # bar for this test (test_cuda.cu:371-373)
            costs_f, ed_f, pd_f = gpu_loss(c)
            fin = np.isfinite(costs_o)
            assert np.array_equal(np.isinf(costs_f), np.isinf(costs_o))
            assert_close(costs_f[fin], costs_o[fin], what="costs (fused)")
            assert_close(ed_f, ed_o, rtol=1e-3, atol=1e-4, what="egrads (fused)")
            assert_close(pd_f, pd_o, rtol=1e-3, atol=1e-4, what="pgrads (fused)")


@pytest.mark.parametrize("V,sigma,ragged", [(100, 1.0, False), (300, 2.0, True)])
def test_boundary_at_T2000(V, sigma, ragged):
    """The lattice at its real length.  alpha reaches ~1e4 here (ulp ~1e-3), so gradients only
    agree if the rounding sequence of every cell follows the reference."""
    E, P, labels, il, ll = long_case(2, V, seed=21, sigma=sigma, ragged=ragged)
    LN = oracle.log_norms_naive(E, P, il, ll)
    costs_o, alphas_o = oracle.forward(E, P, LN, labels, il, ll)
    c = DeviceCase(E, P, labels, il, ll)
    costs, alphas = gpu_forward(c, LN)
    # same expf / log1pf, same order of operations: the same bits in every cell
    assert_same_bits(costs, costs_o, what="costs")
    assert_same_bits(alphas, alphas_o, what="alphas")
    # backward from the device's own alphas, as a caller would chain the two calls
    eg, pg, lng = gpu_backward(c, alphas, LN)
    eg_o, pg_o, lng_o = oracle.backward(E, P, np.nan_to_num(alphas_o), LN, labels, il, ll)
    assert_same_bits(lng, lng_o, what="lngrads")
    assert_same_bits(eg, eg_o, what="egrads (sparse)")
    assert_same_bits(pg, pg_o, what="pgrads (sparse)")
    # every path crosses each anti-diagonal exactly once
    for b in range(E.shape[0]):
        Tb, Ub = il[b], ll[b] + 1
        g = lng[b, :Tb, :Ub].astype(np.float64)
        diag = np.array([np.trace(g[::-1], offset=k) for k in range(-(Tb - 1), Ub)])
        assert np.abs(diag - 1.0).max() < 2e-2


def minus_inf_case(shape, kind, seed=5):
    """Scores of -inf as a caller masks them: the blank from the middle of every utterance on
    (no path reaches the end: cost +inf), one blank score of the predictions, one label score
    of one frame, one label score of the predictions (no path again)."""
    B, T, U, V = shape
    E, P, labels, il, ll = (a.copy() for a in unpack(
        make_inputs(small_config(B, T, U - 1, V, ragged=True), seed=seed)))
    il[0], ll[0] = T, U - 1
    for b in range(B):
        Tb, Ub = il[b], ll[b] + 1
        if kind == "blank_tail":
            E[b, Tb // 2:, 0] = -np.inf
        elif kind == "blank_p":
            P[b, Ub // 2, 0] = -np.inf
        elif kind == "label_cell" and Ub > 1:
            E[b, Tb // 3, labels[b, (Ub - 1) // 2]] = -np.inf
        elif kind == "label_row" and Ub > 1:
            P[b, (Ub - 1) // 2, labels[b, (Ub - 1) // 2]] = -np.inf
    return E, P, labels, il, ll


# U = 1 (first column only), one wavefront, two wavefronts, two blocks of 1024 positions
@pytest.mark.parametrize("shape", [(2, 12, 1, 8), (3, 40, 9, 16), (2, 150, 101, 24),
                                   (2, 20, 1100, 6)])
@pytest.mark.parametrize("kind", ["blank_tail", "blank_p", "label_cell", "label_row"])
def test_minus_inf_scores_follow_the_reference(shape, kind):
    """transducer/transducer_cpu.cpp:16-24,43-60: a score of -inf gives alphas of -inf (not a
    large finite number), an unreachable last cell a cost of +inf, and the backward pass the
    NaN (inf - inf) and 0 (exp(-inf)) entries the reference produces.  Same bits as the
    oracle at the transducer.h boundary, infinities and NaN positions included."""
    E, P, labels, il, ll = minus_inf_case(shape, kind)
    LN = oracle.log_norms_naive(E, P, il, ll)
    assert np.isfinite(LN[~np.isnan(LN)]).all()
    costs_o, alphas_o = oracle.forward(E, P, LN, labels, il, ll)
    c = DeviceCase(E, P, labels, il, ll)
    costs, alphas = gpu_forward(c, LN)
    assert np.array_equal(np.isposinf(costs), np.isposinf(costs_o))
    assert_same_bits(costs, costs_o, what="costs")
    assert np.array_equal(np.isneginf(alphas), np.isneginf(alphas_o)), "-inf alphas"
    assert np.array_equal(np.isnan(alphas), np.isnan(alphas_o)), "cells outside must be untouched"
    assert_same_bits(alphas, alphas_o, what="alphas")
    # backward from these alphas (cells outside the lattice cleared, -inf kept)
    import torch
    from transducer_amd import capi
    from util import dev, ptr
    B, T, U, V = c.dims
    a_in = np.where(np.isnan(alphas_o), np.float32(0), alphas_o)
    eg_o, pg_o, lng_o = oracle.backward(E, P, a_in, LN, labels, il, ll)
    eg = torch.full_like(c.E, float("nan"))
    pg = torch.full_like(c.P, float("nan"))
    lng = torch.full((B, T, U), float("nan"), device=c.E.device)
    d_alphas, d_LN = dev(a_in), dev(LN)
    capi.call("rnnt_hip_backward", ptr(c.E), ptr(c.P), ptr(eg), ptr(pg), ptr(lng), ptr(d_alphas),
              ptr(d_LN), ptr(c.labels), ptr(c.il), ptr(c.ll), B, T, U, V, 0, None)
    torch.cuda.synchronize()
    for got, want, name in ((lng, lng_o, "lngrads"), (eg, eg_o, "egrads (sparse)"),
                            (pg, pg_o, "pgrads (sparse)")):
        got = got.cpu().numpy()
        assert np.array_equal(np.isnan(got), np.isnan(want)), name + ": NaN positions"
        assert_same_bits(got, want, what=name)
    # the whole loss: +inf costs where the oracle has them, finite ones and every finite
    # gradient entry within the tolerance, NaN where the oracle has NaN
    if U > 128:  # (a label axis this long is compared end to end in its own test)
        return
    want = oracle.loss_and_grads(E, P, labels, il, ll)
    costs_f, eg_f, pg_f = gpu_loss(c)
    assert np.array_equal(np.isposinf(costs_f), np.isposinf(want["costs"]))
    fin = np.isfinite(want["costs"])
    assert_close(costs_f[fin], want["costs"][fin], what="costs (whole loss)")
    assert_close(eg_f, want["egrads"], what="egrads (whole loss)")  # (NaN positions included)
    assert_close(pg_f, want["pgrads"], what="pgrads (whole loss)")


@pytest.mark.parametrize("near_ties", [False, True])
def test_viterbi_at_T2000_is_bit_exact(near_ties):
    cfg = small_config(3, 2000, 100, 64, ragged=True)
    d = make_inputs(cfg, seed=31, near_ties=near_ties)
    E, P, labels, il, ll = unpack(d)
    LN = oracle.log_norms_naive(E, P, il, ll)
    want = oracle.viterbi(E, P, LN, il, ll)
    got = gpu_viterbi(DeviceCase(E, P, labels, il, ll), LN)
    assert np.array_equal(got, want)


def test_viterbi_decision_table_in_global_memory():
    """T large enough that the table of decision bits (and the hand-over array of the two
    wavefronts) no longer fits LDS: the kernel's other code paths."""
    cfg = small_config(2, 9000, 100, 12, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=33))
    LN = oracle.log_norms_naive(E, P, il, ll)
    want = oracle.viterbi(E, P, LN, il, ll)
    c = DeviceCase(E, P, labels, il, ll)
    assert np.array_equal(gpu_viterbi(c, LN), want)
    costs_o, alphas_o = oracle.forward(E, P, LN, labels, il, ll)
    costs, alphas = gpu_forward(c, LN)
    assert_close(costs, costs_o, rtol=1e-4, atol=1e-2, what="costs")


def test_viterbi_label_equal_to_nonzero_blank():
    cfg = small_config(2, 40, 12, 9, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=4))
    LN = oracle.log_norms_naive(E, P, il, ll)
    for blank in (3, 8):
        want = oracle.viterbi(E, P, LN, il, ll, blank=blank)
        got = gpu_viterbi(DeviceCase(E, P, labels, il, ll), LN, blank=blank)
        assert np.array_equal(got, want)


def test_labels_may_repeat_and_equal_blank():
    # transducer/benchmark.cpp:47 draws labels from [0,V): blank may appear as a label
    cfg = small_config(3, 30, 8, 5, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=8))
    labels = labels.copy()
    labels[:, ::2] = 0
    labels[:, 1::2] = 2
    LN = oracle.log_norms_naive(E, P, il, ll)
    costs_o, alphas_o = oracle.forward(E, P, LN, labels, il, ll)
    eg_o, pg_o, lng_o = oracle.backward(E, P, np.nan_to_num(alphas_o), LN, labels, il, ll)
    c = DeviceCase(E, P, labels, il, ll)
    costs, alphas = gpu_forward(c, LN)
    assert_close(costs, costs_o, what="costs")
    eg, pg, lng = gpu_backward(c, alphas_o, LN)
    assert_close(eg, eg_o, what="egrads (sparse)")
    assert_close(pg, pg_o, what="pgrads (sparse)")
    assert_close(lng, lng_o, what="lngrads")


def test_long_label_axis_uses_more_cells_per_lane():
    cfg = small_config(2, 60, 300, 11, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=12))
    LN = oracle.log_norms_naive(E, P, il, ll)
    costs_o, alphas_o = oracle.forward(E, P, LN, labels, il, ll)
    c = DeviceCase(E, P, labels, il, ll)
    costs, alphas = gpu_forward(c, LN)
    assert_close(costs, costs_o, what="costs")
    eg, pg, lng = gpu_backward(c, alphas_o, LN)
    eg_o, pg_o, lng_o = oracle.backward(E, P, np.nan_to_num(alphas_o), LN, labels, il, ll)
    assert_close(lng, lng_o, what="lngrads")
    assert_close(eg, eg_o, what="egrads")
    assert np.array_equal(gpu_viterbi(c, LN), oracle.viterbi(E, P, LN, il, ll))


@pytest.mark.parametrize("T", [1, 6, 45])
@pytest.mark.parametrize("U", [128, 129, 192, 256, 257, 300, 512, 513, 768, 1000])
def test_label_axes_dealt_to_several_wavefronts_carry_the_reference_bits(T, U):
    """From 65 label positions the alpha walk and from 129 the dalpha walk deal the label axis to
    two or four wavefronts of one workgroup, which hand the boundary column's score on through
    LDS and wait for each other's progress counters (four from 129 positions; from 257 a small
    batch like this one is walked as two halves side by side, and past 512 a lane owns two to
    four positions, those of the dalpha walk 64 apart).  U counts the rows of predictions and sits on
    either side of every change of that split; T = 1 and 6 leave most wavefronts with less than
    one or two groups of four steps, 45 lets them fall the few groups behind that they run at.
    Same bars as everywhere: the reference's bits in every alpha, dalpha and sparse term, the
    exact path."""
    cfg = small_config(3, T, U - 1, 6, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=1000 * T + U))
    il[0], ll[0] = T, U - 1          # one utterance uses every wavefront
    il[1], ll[1] = max(T - 2, 1), (U - 1) // 2   # one ends inside the label axis
    c = DeviceCase(E, P, labels, il, ll)
    LN = oracle.log_norms_naive(E, P, il, ll)
    costs_o, alphas_o = oracle.forward(E, P, LN, labels, il, ll)
    costs, alphas = gpu_forward(c, LN)
    assert_same_bits(costs, costs_o, what="costs")
    assert_same_bits(alphas, alphas_o, what="alphas")
    eg, pg, lng = gpu_backward(c, alphas, LN)
    eg_o, pg_o, lng_o = oracle.backward(E, P, np.nan_to_num(alphas_o), LN, labels, il, ll)
    assert_same_bits(lng, lng_o, what="lngrads")
    assert_same_bits(eg, eg_o, what="egrads (sparse)")
    assert_same_bits(pg, pg_o, what="pgrads (sparse)")
    assert np.array_equal(gpu_viterbi(c, LN), oracle.viterbi(E, P, LN, il, ll))


@pytest.mark.parametrize("B,T,U", [(11, 300, 400), (3, 700, 258), (17, 150, 512), (96, 40, 300),
                                   (97, 40, 300)])
def test_two_halves_of_a_label_axis_walked_side_by_side_carry_the_reference_bits(B, T, U):
    """257 .. 512 label positions in a batch of at most 96 utterances: the alpha and the dalpha
    walk run the two halves of the label axis as two workgroups at the same time; the values of
    the boundary column cross through memory, each with the number of its step beside it, and
    the half that follows asks again for what was not there yet.  Long enough lattices that it
    runs its steady state a few groups of steps behind the half that leads; batches that fill the last eight
    workgroup slots only partly; 97 utterances take the one-workgroup walk again.  U counts the
    rows of predictions."""
    cfg = small_config(B, T, U - 1, 5, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=B * 1000 + U))
    il[0], ll[0] = T, U - 1                  # one utterance uses both halves to the end
    il[1], ll[1] = max(T // 3, 1), 255       # one ends at the boundary: 256 positions
    il[2], ll[2] = T, 256                    # one puts a single position into the upper half
    c = DeviceCase(E, P, labels, il, ll)
    LN = oracle.log_norms_naive(E, P, il, ll)
    costs_o, alphas_o = oracle.forward(E, P, LN, labels, il, ll)
    eg_o, pg_o, lng_o = oracle.backward(E, P, np.nan_to_num(alphas_o), LN, labels, il, ll)
    for _ in range(2):                       # the second call finds the first one's entries
        costs, alphas = gpu_forward(c, LN)
        assert_same_bits(costs, costs_o, what="costs")
        assert_same_bits(alphas, alphas_o, what="alphas")
        eg, pg, lng = gpu_backward(c, alphas, LN)
        assert_same_bits(lng, lng_o, what="lngrads")
        assert_same_bits(eg, eg_o, what="egrads (sparse)")
        assert_same_bits(pg, pg_o, what="pgrads (sparse)")
    from transducer_amd import capi
    assert capi.load().rnnt_hip_check_kernels(None) == 0


@pytest.mark.parametrize("B,T,U", [(5, 200, 513), (9, 120, 700), (3, 60, 1000), (4, 90, 1025),
                                   (2, 40, 2100), (70, 6, 600), (40, 5, 1025), (12, 4, 4200),
                                   (300, 3, 1100)])
def test_label_axis_as_a_chain_of_blocks_side_by_side_and_where_it_is_not(B, T, U):
    """From 513 label positions the alpha and dalpha walks run three and more blocks of 256
    positions side by side, each following the one before it through its own array of tagged
    entries -- up to 1024 positions as long as the batch leaves the device the CUs for it
    (utterances x blocks at most 192), beyond whatever the batch (40 x 5 workgroups, 300 x 5:
    more than the device runs at once, so later utterances' blocks queue behind earlier ones).
    70 x 3 workgroups for 600 positions are too many and 17 blocks too long: those take one
    workgroup per utterance again, a lane owning several positions, or a launch per 1024
    positions.  Either way the reference's bits.  U counts the rows of
    predictions; ragged batches, so that some utterances end blocks below the top one."""
    cfg = small_config(B, T, U - 1, 4, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=B * 7 + U))
    il[0], ll[0] = T, U - 1
    il[1], ll[1] = max(T // 2, 1), 256        # one position in the second block
    c = DeviceCase(E, P, labels, il, ll)
    LN = oracle.log_norms_naive(E, P, il, ll)
    costs_o, alphas_o = oracle.forward(E, P, LN, labels, il, ll)
    eg_o, pg_o, lng_o = oracle.backward(E, P, np.nan_to_num(alphas_o), LN, labels, il, ll)
    for _ in range(2):
        costs, alphas = gpu_forward(c, LN)
        assert_same_bits(costs, costs_o, what="costs")
        assert_same_bits(alphas, alphas_o, what="alphas")
        eg, pg, lng = gpu_backward(c, alphas, LN)
        assert_same_bits(lng, lng_o, what="lngrads")
        assert_same_bits(eg, eg_o, what="egrads (sparse)")
        assert_same_bits(pg, pg_o, what="pgrads (sparse)")
    from transducer_amd import capi
    assert capi.load().rnnt_hip_check_kernels(None) == 0


@pytest.mark.parametrize("B,T,U", [(2, 13000, 70), (2, 12500, 200), (1, 20000, 300), (3, 12400, 129),
                                   (1, 40000, 30), (1, 37000, 150)])
def test_very_long_utterances_keep_their_wavefronts(B, T, U):
    """Past about 12000 anti-diagonals the three hand-over arrays of four wavefronts no longer fit
    LDS: the walks then deal the label axis to workgroups of two wavefronts (one array, good for
    36000 anti-diagonals), up to 128 positions one workgroup, beyond blocks of 128 side by side;
    past 36000 anti-diagonals one wavefront per utterance walks the whole label axis.
    The reference's bits and the exact path, as everywhere."""
    cfg = small_config(B, T, U - 1, 4, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=T + U))
    il[0], ll[0] = T, U - 1
    c = DeviceCase(E, P, labels, il, ll)
    LN = oracle.log_norms_naive(E, P, il, ll)
    costs_o, alphas_o = oracle.forward(E, P, LN, labels, il, ll)
    costs, alphas = gpu_forward(c, LN)
    assert_same_bits(costs, costs_o, what="costs")
    assert_same_bits(alphas, alphas_o, what="alphas")
    eg, pg, lng = gpu_backward(c, alphas, LN)
    eg_o, pg_o, lng_o = oracle.backward(E, P, np.nan_to_num(alphas_o), LN, labels, il, ll)
    assert_same_bits(lng, lng_o, what="lngrads")
    assert_same_bits(eg, eg_o, what="egrads (sparse)")
    assert np.array_equal(gpu_viterbi(c, LN), oracle.viterbi(E, P, LN, il, ll))


def test_two_halves_side_by_side_keep_their_bits_while_the_device_is_busy():
    """How far the half that follows runs behind the half that leads depends on when their two
    workgroups get their CUs; with matrix products on a second stream keeping every CU busy the
    follower meets entries that are not written yet and takes its bounded wait.  Whatever the
    timing: the reference's bits, call after call, and no wait given up."""
    import torch
    from transducer_amd import capi
    B, T, U = 24, 600, 400
    cfg = small_config(B, T, U - 1, 4, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=77))
    il[0], ll[0] = T, U - 1
    c = DeviceCase(E, P, labels, il, ll)
    LN = oracle.log_norms_naive(E, P, il, ll)
    costs_o, alphas_o = oracle.forward(E, P, LN, labels, il, ll)
    _, _, lng_o = oracle.backward(E, P, np.nan_to_num(alphas_o), LN, labels, il, ll)
    side = torch.cuda.Stream()
    X = torch.randn(4096, 4096, device=c.E.device)
    for _ in range(8):
        with torch.cuda.stream(side):
            for _ in range(4):
                X @ X
        costs, alphas = gpu_forward(c, LN)
        _, _, lng = gpu_backward(c, alphas, LN)
        assert_same_bits(costs, costs_o, what="costs")
        assert_same_bits(alphas, alphas_o, what="alphas")
        assert_same_bits(lng, lng_o, what="lngrads")
    torch.cuda.synchronize()
    assert capi.load().rnnt_hip_check_kernels(None) == 0


@pytest.mark.parametrize("T,U,V", [(40, 1024, 9), (30, 1025, 9), (50, 1500, 7), (24, 2100, 520),
                                   (300, 1300, 5)])
def test_label_axis_longer_than_one_block_of_1024_positions(T, U, V):
    """A workgroup of the lattice walks takes at most 1024 label positions.  A longer axis is
    walked in blocks, the scores of the boundary column handed on through memory: the best path
    a launch per 1024 positions, lowest block first; alpha and dalpha as blocks of 256 positions
    side by side (a batch this small; the other form of theirs is covered by
    test_label_axis_as_a_chain_of_blocks_side_by_side_and_where_it_is_not).  The reference
    strides its loop instead (transducer_cuda.cu:74,150,220).  U counts the rows of predictions:
    for the best path 1024 is the last single block, 1025 the first double one, 2100 takes
    three; V = 520 also takes the whole loss
    through the scattered blank / label terms (the folded ones stop at 1024 labels).  Same bars
    as everywhere: the reference's bits at the boundary, the oracle's tolerance for the loss,
    the exact path."""
    cfg = small_config(2, T, U - 1, V, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=U))
    il[0], ll[0] = T, U - 1          # one utterance uses every block, the other is ragged
    ll[1] = min(ll[1], U - 1)
    c = DeviceCase(E, P, labels, il, ll)
    LN = oracle.log_norms_naive(E, P, il, ll)
    costs_o, alphas_o = oracle.forward(E, P, LN, labels, il, ll)
    costs, alphas = gpu_forward(c, LN)
    assert_same_bits(costs, costs_o, what="costs")
    assert_same_bits(alphas, alphas_o, what="alphas")
    eg, pg, lng = gpu_backward(c, alphas, LN)
    eg_o, pg_o, lng_o = oracle.backward(E, P, np.nan_to_num(alphas_o), LN, labels, il, ll)
    assert_same_bits(lng, lng_o, what="lngrads")
    assert_same_bits(eg, eg_o, what="egrads (sparse)")
    assert_same_bits(pg, pg_o, what="pgrads (sparse)")
    assert np.array_equal(gpu_viterbi(c, LN), oracle.viterbi(E, P, LN, il, ll))
    # the whole loss on the device's own log-normaliser: fed that LN the oracle agrees in every
    # entry; against the oracle's own LN a lattice this long along the label axis moves with the
    # last bit of LN, and the bar is the spread of the reference's result between two summation
    # orders of its own LN
    costs, eg, pg = gpu_loss(c)
    LNd = gpu_log_norms(c)
    oc, oa = oracle.forward(E, P, LNd, labels, il, ll)
    oeg, opg, olng = oracle.backward(E, P, np.nan_to_num(oa), LNd, labels, il, ll)
    deg, dpg = oracle.accumulate_grads(E, P, oeg, opg, olng, LNd, il, ll)
    assert_close(costs, oc, what="costs, shared LN")
    # (the dense sums run over a thousand and more label positions here, in a dozen slices on
    # the device and one sequential fp32 sum in the oracle: a few entries in ten thousand that
    # are small differences of large terms land just outside; none is far off)
    for got, ref, name in ((eg, deg, "egrads"), (pg, dpg, "pgrads")):
        frac, worst = violations(got, ref)
        print("%s, shared LN: %.4f%% outside, max abs err %.3g" % (name, 100 * frac, worst))
        # (with V = 7 and 50 frames egrads has 700 entries: up to two of them may be such)
        assert frac <= max(1e-3, 2.5 / got.size)
        assert violations(got, ref, rtol=1e-3, atol=1e-4)[0] == 0.0
    # Against the oracle's OWN log-normaliser such a lattice (a thousand and more label
    # positions, a handful of symbols) moves with the last bit of LN far more than the benchmark
    # shapes do -- the reference's result does too when only the order of its LN sum changes --
    # so end to end only the costs and a cap on the fraction are held here; the entry-wise bar
    # is the shared-LN comparison above.
    want = oracle.loss_and_grads(E, P, labels, il, ll)
    assert_close(costs, want["costs"], rtol=1e-4, atol=1e-3, what="costs")
    sep, sep8 = (oracle.loss_and_grads(E, P, labels, il, ll, lse=k) for k in ("sep", "sep8"))
    for got, name in ((eg, "egrads"), (pg, "pgrads")):
        spread = max(violations(sep[name], want[name])[0], violations(sep8[name], sep[name])[0])
        frac, worst = violations(got, want[name])
        print("%s: %.4f%% outside end to end (the reference's own spread between orders of its "
              "LN sum: %.4f%%), max abs err %.3g" % (name, 100 * frac, 100 * spread, worst))
        if V >= 64:  # (below that the eight partial sums of the second order hold one term each)
            assert frac <= max(3 * spread, 4e-3)
    import torch
    from transducer_amd import capi
    from util import ptr
    out = torch.full((2, U - 1), -1, dtype=torch.int32, device="cuda:0")
    capi.call("rnnt_hip_viterbi_decode", ptr(c.E), ptr(c.P), ptr(c.il), ptr(c.ll), ptr(out),
              2, T, U, V, 0, None)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), oracle.viterbi(E, P, LNd, il, ll))


# ------------------------------------------------------------------ log-normaliser
@pytest.mark.parametrize("B,T,U,V,sigma", [(2, 70, 9, 31, 1.0), (1, 200, 101, 1000, 2.0),
                                           (3, 129, 130, 257, 1.0), (1, 64, 17, 4099, 3.0),
                                           (1, 64, 17, 4100, 3.0), (2, 150, 40, 10000, 1.0),
                                           (70, 500, 9, 33, 1.0), (45, 300, 130, 24, 1.0)])
def test_log_norms_against_fp64(B, T, U, V, sigma):
    # (the last two give at least 256 tiles of 128 frames and so take the kernel with tiles of
    # that height; the smaller grids take tiles of 64 frames)
    cfg = small_config(B, T, U - 1, V, sigma=sigma, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=V))
    c = DeviceCase(E, P, labels, il, ll)
    truth = oracle.log_norms_truth(E, P)
    got = gpu_log_norms(c, with_lengths=False)
    # Bar: a few ulp of LN (|LN| ~ 10-20), and never worse than the reference's own two fp32
    # forms (test.h naive sum, torch_binding separable sum), whose error grows when a handful
    # of terms dominate a long sum (sigma=3 case).
    floor = max(np.abs(oracle.log_norms_naive(E, P) - truth).max(),
                np.abs(oracle.log_norms_sep(E, P) - truth).max())
    tol = max(4e-6, 1.25 * floor)
    assert np.abs(got - truth).max() < tol
    got = gpu_log_norms(c, with_lengths=True)
    masked = oracle.log_norms_truth(E, P, il, ll)
    assert np.abs(got - masked).max() < tol
    for b in range(B):
        assert not got[b, il[b]:].any() and not got[b, :, ll[b] + 1:].any()


def test_log_norms_reference_moves_late_in_the_row():
    """Large scores far from the start of a row, rows that start with -inf, a row whose largest
    value sits in the last column: the per-frame reference of the streaming kernel has to move
    (and rescale what it has summed) without losing accuracy."""
    rng = np.random.default_rng(1)
    V = 1200
    E = rng.standard_normal((1, 70, V)).astype(np.float32)
    P = rng.standard_normal((1, 9, V)).astype(np.float32)
    E[0, 0:20, 700] += 100.0          # one jump
    E[0, 20:40, 300] += 50.0          # two jumps
    E[0, 20:40, 900] += 120.0
    E[0, 40:50, :64] = -np.inf        # first slabs hold nothing
    E[0, 50:60, V - 1] += 300.0       # last column
    E[0, 60:70, 100:1100] -= 80.0     # large early, tiny later: no jump
    c = DeviceCase(E, P, np.zeros((1, 8), np.int32), np.array([70], np.int32),
                   np.array([8], np.int32))
    got = gpu_log_norms(c, with_lengths=False)
    truth = oracle.log_norms_truth(E, P)
    assert np.isfinite(got).all()
    assert np.abs(got - truth).max() < 4e-6 * max(1.0, np.abs(truth).max())


@pytest.mark.parametrize("off_e,off_p", [(300.0, 0.0), (-300.0, 150.0), (120.0, -400.0)])
@pytest.mark.parametrize("V", [200, 700])
def test_gradients_of_scores_far_from_zero(off_e, off_p, V):
    """Scores with a large common offset (un-normalised logits).  The gradient kernels subtract a
    per-frame reference that they have multiplied by log2(e) beforehand; the rounding of that
    product grows with the reference's size (6e-6 relative at 100, past the tolerance from about
    1700) and is taken out again through the W planes.  Costs and both gradients against the
    oracle on the device's log_norms, every entry inside rel 1e-4 / abs 1e-5; the worst entry is
    printed in units of that tolerance."""
    cfg = small_config(2, 90, 20, V, ragged=True)
    E, P, labels, il, ll = (a.copy() for a in unpack(make_inputs(cfg, seed=int(abs(off_e)) + V)))
    E += np.float32(off_e)
    P += np.float32(off_p)
    c = DeviceCase(E, P, labels, il, ll)
    costs, eg, pg = gpu_loss(c)
    LN = gpu_log_norms(c)
    oc, oa = oracle.forward(E, P, LN, labels, il, ll)
    oeg, opg, olng = oracle.backward(E, P, np.nan_to_num(oa), LN, labels, il, ll)
    deg, dpg = oracle.accumulate_grads(E, P, oeg, opg, olng, LN, il, ll)
    assert_close(costs, oc, what="costs")
    for got, ref, name in ((eg, deg, "egrads"), (pg, dpg, "pgrads")):
        ratio = np.abs(got.astype(np.float64) - ref) / (1e-5 + 1e-4 * np.abs(ref))
        print("offsets %+g / %+g, V=%d: %s worst entry at %.3f of the tolerance"
              % (off_e, off_p, V, name, ratio.max()))
        assert_close(got, ref, what=name)


def test_log_norms_wide_dynamic_range():
    # maxima of the two operands at different v: the separable shift must not lose the sum
    rng = np.random.default_rng(0)
    E = rng.standard_normal((1, 40, 500)).astype(np.float32)
    P = rng.standard_normal((1, 6, 500)).astype(np.float32)
    E[0, :, 7] += 25.0
    P[0, :, 300] += 30.0
    c = DeviceCase(E, P, np.zeros((1, 5), np.int32), np.array([40], np.int32),
                   np.array([5], np.int32))
    got = gpu_log_norms(c, with_lengths=False)
    truth = oracle.log_norms_truth(E, P)
    assert np.abs(got - truth).max() < 1e-5


# ------------------------------------------------------------------ dense gradient kernels
# (U counts the rows of predictions; 113, 224, 225 sit on the edges of the 112-position slices
# the egrads kernel contracts per launch)
# (V = 16 mod 32, where every other row starts half a cache line in: one frame, an odd and an even
# number of frames, rows past a tile)
@pytest.mark.parametrize("B,T,U,V", [(2, 50, 11, 32), (2, 130, 101, 333), (1, 300, 140, 64),
                                     (2, 40, 113, 128), (2, 36, 224, 516), (3, 36, 225, 64),
                                     (2, 20, 470, 40), (3, 1, 5, 16), (2, 2, 3, 48),
                                     (2, 65, 20, 528), (1, 127, 101, 1040), (2, 64, 9, 16),
                                     (2, 130, 120, 80)])
def test_dense_grads_against_oracle(B, T, U, V):
    cfg = small_config(B, T, U - 1, V, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=T))
    LN = oracle.log_norms_naive(E, P, il, ll)
    _, alphas = oracle.forward(E, P, LN, labels, il, ll)
    eg, pg, lng = oracle.backward(E, P, np.nan_to_num(alphas), LN, labels, il, ll)
    deltas = np.linspace(0.5, 1.5, B).astype(np.float32)
    want_e, want_p = oracle.accumulate_grads(E.astype(np.float64), P.astype(np.float64), eg, pg,
                                             lng, LN, il, ll, precision="f64")
    want_e *= deltas[:, None, None]
    want_p *= deltas[:, None, None]
    got_e, got_p = gpu_dense_grads(DeviceCase(E, P, labels, il, ll), eg, pg, lng, LN, deltas)
    assert_close(got_e, want_e, what="egrads")
    assert_close(got_p, want_p, what="pgrads")
    for b in range(B):
        assert not got_e[b, il[b]:].any() and not got_p[b, ll[b] + 1:].any()


# ------------------------------------------------------------------ end to end
@pytest.mark.parametrize("cfg,seed", [("cfg1", 0), ("cfg1", 1)])
def test_whole_loss_cfg1(cfg, seed):
    E, P, labels, il, ll = unpack(make_inputs(CONFIGS[cfg], seed=seed))
    want = oracle.loss_and_grads(E, P, labels, il, ll)
    costs, eg, pg = gpu_loss(DeviceCase(E, P, labels, il, ll))
    assert_close(costs, want["costs"], what="costs")
    assert_close(eg, want["egrads"], what="egrads")
    assert_close(pg, want["pgrads"], what="pgrads")
    if seed == 0:  # same inputs as the fixture the reference's compiled sources produced
        f = CASES["cfg1"]
        assert_close(costs, f["costs"], what="costs vs reference fixture")
        assert_close(eg, f["egrads"], what="egrads vs reference fixture")
        assert_close(pg, f["pgrads"], what="pgrads vs reference fixture")


@pytest.mark.parametrize("T,U,V", [(60, 150, 36), (60, 150, 37), (40, 260, 16), (33, 113, 520),
                                   (40, 111, 520), (40, 112, 520), (36, 223, 516), (36, 224, 1028),
                                   (20, 500, 64), (33, 113, 528), (70, 100, 528)])
def test_whole_loss_with_a_label_axis_longer_than_one_slice(T, U, V):
    """egrads contracts 112 label positions per launch; a longer axis goes slice by slice, the
    later slices adding to what is in egrads and only the last one applying the upstream factors
    (so U + 1 = 112, 113, 224, 225 sit on the slice edges).  With V >= 512 the blank/label terms
    ride in the first slice's write-out, below that they are scattered; odd V also takes the
    log-normaliser's unaligned row loads.  Same entry points, same bar."""
    cfg = small_config(2, T, U, V, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=T + U + V))
    deltas = np.array([0.5, 3.0], np.float32)
    want = oracle.loss_and_grads(E, P, labels, il, ll, lse="naive", deltas=deltas)
    other = oracle.loss_and_grads(E, P, labels, il, ll, lse="sep", deltas=deltas)
    costs, eg, pg = gpu_loss(DeviceCase(E, P, labels, il, ll), deltas=deltas)
    assert_close(costs, want["costs"], what="costs")
    # a lattice this long along the label axis moves by more than the tolerance when LN moves in
    # its last bits: the bar is the oracle's own spread between its two summation orders of LN
    for got, name in ((eg, "egrads"), (pg, "pgrads")):
        floor, _ = violations(other[name], want[name])
        frac, worst = violations(got, want[name])
        print("%s: %.4f%% outside (oracle's own two LN orders: %.4f%%), max abs err %.3g"
              % (name, 100 * frac, 100 * floor, worst))
        assert frac <= max(2 * floor, 1e-3)
        # and nothing is far off: the reference's own CPU/GPU bar (test_cuda.cu:371-373)
        assert violations(got, want[name], rtol=1e-3, atol=1e-4)[0] == 0.0
    for b in range(2):
        assert not eg[b, il[b]:].any() and not pg[b, ll[b] + 1:].any()


def test_whole_loss_handles_empty_utterance_and_empty_label():
    cfg = small_config(4, 20, 6, 12, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=2))
    il, ll = il.copy(), ll.copy()
    il[1] = 0
    ll[2] = 0
    want = oracle.loss_and_grads(E, P, labels, il, ll)
    costs, eg, pg = gpu_loss(DeviceCase(E, P, labels, il, ll))
    assert np.isposinf(costs[1])
    fin = np.isfinite(want["costs"])
    assert_close(costs[fin], want["costs"][fin], what="costs")
    assert_close(eg, want["egrads"], what="egrads")
    assert_close(pg, want["pgrads"], what="pgrads")
    assert not eg[1].any() and not pg[1].any()


@pytest.mark.parametrize("V", [40, 600])
def test_labels_outside_the_vocabulary_act_as_the_nearest_valid_index(V):
    """The reference indexes its score rows with whatever the label array holds
    (transducer_cpu.cpp:63-66), which reads and writes past the row for a value outside [0, V).
    Every kernel here reads labels through one clamping function, so such a label means column
    0 or V-1 everywhere: same bits as the clamped labels, in the whole loss (scattered terms
    below 512 columns, folded ones from there on) and in the three boundary functions."""
    cfg = small_config(3, 70, 20, V, ragged=True)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=V))
    il[:] = 70
    ll[:] = 20
    bad = labels.copy()
    bad[0, 3], bad[0, 7], bad[1, 0], bad[2, 19] = -5, V, V + 1000, -(1 << 30)
    good = np.clip(bad, 0, V - 1)
    for got, want in zip(gpu_loss(DeviceCase(E, P, bad, il, ll)),
                         gpu_loss(DeviceCase(E, P, good, il, ll))):
        assert np.array_equal(got, want)
    LN = oracle.log_norms_naive(E, P, il, ll)
    cb, cg = DeviceCase(E, P, bad, il, ll), DeviceCase(E, P, good, il, ll)
    (costs_b, alphas_b), (costs_g, alphas_g) = gpu_forward(cb, LN), gpu_forward(cg, LN)
    assert np.array_equal(costs_b, costs_g) and np.array_equal(alphas_b, alphas_g)
    for got, want in zip(gpu_backward(cb, alphas_g, LN), gpu_backward(cg, alphas_g, LN)):
        assert np.array_equal(got, want)
    want = oracle.loss_and_grads(E, P, good, il, ll)
    assert_close(costs_g, want["costs"], what="costs")


def test_whole_loss_at_T2000_violation_fraction():
    """End to end at the real lattice length.  The two sides compute LN with different summation
    orders, and the reference's gradients are sensitive to the last bits of LN (its own fp32
    result moves by more than the tolerance when LN moves by a few ulp); so the bar here is a
    bounded violation fraction next to the oracle's own floor between two LN orders."""
    E, P, labels, il, ll = long_case(2, 100, seed=5)
    a = oracle.loss_and_grads(E, P, labels, il, ll, lse="naive")
    b = oracle.loss_and_grads(E, P, labels, il, ll, lse="sep")
    floor_e, _ = violations(b["egrads"], a["egrads"])
    floor_p, _ = violations(b["pgrads"], a["pgrads"])
    costs, eg, pg = gpu_loss(DeviceCase(E, P, labels, il, ll))
    assert_close(costs, a["costs"], rtol=1e-4, atol=1e-3, what="costs")
    ve, worst_e = violations(eg, a["egrads"])
    vp, worst_p = violations(pg, a["pgrads"])
    print("violations egrads %.4f%% (oracle floor %.4f%%), pgrads %.4f%% (floor %.4f%%); "
          "max abs err %.3g / %.3g" % (100 * ve, 100 * floor_e, 100 * vp, 100 * floor_p,
                                       worst_e, worst_p))
    # (measured: 0.0003 % / 0.416 % with floors of 0.505 % / 1.267 % on these inputs)
    assert ve <= max(2 * floor_e, 1e-3) and vp <= max(2 * floor_p, 1e-3)
    # fp64 truth: the device result must not be further from it than the reference's fp32 is
    t = oracle.loss_and_grads(E, P, labels, il, ll, precision="f64")
    err_dev = np.abs(eg - t["egrads"]).max()
    err_ref = np.abs(a["egrads"] - t["egrads"]).max()
    assert err_dev < 4 * err_ref + 1e-5


def test_pgrads_split_over_frames_gives_the_bits_of_the_unsplit_walk():
    """With a small vocabulary and a small batch several workgroups share a tile's frames
    (chunks of 8 slabs, summed in chunk order); the additions are the ones the unsplit walk
    performs, so one utterance alone (split) and the same utterance repeated 130 times (too
    many tiles to split) must agree bit for bit, and so must a batch of 3."""
    cfg = small_config(1, 600, 20, 100, ragged=False)
    E, P, labels, il, ll = unpack(make_inputs(cfg, seed=4))
    il = np.array([571], np.int32)   # not a multiple of a chunk, nor of a slab
    ll = np.array([17], np.int32)
    one = gpu_loss(DeviceCase(E, P, labels, il, ll))
    for copies in (3, 130):
        rep = lambda a: np.repeat(a, copies, axis=0)
        many = gpu_loss(DeviceCase(rep(E), rep(P), rep(labels), rep(il), rep(ll)))
        for got, want in zip(many, one):
            assert np.array_equal(got[0], want[0]) and np.array_equal(got[-1], want[0])
    want = oracle.loss_and_grads(E, P, labels, il, ll)
    assert_close(one[0], want["costs"], what="costs")
    assert_close(one[2], want["pgrads"], what="pgrads")
