"""Seeded random shapes around the kernels' tile edges (32, 64, 128 frames and label positions;
vocabularies off and on the 4- and 8-element vector widths, below and above the 512 columns
where the sparse terms are folded into the dense kernels), ragged and empty utterances, any
blank index: the whole loss, the three functions of the reference's C++ interface
(transducer.h:3-49) and the best path against the oracle.

A vocabulary of one symbol with labels to emit is left out: the reference's back-trace then
walks off the front of its table (transducer_cpu.cpp:210-219 with paths[0,u] == blank), so no
answer is defined there."""
import numpy as np
import pytest

from util import (DeviceCase, assert_close, assert_same_bits, gpu_backward, gpu_forward,
                  gpu_log_norms, gpu_loss, gpu_viterbi, violations)

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
import oracle  # noqa: E402

# fraction of gradient entries that may sit outside rel 1e-4 / abs 1e-5 end to end, each side
# with its own log-normaliser (largest measured over these seeds: 0.112 % of egrads, 0.082 % of
# pgrads, both on one lattice of 131 x 129 cells; 34 of the 40 cases have none)
END_TO_END_BAR = 0.004

EDGES = [1, 2, 3, 31, 32, 33, 63, 64, 65, 96, 97, 127, 128, 129]
VOCABS = [1, 2, 3, 4, 5, 7, 8, 9, 31, 32, 33, 100, 127, 128, 129, 255, 256, 260, 511, 512, 513,
          516, 1000, 1024, 1028]


def draw(seed):
    rng = np.random.default_rng(seed)
    B = int(rng.integers(1, 6))
    T = int(rng.choice(EDGES)) if rng.random() < 0.5 else int(rng.integers(1, 400))
    U = int(rng.choice(EDGES)) if rng.random() < 0.5 else int(rng.integers(1, 150))
    V = int(rng.choice(VOCABS)) if rng.random() < 0.6 else int(rng.integers(1, 2500))
    while B * T * U * V > 3e7:  # keep the oracle at a fraction of a second
        if V > 64 and rng.random() < 0.5:
            V = max(1, V // 2)
        elif T > 8:
            T = max(1, T // 2)
        else:
            U = max(1, U // 2)
    if V == 1 and U > 1:
        V = 2
    blank = int(rng.integers(0, V)) if rng.random() < 0.5 else 0
    sigma = float(rng.choice([0.5, 1.0, 2.0, 4.0]))
    E = (rng.standard_normal((B, T, V)) * sigma).astype(np.float32)
    P = (rng.standard_normal((B, U, V)) * sigma).astype(np.float32)
    labels = rng.integers(0, V, (B, max(U - 1, 0))).astype(np.int32)
    if rng.random() < 0.8 and V > 1:  # mostly off the blank, as real transcripts are
        labels = np.where(labels == blank, (labels + 1) % V, labels).astype(np.int32)
    if rng.random() < 0.3:
        il, ll = np.full(B, T, np.int32), np.full(B, U - 1, np.int32)
    else:
        il = rng.integers(0 if rng.random() < 0.3 else 1, T + 1, B).astype(np.int32)
        ll = rng.integers(0, U, B).astype(np.int32)
    return E, P, labels, il, ll, blank


@pytest.mark.parametrize("seed", range(7000, 7040))
def test_random_shape_against_the_oracle(seed):
    E, P, labels, il, ll, blank = draw(seed)
    B, T, V = E.shape
    U = P.shape[1]
    print("B=%d T=%d U'=%d V=%d blank=%d input_lengths=%s label_lengths=%s"
          % (B, T, U, V, blank, il.tolist(), ll.tolist()), flush=True)
    c = DeviceCase(E, P, labels, il, ll)

    # whole loss end to end, each side with its own log-normaliser: costs to the tolerance (they
    # are O(T) sums: absolute 1e-3 as for the long configurations); gradients move with the last
    # bit of LN where the lattice is long, so a small fraction of entries may sit outside
    want = oracle.loss_and_grads(E, P, labels, il, ll, blank=blank)
    costs, eg, pg = gpu_loss(c, blank=blank)
    assert np.allclose(costs, want["costs"], rtol=1e-4, atol=1e-3, equal_nan=True)
    assert np.isfinite(eg).all() and np.isfinite(pg).all()
    live = np.isfinite(want["costs"])
    if live.any():
        fe = violations(eg[live], want["egrads"][live])[0]
        fp = violations(pg[live], want["pgrads"][live])[0]
        print("end to end: %.4f%% of egrads, %.4f%% of pgrads outside" % (100 * fe, 100 * fp))
        assert fe <= END_TO_END_BAR and fp <= END_TO_END_BAR
    for b in range(B):
        assert not eg[b, il[b]:].any() and not pg[b, ll[b] + 1:].any()

    # the same with ONE log-normaliser (the device's) on both sides: no entry outside
    LN = gpu_log_norms(c)
    oc, oa = oracle.forward(E, P, LN, labels, il, ll, blank=blank)
    oeg, opg, olng = oracle.backward(E, P, np.nan_to_num(oa), LN, labels, il, ll, blank=blank)
    deg, dpg = oracle.accumulate_grads(E, P, oeg, opg, olng, LN, il, ll)
    if live.any():
        assert_close(costs[live], oc[live], what="costs, shared LN")
        assert_close(eg[live], deg[live], what="egrads, shared LN")
        assert_close(pg[live], dpg[live], what="pgrads, shared LN")

    # the C++ interface's three functions on that LN: the reference's bits in every alpha, every
    # dalpha and every blank / label term (same expf / log1pf, same order of operations)
    gc, ga = gpu_forward(c, LN, blank=blank)
    assert_same_bits(gc, oc, what="costs")
    assert_same_bits(ga, oa, what="alphas")
    geg, gpg, glng = gpu_backward(c, ga, LN, blank=blank)
    assert_same_bits(glng, olng, what="lngrads")
    assert_same_bits(geg, oeg, what="egrads (sparse)")
    assert_same_bits(gpg, opg, what="pgrads (sparse)")

    # best path: exact
    if U > 1:
        paths = gpu_viterbi(c, LN, blank=blank)
        wantp = oracle.viterbi(E, P, LN, il, ll, blank=blank)
        for b in range(B):
            if il[b] > 0:
                assert np.array_equal(paths[b, :ll[b]], wantp[b, :ll[b]])
        # and with the table of best labels built from candidate lists instead of every column
        from transducer_amd import capi
        capi.call("rnnt_hip_set_maxplus_mode", 2)
        try:
            paths_lists = gpu_viterbi(c, LN, blank=blank)
        finally:
            capi.call("rnnt_hip_set_maxplus_mode", 0)
        assert np.array_equal(paths_lists, paths)
