"""The two ways of building the best-path table give the same table.

best[t,u] = max over v != blank of E[t,v] + P[u,v] with the lowest index reaching it
(transducer/transducer_cpu.cpp:158-171) is built either by looking at every column
(`rnnt_hip_set_maxplus_mode(1)`) or from short candidate lists with an exactness test per cell
(mode 2: lists wherever the shape allows; mode 0 picks by vocabulary size).  Both must return
the reference's table bit for bit, ties included: checked here against a brute-force numpy
statement of the reference's scan, on data chosen to break a wrong list (exact ties, quantised
scores, constant rows, -inf and +inf entries, a winner that only the other side's list holds,
lists that overflow), and end to end against the oracle's labels."""
import numpy as np
import pytest

import oracle
from transducer_amd import capi
from util import dev, ptr

pytestmark = pytest.mark.gpu


def brute(E, P, il, ll, blank):
    """getMax of transducer_cpu.cpp:158-171 for every cell (NaN sums never win, as `>` has it)."""
    B, T, V = E.shape
    U = P.shape[1]
    best = np.full((B, T, U), -np.inf, np.float32)
    arg = np.full((B, T, U), -1, np.int32)
    for b in range(B):
        Tb, Ub = min(int(il[b]), T), min(int(ll[b]) + 1, U)
        for t in range(Tb):
            with np.errstate(invalid="ignore"):
                s = E[b, t][None, :] + P[b, :Ub]
            s[:, blank] = -np.inf
            s = np.where(np.isnan(s), -np.inf, s)
            top = s.max(axis=1)
            first = (s == top[:, None]).argmax(axis=1)
            best[b, t, :Ub] = top
            arg[b, t, :Ub] = np.where(top > -np.inf, first, 0)
    return best, arg


def table(E, P, il, ll, blank, mode):
    import torch
    B, T, V = E.shape
    U = P.shape[1]
    dE, dP, dil, dll = dev(E), dev(P), dev(il), dev(ll)
    best = torch.full((B, T, U), float("nan"), device=dE.device)
    arg = torch.full((B, T, U), -7, dtype=torch.int32, device=dE.device)
    capi.call("rnnt_hip_set_maxplus_mode", mode)
    try:
        capi.call("rnnt_hip_maxplus_table", ptr(dE), ptr(dP), ptr(dil), ptr(dll), ptr(best),
                  ptr(arg), B, T, U, V, blank, None)
        torch.cuda.synchronize()
    finally:
        capi.call("rnnt_hip_set_maxplus_mode", 0)
    return best.cpu().numpy(), arg.cpu().numpy()


def check(E, P, il, ll, blank=0, modes=(1, 2)):
    E, P = np.ascontiguousarray(E, np.float32), np.ascontiguousarray(P, np.float32)
    il, ll = np.asarray(il, np.int32), np.asarray(ll, np.int32)
    want_best, want_arg = brute(E, P, il, ll, blank)
    for mode in modes:
        best, arg = table(E, P, il, ll, blank, mode)
        assert np.array_equal(arg, want_arg), "mode %d: %d indices differ" % (
            mode, int((arg != want_arg).sum()))
        assert np.array_equal(best.view(np.uint32), want_best.view(np.uint32)), "mode %d" % mode


def lengths(rng, B, T, U):
    il = rng.integers(max(1, T // 2), T + 1, B).astype(np.int32)
    ll = rng.integers(0, U, B).astype(np.int32)
    il[0], ll[0] = T, U - 1
    return il, ll


SHAPES = [(2, 9, 5, 12, 0), (1, 3, 2, 5, 4), (2, 17, 7, 100, 3), (1, 40, 70, 130, 0),
          (2, 33, 101, 1000, 999), (1, 20, 130, 515, 7), (2, 21, 9, 4096, 0),
          (1, 35, 66, 10000, 0), (1, 19, 4, 10001, 10000), (1, 5, 3, 4, 1),
          (1, 6, 3, 16000, 0),   # a row past 64 KB of LDS
          (1, 3, 2, 17408, 5),   # the longest row the list path takes
          (1, 3, 2, 17409, 5),   # one column more: every column (the mode setting cannot force lists)
          (2, 9, 300, 700, 3),   # three blocks of 128 label positions
          (8, 40, 9, 300, 2),    # utterance counts that are multiples of eight: workgroups are dealt
          (16, 35, 70, 260, 0)]  # out so that each of the eight dies works through utterances of its own


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "B%d_T%d_U%d_V%d_blank%d" % s)
def test_gaussian_scores(shape):
    B, T, U, V, blank = shape
    rng = np.random.default_rng(sum(shape))
    il, ll = lengths(rng, B, T, U)
    check(rng.standard_normal((B, T, V)), rng.standard_normal((B, U, V)), il, ll, blank)


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_lengths_and_distributions(seed):
    rng = np.random.default_rng(9000 + seed)
    B = int(rng.integers(1, 5))
    T = int(rng.choice([1, 2, 15, 16, 17, 33, 129])) if rng.random() < 0.5 else int(rng.integers(1, 200))
    U = int(rng.choice([1, 2, 63, 64, 65, 128, 129])) if rng.random() < 0.5 else int(rng.integers(1, 140))
    V = int(rng.choice([4, 5, 255, 256, 257, 1024, 1027, 4096, 8192, 12001])) if rng.random() < 0.6 \
        else int(rng.integers(4, 3000))
    while B * T * U * V > 2e7:
        if T > 4: T //= 2
        elif U > 4: U //= 2
        else: V //= 2
    blank = int(rng.integers(0, V))
    kind = int(rng.integers(0, 4))
    if kind == 0:
        E, P = rng.standard_normal((B, T, V)) * 3, rng.standard_normal((B, U, V))
    elif kind == 1:
        E, P = rng.random((B, T, V)), rng.random((B, U, V))
    elif kind == 2:  # few distinct values
        E, P = rng.integers(-2, 3, (B, T, V)) * 0.5, rng.integers(-2, 3, (B, U, V)) * 0.25
    else:  # values rounded to bfloat16 (many equal sums), some -inf
        E = rng.standard_normal((B, T, V)).astype(np.float32)
        P = rng.standard_normal((B, U, V)).astype(np.float32)
        E = (E.view(np.uint32) & 0xffff0000).view(np.float32).copy()
        P = (P.view(np.uint32) & 0xffff0000).view(np.float32).copy()
        E[rng.random(E.shape) < 0.01] = -np.inf
    il = rng.integers(0, T + 1, B).astype(np.int32)
    ll = rng.integers(0, U, B).astype(np.int32)
    if rng.random() < 0.5:
        il[0], ll[0] = T, U - 1
    print("B=%d T=%d U=%d V=%d blank=%d kind=%d il=%s ll=%s" % (B, T, U, V, blank, kind, il.tolist(),
                                                           ll.tolist()), flush=True)
    check(E, P, il, ll, blank, modes=(0, 1, 2))


@pytest.mark.parametrize("shape", [(2, 12, 6, 40, 0), (1, 30, 20, 2048, 5), (1, 16, 101, 10000, 0)],
                         ids=lambda s: "B%d_T%d_U%d_V%d_blank%d" % s)
def test_quantised_scores_tie_everywhere(shape):
    # a handful of distinct values: every cell's maximum is reached by many columns, and the
    # rows' own maxima are reached by a quarter of their columns (lists stay empty or overflow)
    B, T, U, V, blank = shape
    rng = np.random.default_rng(1 + sum(shape))
    il, ll = lengths(rng, B, T, U)
    E = rng.integers(0, 4, (B, T, V)).astype(np.float32)
    P = rng.integers(0, 3, (B, U, V)).astype(np.float32) * 0.5
    check(E, P, il, ll, blank)


def test_constant_and_degenerate_rows():
    rng = np.random.default_rng(5)
    B, T, U, V = 1, 12, 6, 3000
    E = rng.standard_normal((B, T, V)).astype(np.float32)
    P = rng.standard_normal((B, U, V)).astype(np.float32)
    E[0, 0] = 1.25                      # constant row
    E[0, 1] = -np.inf                   # nothing can win: index 0 stays (even though 0 is blank)
    E[0, 2] = -np.inf; E[0, 2, 1777] = 0.5   # one finite column
    E[0, 3, 5] = np.inf                 # +inf wins, lowest index of the infinite ones
    E[0, 3, 9] = np.inf
    E[0, 4, 100:200] = np.nan           # NaN never wins
    E[0, 5] = np.arange(V, dtype=np.float32)          # sorted rows: the list is one run of columns
    E[0, 6] = -np.arange(V, dtype=np.float32)
    P[0, 1] = 0.0                       # constant row of P
    P[0, 2] = -np.inf
    P[0, 3, 7] = np.inf                 # with E = -inf at 7 in row 2: a NaN sum
    P[0, 4] = np.arange(V, dtype=np.float32) * 0.001
    il, ll = np.array([T], np.int32), np.array([U - 1], np.int32)
    check(E, P, il, ll, 0)


def test_winner_held_by_one_side_only():
    # the maximum sits in a column where E is unremarkable and P is huge, and the other way round
    rng = np.random.default_rng(6)
    B, T, U, V = 1, 10, 8, 5000
    E = rng.standard_normal((B, T, V)).astype(np.float32)
    P = rng.standard_normal((B, U, V)).astype(np.float32)
    for u in range(U):
        P[0, u, 37 * u + 11] += 50.0
    for t in range(0, T, 2):
        E[0, t, 4000 - 13 * t] += 60.0
    il, ll = np.array([T], np.int32), np.array([U - 1], np.int32)
    check(E, P, il, ll, 3)


def test_exact_ties_between_the_two_lists():
    # two columns reach the same sum, one through a large E (only on the frame's list), one
    # through a large P (only on the label position's list): the lower index must win, whichever
    # list holds it (utterance 0: the label position's; utterance 1: the frame's)
    B, T, U, V = 2, 6, 5, 2500
    rng = np.random.default_rng(7)
    E = rng.integers(-3, 4, (B, T, V)).astype(np.float32) * 0.25
    P = rng.integers(-3, 4, (B, U, V)).astype(np.float32) * 0.25
    for t in range(T):
        for u in range(U):
            hi, lo = 2000 - 7 * t - u, 300 + 11 * t + u
            E[0, t, hi], P[0, u, hi] = 8.0, 1.0
            P[0, u, lo], E[0, t, lo] = 8.0, 1.0
            E[1, t, lo], P[1, u, lo] = 8.0, 1.0
            P[1, u, hi], E[1, t, hi] = 8.0, 1.0
    il, ll = np.array([T, T], np.int32), np.array([U - 1, U - 1], np.int32)
    want_best, want_arg = brute(E, P, il, ll, 0)
    assert (want_best == 9.0).all() and (want_arg < 400).all()
    check(E, P, il, ll, 0)


def test_overflowing_lists_fall_back():
    # many more columns above any sensible threshold than a list holds, in one half of the row
    rng = np.random.default_rng(8)
    B, T, U, V = 1, 8, 5, 4000
    E = rng.standard_normal((B, T, V)).astype(np.float32) * 0.01
    P = rng.standard_normal((B, U, V)).astype(np.float32) * 0.01
    E[0, :, 100:900] += 5.0 + rng.standard_normal((T, 800)).astype(np.float32)
    P[0, 1, 2500:3500] += 5.0 + rng.standard_normal(1000).astype(np.float32)
    il, ll = np.array([T], np.int32), np.array([U - 1], np.int32)
    check(E, P, il, ll, 0)


def test_many_failing_cells_in_a_tile_and_few():
    # utterance 0, quantised scores: the test fails for most cells and the all-columns kernel
    # redoes whole tiles.  Utterance 1: two quantised rows of P, so two label positions fail in
    # every frame: 256 cells in the first tile of frames (more than a tile's list of flagged
    # cells holds: redone as a tile), 6 in the second (redone cell by cell)
    rng = np.random.default_rng(9)
    B, T, U, V = 2, 140, 70, 2304
    E = rng.standard_normal((B, T, V)).astype(np.float32)
    P = rng.standard_normal((B, U, V)).astype(np.float32)
    E[0] = np.round(E[0] * 2) * 0.5
    P[0] = np.round(P[0] * 2) * 0.5
    P[1, 5:7] = np.round(P[1, 5:7] * 2) * 0.5
    il, ll = np.array([T, 131], np.int32), np.array([U - 1, U - 5], np.int32)
    check(E, P, il, ll, 0)


@pytest.mark.parametrize("U,V", [(70, 8192), (33, 8192), (101, 3000)])
@pytest.mark.parametrize("dist", ["normal", "uniform", "quantised"])
def test_default_mode_in_the_range_where_lists_are_tried(dist, U, V):
    # Shapes inside the range where the default mode starts on lists (3000 columns or more,
    # U x V of 250000 or more) and lets a sample of the cells (two utterances, one frame in
    # sixteen) decide whether to go on.  Uniform scores fail the bound too often and send the
    # call on to a second pair of longer lists, quantised ones fail with those too and send it
    # back to every column, normal ones pass at once; a third utterance is outside the sample
    # either way.
    rng = np.random.default_rng(21)
    B, T = 3, 130  # (the sample must hold a thousand cells to count: two utterances x 9 frames x U)
    assert capi.load().rnnt_hip_maxplus_tries_lists(B, T, U, V) == 1
    if dist == "normal":
        E, P = rng.standard_normal((B, T, V)), rng.standard_normal((B, U, V))
    elif dist == "uniform":
        E, P = rng.random((B, T, V)), rng.random((B, U, V))
    else:
        E, P = rng.integers(0, 5, (B, T, V)) * 0.5, rng.integers(0, 5, (B, U, V)) * 0.25
    il, ll = np.array([T, T - 5, T - 1], np.int32), np.array([U - 1, U - 3, U - 2], np.int32)
    check(E, P, il, ll, 0, modes=(0,))


@pytest.mark.parametrize("dist", ["normal", "uniform"])
def test_default_mode_when_the_sampled_utterances_are_empty_or_short(dist):
    # The sample takes utterances 0 and B/2.  With no frames (or a handful) in both, the sample
    # says nothing about the scores: the call then goes over every column instead of trusting
    # lists it has no evidence for.  Either way the table is the reference's.
    rng = np.random.default_rng(5)
    B, T, U, V = 4, 60, 70, 8192
    assert capi.load().rnnt_hip_maxplus_tries_lists(B, T, U, V) == 1
    E = rng.standard_normal((B, T, V)) if dist == "normal" else rng.random((B, T, V))
    P = rng.standard_normal((B, U, V)) if dist == "normal" else rng.random((B, U, V))
    for il in ([0, T, 0, T - 7], [3, T, 1, T]):
        check(E, P, np.array(il, np.int32), np.array([U - 1, U - 2, 5, U - 1], np.int32), 0,
              modes=(0,))


@pytest.mark.parametrize("shape", [(2, 60, 14, 2100), (2, 40, 80, 3200)],
                         ids=lambda s: "B%d_T%d_U%d_V%d" % s)
@pytest.mark.parametrize("mode", [0, 1, 2])
def test_decode_labels_against_oracle(mode, shape):
    # (the second shape is inside the range where the default mode starts on lists)
    import torch
    rng = np.random.default_rng(11)
    B, T, U, V = shape
    E = rng.standard_normal((B, T, V)).astype(np.float32)
    P = rng.standard_normal((B, U, V)).astype(np.float32)
    il, ll = np.array([T, T - 7], np.int32), np.array([U - 1, U - 4], np.int32)
    LN = oracle.log_norms_naive(E, P, il, ll)
    want = oracle.viterbi(E, P, LN, il, ll)
    dE, dP, dil, dll = dev(E), dev(P), dev(il), dev(ll)
    out = torch.full((B, U - 1), -1, dtype=torch.int32, device=dE.device)
    capi.call("rnnt_hip_set_maxplus_mode", mode)
    try:
        capi.call("rnnt_hip_viterbi_decode", ptr(dE), ptr(dP), ptr(dil), ptr(dll), ptr(out), B, T,
                  U, V, 0, None)
        torch.cuda.synchronize()
    finally:
        capi.call("rnnt_hip_set_maxplus_mode", 0)
    got = out.cpu().numpy()
    for b in range(B):
        assert np.array_equal(got[b, :ll[b]], want[b, :ll[b]])


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_16bit_decode_same_labels_in_both_modes(dtype):
    import torch
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float16
    rng = np.random.default_rng(12)
    B, T, U, V = 2, 50, 12, 4104
    E = torch.from_numpy(rng.standard_normal((B, T, V)).astype(np.float32)).to("cuda:0").to(tdt)
    P = torch.from_numpy(rng.standard_normal((B, U, V)).astype(np.float32)).to("cuda:0").to(tdt)
    il, ll = dev(np.array([T, T - 3], np.int32)), dev(np.array([U - 1, U - 2], np.int32))
    outs = []
    for mode in (1, 2):
        out = torch.full((B, U - 1), -1, dtype=torch.int32, device=E.device)
        capi.call("rnnt_hip_set_maxplus_mode", mode)
        try:
            capi.call("rnnt_hip_viterbi_decode_" + dtype, ptr(E), ptr(P), ptr(il), ptr(ll), ptr(out),
                      B, T, U, V, 0, None)
            torch.cuda.synchronize()
        finally:
            capi.call("rnnt_hip_set_maxplus_mode", 0)
        outs.append(out.cpu().numpy())
    assert np.array_equal(outs[0], outs[1])
    # and the table of the upcast scores, which is what both are built from
    check(E.float().cpu().numpy(), P.float().cpu().numpy(), il.cpu().numpy(), ll.cpu().numpy(), 0)


def test_mode_is_validated():
    with pytest.raises(Exception):
        capi.call("rnnt_hip_set_maxplus_mode", 3)
