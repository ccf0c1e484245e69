"""Writes tests/golden/ref_cases.npz: inputs and outputs of the REFERENCE's own CPU sources
(compiled as oracle/_ref/libtransducer_ref.so by oracle/Makefile) for seeded cases -- the
CPU-runnable benchmark configuration, a ragged grid in the spirit of the reference's CPU-vs-GPU
stress test (transducer/test_cuda.cu:323-378, including empty utterances and empty labels),
and viterbi inputs with exact score ties.  Run in the build container, where /root/reference
exists; the .npz travels, the reference does not.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
from transducer_amd.synthetic import CONFIGS, make_inputs  # noqa: E402


def run_reference(E, P, labels, il, ll):
    LN = oracle.ref_log_norms(E, P, il, ll)
    costs, alphas = oracle.ref_forward(E, P, LN, labels, il, ll)
    eg, pg, lng = oracle.ref_backward(E, P, np.nan_to_num(alphas), LN, labels, il, ll)
    eg_full, pg_full = oracle.ref_accumulate_grads(E, P, eg, pg, lng, LN, il, ll)
    out = dict(log_norms=LN, costs=costs, alphas=alphas, egrads_sparse=eg, pgrads_sparse=pg,
               lngrads=lng, egrads=eg_full, pgrads=pg_full)
    if P.shape[1] > 1 and E.shape[1] > 0:
        out["viterbi"] = oracle.ref_viterbi(E, P, LN, il, ll)
    return out


def stress_case(rng, B, T, U, V):
    """Uniform[0,1) scores, input lengths in [0,T], label lengths in [0,U-1], labels in [1,V)."""
    E = rng.random((B, T, V), dtype=np.float32)
    P = rng.random((B, U, V), dtype=np.float32)
    il = rng.integers(0, T + 1, B).astype(np.int32)
    ll = rng.integers(0, U, B).astype(np.int32)
    labels = rng.integers(1, V, (B, max(U - 1, 0))).astype(np.int32)
    return E, P, labels, il, ll


def main():
    assert oracle.have_ref(), "build oracle/_ref first: make -C oracle ref"
    cases = {}

    d = make_inputs(CONFIGS["cfg1"], seed=0)
    cases["cfg1"] = (d["emissions"], d["predictions"], d["labels"], d["input_lengths"],
                     d["label_lengths"])

    rng = np.random.Generator(np.random.Philox(key=7))
    for B in (1, 5):
        for T in (1, 10, 40):
            for U in (1, 10, 33):
                for V in (8, 20, 33):
                    cases["stress_B%d_T%d_U%d_V%d" % (B, T, U, V)] = stress_case(rng, B, T, U, V)

    # exact ties: scores on a coarse grid, so distinct labels and distinct paths score alike
    for k, (B, T, U, V) in enumerate([(3, 12, 5, 6), (2, 30, 9, 4), (4, 7, 7, 16)]):
        E = (rng.integers(0, 3, (B, T, V)) * 0.5).astype(np.float32)
        P = (rng.integers(0, 3, (B, U, V)) * 0.5).astype(np.float32)
        il = rng.integers(max(1, T // 2), T + 1, B).astype(np.int32)
        ll = rng.integers(1, U, B).astype(np.int32)
        il[0], ll[0] = T, U - 1
        labels = rng.integers(1, V, (B, U - 1)).astype(np.int32)
        cases["ties_%d" % k] = (E, P, labels, il, ll)

    blob = {}
    for name, (E, P, labels, il, ll) in cases.items():
        out = run_reference(E, P, labels, il, ll)
        blob[name + "/emissions"] = E
        blob[name + "/predictions"] = P
        blob[name + "/labels"] = labels
        blob[name + "/input_lengths"] = il
        blob[name + "/label_lengths"] = ll
        for k, v in out.items():
            blob[name + "/" + k] = v
    path = os.path.join(HERE, "ref_cases.npz")
    np.savez_compressed(path, **blob)
    print("wrote", path, "%d cases, %.1f KiB" % (len(cases), os.path.getsize(path) / 1024))


if __name__ == "__main__":
    main()
