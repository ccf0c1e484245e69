"""The backward pass's one-kernel form of the two dense gradients (each row of the emissions
read once) against the two separate contractions and against the oracle.

The fused walk performs the additions of the separate kernels: egrads must come out with the
same bits; pgrads feeds the frames of a slab to the matrix instruction in another order (the
order the egrads block holds them in), which the instruction's internal sum may round
differently, so it is held to a few units in the last place of the separate result and, like
everything else, to the oracle at rel 1e-4 / abs 1e-5."""
import numpy as np
import pytest

import oracle
from transducer_amd import capi
from transducer_amd.synthetic import make_inputs, small_config
from util import DeviceCase, assert_close, assert_same_bits, gpu_log_norms, gpu_loss, violations

# Switched off with the code path: at the headline shape the fused kernel left NaN entries in
# pgrads on one input and made an illegal memory access on another (these small shapes passed),
# and the cause has not been found.  rnnt_hip_set_fused_grads refuses every mode but 0; the tests
# stay for the day the kernel is switched on again.
pytestmark = [pytest.mark.gpu,
              pytest.mark.skip(reason="fused gradient kernel switched off: unexplained GPU "
                                      "fault at the headline shape")]

KEYS = ("emissions", "predictions", "labels", "input_lengths", "label_lengths")


def loss_in_mode(c, mode, deltas=None, blank=0):
    before = capi.load().rnnt_hip_set_fused_grads(mode)
    try:
        return gpu_loss(c, deltas=deltas, blank=blank)
    finally:
        capi.load().rnnt_hip_set_fused_grads(before)


def oracle_on_device_log_norms(E, P, labels, il, ll, c, blank=0):
    LN = gpu_log_norms(c)
    costs, alphas = oracle.forward(E, P, LN, labels, il, ll, blank=blank)
    eg, pg, lng = oracle.backward(E, P, np.nan_to_num(alphas), LN, labels, il, ll, blank=blank)
    eg, pg = oracle.accumulate_grads(E, P, eg, pg, lng, LN, il, ll)
    return costs, eg, pg


# (B, T, U = rows of predictions, V): label positions either side of the 32-row blocks and 16-row
# steps the kernel is instantiated for, frames either side of a slab of 32 and of the 8-slab
# flush, vocabularies off the 32-column blocks and the 128-column tiles
SHAPES = [(2, 70, 2, 40), (2, 70, 3, 600), (3, 33, 17, 129), (2, 300, 33, 200), (3, 257, 64, 96),
          (2, 64, 65, 513), (2, 530, 81, 160), (2, 100, 97, 31), (2, 288, 101, 1000),
          (1, 1000, 112, 260)]


@pytest.mark.parametrize("shape", SHAPES)
def test_fused_walk_equals_the_two_contractions_and_the_oracle(shape):
    B, T, U, V = shape
    E, P, labels, il, ll = (make_inputs(small_config(B, T, U - 1, V, ragged=True),
                                        seed=B + T + U + V)[k] for k in KEYS)
    il[0], ll[0] = T, U - 1
    if B > 2:
        il[1] = 0  # an utterance without frames
    deltas = np.linspace(0.5, 2.0, B).astype(np.float32)
    c = DeviceCase(E, P, labels, il, ll)
    costs0, eg0, pg0 = loss_in_mode(c, 0, deltas)
    costs2, eg2, pg2 = loss_in_mode(c, 2, deltas)
    assert_same_bits(costs2, costs0, what="costs")
    if V >= 512 and len(np.unique(labels[0])) == labels.shape[1]:
        assert_same_bits(eg2, eg0, what="egrads, fused against separate")
    else:
        # (a label that repeats inside an utterance puts two terms on one entry, which the two
        # forms add in a different order)
        # (below 512 columns the separate path adds the blank / label terms after the dense
        # kernel, delta * dense + delta * term instead of delta * (dense + term): those entries
        # round differently)
        assert violations(eg2, eg0, rtol=1e-6, atol=1e-6)[0] == 0.0
        differ = eg2 != eg0
        assert differ.sum() <= B * T * U, "only blank / label entries may differ"
    assert np.array_equal(pg2 == 0, pg0 == 0), "pgrads: exact zeros in the same places"
    # (an entry that is the small sum of a dense part and a blank / label total carries the
    # rounding of the dense part: the scale is the row's largest entry)
    err = np.abs(pg2.astype(np.float64) - pg0)
    scale = np.abs(pg0).max(axis=-1, keepdims=True)
    assert (err <= 4 * np.spacing(np.abs(pg0)) + 1e-5 * scale).all(), \
        "pgrads: fused %g from separate at worst" % err.max()
    want = oracle_on_device_log_norms(E, P, labels, il, ll, c)
    sc = deltas[:, None, None]
    assert_close(eg2, sc * want[1], what="egrads against the oracle (shared LN)")
    assert_close(pg2, sc * want[2], what="pgrads against the oracle (shared LN)")


def test_fused_walk_nonzero_blank_and_repeated_labels():
    B, T, U, V = 3, 150, 40, 300
    E, P, labels, il, ll = (make_inputs(small_config(B, T, U - 1, V, ragged=True), seed=77)[k]
                            for k in KEYS)
    labels = labels.copy()
    labels[:, ::3] = 5       # many labels in one wavefront's 32 columns
    labels[:, 1::3] = 7      # ... and the blank itself as a label
    blank = 7
    c = DeviceCase(E, P, labels, il, ll)
    costs0, eg0, pg0 = loss_in_mode(c, 0, blank=blank)
    costs2, eg2, pg2 = loss_in_mode(c, 2, blank=blank)
    assert violations(eg2, eg0, rtol=1e-6, atol=1e-6)[0] == 0.0
    assert violations(pg2, pg0, rtol=1e-5, atol=1e-5)[0] == 0.0
    want = oracle_on_device_log_norms(E, P, labels, il, ll, c, blank=blank)
    assert_close(eg2, want[1], what="egrads against the oracle (shared LN)")
    assert_close(pg2, want[2], what="pgrads against the oracle (shared LN)")


def test_default_mode_takes_the_fused_walk_only_where_it_pays():
    # a small grid keeps the two contractions by default: same bits as mode 0
    E, P, labels, il, ll = (make_inputs(small_config(2, 90, 20, 600, ragged=True), seed=3)[k]
                            for k in KEYS)
    c = DeviceCase(E, P, labels, il, ll)
    _, eg0, pg0 = loss_in_mode(c, 0)
    _, eg1, pg1 = loss_in_mode(c, 1)
    assert_same_bits(eg1, eg0)
    assert_same_bits(pg1, pg0)
