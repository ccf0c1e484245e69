"""rnnt_hip_viterbi_decode_static: the best-path decode that allocates nothing (its scratch is an
array built into the library).  Called through the C interface and held to the allocating entry
point's labels, exactly, on two calls in a row, the second on a smaller problem -- the array
keeps the first call's contents, so anything the second call wrongly relied on would show --
then to the oracle, and a problem whose scratch does not fit must be refused, not attempted."""
import numpy as np
import pytest

from util import DeviceCase, gpu_log_norms, ptr

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
import oracle  # noqa: E402
from transducer_amd import capi  # noqa: E402
from transducer_amd.synthetic import make_inputs, small_config  # noqa: E402

KEYS = ("emissions", "predictions", "labels", "input_lengths", "label_lengths")


def decode(c, entry, blank=0):
    B, T, U, V = c.dims
    out = torch.full((B, U - 1), -1, dtype=torch.int32, device="cuda:0")
    capi.call(entry, ptr(c.E), ptr(c.P), ptr(c.il), ptr(c.ll), ptr(out), B, T, U, V, blank, None)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def case(B, T, U, V, seed):
    d = make_inputs(small_config(B, T, U, V, ragged=True), seed=seed)
    return tuple(d[k] for k in KEYS)


def test_static_decode_equals_the_allocating_decode_twice_in_a_row_second_call_smaller():
    # one utterance of the headline shape (16 MB of the array; its table of best labels comes from
    # candidate lists at this vocabulary), then a small ragged batch with a
    # different vocabulary, label axis and blank index, then the first again
    first = case(1, 2000, 100, 10000, seed=1)
    second = case(3, 130, 37, 515, seed=2)
    for (E, P, labels, il, ll), blank in ((first, 0), (second, 3), (first, 0)):
        c = DeviceCase(E, P, labels, il, ll)
        got = decode(c, "rnnt_hip_viterbi_decode_static", blank)
        want = decode(c, "rnnt_hip_viterbi_decode", blank)
        assert np.array_equal(got, want)
        for b in range(E.shape[0]):  # padding untouched, labels inside the vocabulary
            assert (got[b, ll[b]:] == -1).all()
            assert ((got[b, :ll[b]] >= 0) & (got[b, :ll[b]] < E.shape[2])).all()
    # the small batch against the oracle as well (device LN on both sides: paths are bit-exact
    # given the log-normaliser)
    E, P, labels, il, ll = second
    c = DeviceCase(E, P, labels, il, ll)
    LN = gpu_log_norms(c)
    want = oracle.viterbi(E, P, LN, il, ll, blank=3)
    got = decode(c, "rnnt_hip_viterbi_decode_static", 3)
    for b in range(E.shape[0]):
        assert np.array_equal(got[b, :ll[b]], want[b, :ll[b]])


def test_static_decode_refuses_what_does_not_fit_and_runs_nothing():
    lib = capi.load()
    assert lib.rnnt_hip_static_scratch_bytes() == 64 << 20
    E, P, labels, il, ll = case(2, 40, 9, 64, seed=3)
    c = DeviceCase(E, P, labels, il, ll)
    out = torch.full((32, 100), -1, dtype=torch.int32, device="cuda:0")
    # sizes of the headline batch: 200+ MB of planes; the pointers are never followed
    status = lib.rnnt_hip_viterbi_decode_static(ptr(c.E), ptr(c.P), ptr(c.il), ptr(c.ll), ptr(out),
                                                32, 2000, 101, 10000, 0, None)
    assert status == 3
    assert b"built-in array" in lib.rnnt_hip_last_error()
    torch.cuda.synchronize()
    assert (out == -1).all()


def test_static_decode_replays_from_a_captured_graph_also_where_it_builds_its_table_from_lists():
    # the callers this entry point is for capture it into a HIP graph: every replay (with eager
    # work and synchronisation in between, and the outputs overwritten) must give the eager
    # labels.  5120 columns and 70 label positions are inside the range where the table of best
    # labels comes from candidate lists, whose counters must be cleared inside every replay.
    import ctypes
    assert capi.load().rnnt_hip_maxplus_tries_lists(2, 80, 70, 5120) == 1
    E, P, labels, il, ll = case(2, 80, 69, 5120, seed=4)
    c = DeviceCase(E, P, labels, il, ll)
    B, T, U, V = c.dims
    out = torch.full((B, U - 1), -1, dtype=torch.int32, device="cuda:0")

    def run(stream):
        capi.call("rnnt_hip_viterbi_decode_static", ptr(c.E), ptr(c.P), ptr(c.il), ptr(c.ll),
                  ptr(out), B, T, U, V, 0, stream)

    run(None)
    torch.cuda.synchronize()
    want = out.clone()
    assert np.array_equal(want.cpu().numpy(), decode(c, "rnnt_hip_viterbi_decode", 0))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    for _ in range(3):
        out.fill_(-1)
        (c.E * 2.0).sum().item()  # eager work of the program's own between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
