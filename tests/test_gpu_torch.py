"""TransducerLoss / criterion.viterbi on HIP tensors: the reference's Python tests
(torch_test.py) replayed against this build, plus what its autograd contract implies."""
import numpy as np
import pytest
import torch

import oracle
from transducer_amd import TransducerLoss
from transducer_amd.synthetic import make_inputs, small_config
from util import assert_close, reference_vectors

pytestmark = pytest.mark.gpu
VEC = reference_vectors()


def apply_transducer(emissions, predictions, labels, scales=None):
    """torch_test.py:11-30 on the HIP device."""
    device = torch.device("cuda")
    emissions = torch.tensor(emissions, dtype=torch.float32, device=device, requires_grad=True)
    predictions = torch.tensor(predictions, dtype=torch.float32, device=device, requires_grad=True)
    lengths = torch.tensor([emissions.shape[1]] * emissions.shape[0], dtype=torch.int32,
                           device=device)
    label_lengths = torch.tensor([len(l) for l in labels], dtype=torch.int32, device=device)
    labels = torch.tensor(labels, dtype=torch.int32, device=device)
    costs = TransducerLoss()(emissions, predictions, labels, lengths, label_lengths)
    if scales is None:
        torch.sum(costs).backward()
    else:
        (costs * torch.tensor(scales, device=device)).sum().backward()
    return costs.detach().cpu(), emissions.grad.cpu(), predictions.grad.cpu()


@pytest.mark.parametrize("name", ["small", "big"])
def test_reference_python_goldens(name):
    v = VEC[name]
    costs, eg, pg = apply_transducer(v["emissions"], v["predictions"], v["labels"])
    # the reference's CPU bar (torch.allclose defaults), stricter than its CUDA bar of 1e-3
    assert torch.allclose(costs, torch.tensor(v["costs"]), rtol=1e-5, atol=1e-6)
    assert torch.allclose(eg, torch.tensor(v["egrads"]), rtol=1e-5, atol=1e-6)
    assert torch.allclose(pg, torch.tensor(v["pgrads"]), rtol=1e-5, atol=1e-6)


def test_reference_python_viterbi():
    v = VEC["viterbi_bigger"]
    dev = torch.device("cuda")
    labels = TransducerLoss().viterbi(
        torch.tensor(v["emissions"], device=dev), torch.tensor(v["predictions"], device=dev),
        torch.tensor(v["input_lengths"], dtype=torch.int32, device=dev),
        torch.tensor(v["label_lengths"], dtype=torch.int32, device=dev))
    assert labels.dtype == torch.int32 and labels.is_cuda
    assert torch.equal(labels.cpu(), torch.tensor(v["labels"], dtype=torch.int32))


def test_upstream_gradient_scales_rows():
    v = VEC["big"]
    c1, e1, p1 = apply_transducer(v["emissions"], v["predictions"], v["labels"])
    c2, e2, p2 = apply_transducer(v["emissions"], v["predictions"], v["labels"], [0.25, 3.0])
    s = torch.tensor([0.25, 3.0])[:, None, None]
    assert torch.equal(c1, c2)
    assert torch.allclose(e2, s * e1, rtol=1e-6, atol=1e-7)
    assert torch.allclose(p2, s * p1, rtol=1e-6, atol=1e-7)


def test_finite_differences_like_the_reference():
    """torch_test.py:209-269: central differences, epsilon 1e-2, every element, ragged."""
    torch.manual_seed(0)
    B, T, U, V = 3, 6, 3, 4
    dev = torch.device("cuda")
    E = torch.rand((B, T, V), device=dev)
    P = torch.rand((B, U, V), device=dev)
    labels = torch.randint(1, V, (B, U - 1), dtype=torch.int32, device=dev)
    il = torch.tensor([T, 4, 2], dtype=torch.int32, device=dev)
    ll = torch.tensor([U - 1, 1, 2], dtype=torch.int32, device=dev)
    crit = TransducerLoss()
    E.requires_grad = True
    P.requires_grad = True
    crit(E, P, labels, il, ll).sum().backward()
    eg, pg = E.grad.clone(), P.grad.clone()
    E.requires_grad = False
    P.requires_grad = False
    eps = 1e-2
    for arr, grad in ((E, eg), (P, pg)):
        flat = arr.view(-1)
        for i in range(flat.numel()):
            flat[i] += eps
            up = crit(E, P, labels, il, ll).sum().item()
            flat[i] -= 2 * eps
            dn = crit(E, P, labels, il, ll).sum().item()
            flat[i] += eps
            num = (up - dn) / (2 * eps)
            assert abs(num - grad.view(-1)[i].item()) <= 1e-3 + 1e-3 * abs(grad.view(-1)[i].item())


def test_module_against_oracle_ragged_with_padding_rows():
    cfg = small_config(4, 33, 9, 29, ragged=True)
    d = make_inputs(cfg, seed=6)
    dev = torch.device("cuda")
    E = torch.tensor(d["emissions"], device=dev, requires_grad=True)
    P = torch.tensor(d["predictions"], device=dev, requires_grad=True)
    labels = torch.tensor(d["labels"], device=dev)
    il = torch.tensor(d["input_lengths"], device=dev)
    ll = torch.tensor(d["label_lengths"], device=dev)
    costs = TransducerLoss()(E, P, labels, il, ll)
    assert costs.shape == (4,) and costs.dtype == torch.float32
    costs.sum().backward()
    want = oracle.loss_and_grads(d["emissions"], d["predictions"], d["labels"],
                                 d["input_lengths"], d["label_lengths"])
    assert_close(costs.detach().cpu().numpy(), want["costs"], what="costs")
    assert_close(E.grad.cpu().numpy(), want["egrads"], what="egrads")
    assert_close(P.grad.cpu().numpy(), want["pgrads"], what="pgrads")
    got = TransducerLoss().viterbi(E.detach(), P.detach(), il, ll).cpu().numpy()
    LN = oracle.log_norms_naive(d["emissions"], d["predictions"], d["input_lengths"],
                                d["label_lengths"])
    ref = oracle.viterbi(d["emissions"], d["predictions"], LN, d["input_lengths"],
                         d["label_lengths"])
    for b in range(4):
        n = d["label_lengths"][b]
        assert np.array_equal(got[b, :n], ref[b, :n])


def test_nonzero_blank_and_noncontiguous_scores():
    cfg = small_config(2, 12, 4, 10, ragged=False)
    d = make_inputs(cfg, seed=13)
    dev = torch.device("cuda")
    blank = 4
    labels_np = np.where(d["labels"] == blank, 1, d["labels"]).astype(np.int32)
    # non-contiguous views of the scores: the reference would read them wrongly
    # (torch_binding.py passes data_ptr() unchecked); here they are made dense first
    E = torch.tensor(d["emissions"], device=dev).transpose(0, 1).contiguous().transpose(0, 1)
    assert not E.is_contiguous()
    P = torch.tensor(d["predictions"], device=dev)
    costs = TransducerLoss(blank=blank)(E, P, torch.tensor(labels_np, device=dev),
                                        torch.tensor(d["input_lengths"], device=dev),
                                        torch.tensor(d["label_lengths"], device=dev))
    want = oracle.loss_and_grads(d["emissions"], d["predictions"], labels_np, d["input_lengths"],
                                 d["label_lengths"], blank=blank)
    assert_close(costs.cpu().numpy(), want["costs"], what="costs")


def test_backward_twice_on_one_forward_gives_the_same_gradients():
    """benchmarks/torch_benchmarks.py:76-82 repeats loss.backward(retain_graph=True): the state
    the forward pass leaves behind must survive a backward pass."""
    d = make_inputs(small_config(3, 90, 12, 40, ragged=True), seed=17)
    dev = torch.device("cuda")
    E = torch.tensor(d["emissions"], device=dev, requires_grad=True)
    P = torch.tensor(d["predictions"], device=dev, requires_grad=True)
    labels = torch.tensor(d["labels"], device=dev)
    il = torch.tensor(d["input_lengths"], device=dev)
    ll = torch.tensor(d["label_lengths"], device=dev)
    loss = TransducerLoss()(E, P, labels, il, ll).sum()
    loss.backward(retain_graph=True)
    e1, p1 = E.grad.clone(), P.grad.clone()
    E.grad = None
    P.grad = None
    loss.backward(retain_graph=True)
    assert torch.equal(E.grad, e1) and torch.equal(P.grad, p1)


def _small_problem(seed=23, shape=(3, 150, 20, 260)):
    d = make_inputs(small_config(*shape, ragged=True), seed=seed)
    dev = torch.device("cuda")
    return (torch.tensor(d["emissions"], device=dev), torch.tensor(d["predictions"], device=dev),
            torch.tensor(d["labels"], device=dev), torch.tensor(d["input_lengths"], device=dev),
            torch.tensor(d["label_lengths"], device=dev))


def test_loss_on_a_side_stream_matches_the_default_stream():
    """The C interface takes the stream to enqueue on (the reference is wired to stream 0,
    transducer_cuda.cu:326-331); the torch front end passes torch's current stream."""
    E, P, labels, il, ll = _small_problem()
    E1, P1 = E.clone().requires_grad_(), P.clone().requires_grad_()
    TransducerLoss()(E1, P1, labels, il, ll).sum().backward()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()  # default priority
    E2, P2 = E.clone().requires_grad_(), P.clone().requires_grad_()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        costs = TransducerLoss()(E2, P2, labels, il, ll)
        costs.sum().backward()
        paths = TransducerLoss().viterbi(E, P, il, ll)
    side.synchronize()
    assert torch.equal(E1.grad, E2.grad) and torch.equal(P1.grad, P2.grad)
    # entries past an utterance's label length are unwritten padding, as in the reference
    written = torch.arange(paths.shape[1], device=paths.device)[None, :] < ll[:, None]
    again = TransducerLoss().viterbi(E, P, il, ll)
    assert torch.equal(paths[written], again[written])


# the second shape has 19 slabs of frames on few tiles: the prediction-gradient walk splits over
# frames there, and its arrival counters must be cleared again inside every replay; the last two
# have 300 and 700 labels: the lattice walks run blocks of the label axis side by side, whose
# tagged entries must be cleared inside every replay too (and the emission gradients of 700
# labels add up over several launches)
@pytest.mark.parametrize("shape", [(3, 150, 20, 260), (2, 600, 20, 1024), (2, 150, 300, 40),
                                   (2, 60, 700, 24)])
def test_fused_entry_points_replay_from_a_captured_graph(shape):
    """rnnt_hip_loss_forward / rnnt_hip_loss_backward allocate nothing and use kernels only, so
    a caller may capture them; every replay (with eager work and synchronisation in between)
    must reproduce the eager result bit for bit."""
    import ctypes
    from transducer_amd import capi
    E, P, labels, il, ll = _small_problem(seed=29, shape=shape)
    B, T, V = E.shape
    U = P.shape[1]
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    nbytes = capi.load().rnnt_hip_loss_workspace_bytes(B, T, U, V)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=E.device)
    costs, eg, pg = torch.empty(B, device=E.device), torch.empty_like(E), torch.empty_like(P)

    def run(stream):
        capi.call("rnnt_hip_loss_forward", p(E), p(P), p(labels), p(il), p(ll), p(costs), p(ws),
                  nbytes, B, T, U, V, 0, stream)
        capi.call("rnnt_hip_loss_backward", p(E), p(P), p(labels), p(il), p(ll), None, p(eg), p(pg),
                  p(ws), nbytes, B, T, U, V, 0, stream)

    run(None)
    torch.cuda.synchronize()
    want = (costs.clone(), eg.clone(), pg.clone())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    for _ in range(3):
        costs.fill_(float("nan")); eg.fill_(float("nan")); pg.fill_(float("nan"))
        ws.fill_(0xff)  # the calls may assume nothing about the workspace's contents
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(costs, want[0]) and torch.equal(eg, want[1]) and torch.equal(pg, want[2])
