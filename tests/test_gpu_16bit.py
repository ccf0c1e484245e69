"""16-bit scores and gradients (bf16, fp16) through rnnt_hip_loss_forward_* /
rnnt_hip_loss_backward_*, and the best path through rnnt_hip_viterbi_decode_*.

The reference takes float32 only (transducer/torch_binding.py:195-201), so there is no reference
output to match.  What pins these entry points:

* a 16-bit score converts to fp32 exactly, and the kernels are the fp32 ones with other loads
  and stores, so the costs must EQUAL the fp32 entry points' costs on the upcast inputs, and each
  gradient element must be the fp32 entry points' element rounded once to the 16-bit type
  (allowing one unit where the two paths order an addition differently: the blank/label terms
  are always folded into the dense kernels here, the fp32 path scatters them when the
  vocabulary is small);
* against the CPU oracle on the upcast inputs the tolerance is the fp32 one plus half a unit of
  the type: |got - want| <= 1e-5 + (1e-4 + 2**-8) * |want| for bf16, 2**-11 for fp16 (plus
  fp16's absolute floor of 2**-25 near zero, which the 1e-5 covers).
"""
import numpy as np
import pytest

from util import ATOL, RTOL, dev, ptr, violations

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
import oracle  # noqa: E402
from transducer_amd import capi  # noqa: E402
from transducer_amd.synthetic import CONFIGS  # noqa: E402

# (torch type, entry-point suffix, relative half unit)
KINDS = {"bf16": (torch.bfloat16, "_bf16", 2.0 ** -8), "f16": (torch.float16, "_f16", 2.0 ** -11)}
KIND_NAMES = sorted(KINDS)


def draw(B, T, U, V, seed, sigma=1.0, ragged=True, kind="bf16"):
    g = torch.Generator(device="cuda:0")
    g.manual_seed(seed)
    dtype = KINDS[kind][0]
    E = (torch.randn((B, T, V), generator=g, device="cuda:0") * sigma).to(dtype)
    P = (torch.randn((B, U, V), generator=g, device="cuda:0") * sigma).to(dtype)
    labels = torch.randint(1, V, (B, max(U - 1, 0)), generator=g, device="cuda:0",
                           dtype=torch.int32)
    rng = np.random.default_rng(seed)
    il = np.full(B, T, np.int32)
    ll = np.full(B, U - 1, np.int32)
    if ragged and B > 1:
        il[1:] = rng.integers(max(T // 2, 1), T + 1, B - 1)
        ll[:-1] = rng.integers(0, U, B - 1)
    return E, P, labels, il, ll


def suffix_of(t):
    return {torch.bfloat16: "_bf16", torch.float16: "_f16"}[t.dtype]


def loss_16bit(E, P, labels, il, ll, deltas=None, blank=0):
    """The 16-bit entry points that match the tensors' type."""
    B, T, V = E.shape
    U = P.shape[1]
    d_il, d_ll = dev(il), dev(ll)
    nbytes = capi.load().rnnt_hip_loss_workspace_bytes(B, T, U, V)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0")
    costs = torch.full((B,), float("nan"), device="cuda:0")
    eg = torch.full_like(E, float("nan"))
    pg = torch.full_like(P, float("nan"))
    capi.call("rnnt_hip_loss_forward" + suffix_of(E), ptr(E), ptr(P), ptr(labels), ptr(d_il),
              ptr(d_ll), ptr(costs), ptr(ws), nbytes, B, T, U, V, blank, None)
    capi.call("rnnt_hip_loss_backward" + suffix_of(E), ptr(E), ptr(P), ptr(labels), ptr(d_il),
              ptr(d_ll), ptr(deltas), ptr(eg), ptr(pg), ptr(ws), nbytes, B, T, U, V, blank, None)
    torch.cuda.synchronize()
    return costs, eg, pg


def loss_fp32(E, P, labels, il, ll, deltas=None, blank=0):
    """The fp32 entry points on the same values."""
    E, P = E.float().contiguous(), P.float().contiguous()
    B, T, V = E.shape
    U = P.shape[1]
    d_il, d_ll = dev(il), dev(ll)
    nbytes = capi.load().rnnt_hip_loss_workspace_bytes(B, T, U, V)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0")
    costs = torch.full((B,), float("nan"), device="cuda:0")
    eg = torch.full_like(E, float("nan"))
    pg = torch.full_like(P, float("nan"))
    capi.call("rnnt_hip_loss_forward", ptr(E), ptr(P), ptr(labels), ptr(d_il), ptr(d_ll),
              ptr(costs), ptr(ws), nbytes, B, T, U, V, blank, None)
    capi.call("rnnt_hip_loss_backward", ptr(E), ptr(P), ptr(labels), ptr(d_il), ptr(d_ll),
              ptr(deltas), ptr(eg), ptr(pg), ptr(ws), nbytes, B, T, U, V, blank, None)
    torch.cuda.synchronize()
    return costs, eg, pg


def units_apart(got, want_fp32):
    """|got - round(want)| in units of got's 16-bit type at want's magnitude, elementwise."""
    want = want_fp32.to(got.dtype)
    gi = got.view(torch.int16).to(torch.int32)
    wi = want.view(torch.int16).to(torch.int32)
    # sign-magnitude -> monotone integers
    gi = torch.where(gi < 0, -(gi & 0x7FFF), gi)
    wi = torch.where(wi < 0, -(wi & 0x7FFF), wi)
    return (gi - wi).abs()


def assert_rounds_the_fp32_result(got, want_fp32, what, exact_fraction):
    assert got.dtype in (torch.bfloat16, torch.float16)
    apart = units_apart(got, want_fp32)
    # around zero one unit of the integer view is a denormal step: judge those by value
    # (fp16 keeps nothing below 2**-25 = 3e-8)
    floor = 1e-30 if got.dtype is torch.bfloat16 else 1e-7
    small = want_fp32.abs() < floor
    step = 1e-30 if got.dtype is torch.bfloat16 else 2.0 ** -24  # fp16's smallest step
    assert bool(((got.float() - want_fp32)[small].abs() <= step).all())
    apart = apart[~small]
    worst = int(apart.max()) if apart.numel() else 0
    same = float((apart == 0).float().mean()) if apart.numel() else 1.0
    print("%s: %.5f%% of elements are the rounded fp32 result, worst %d unit(s)"
          % (what, 100 * same, worst))
    assert worst <= 1 and same >= exact_fraction


SHAPES = [
    # B, T, U, V
    (1, 1, 1, 8),
    (2, 5, 1, 16),
    (3, 37, 9, 64),
    (2, 64, 33, 128),
    (4, 50, 11, 32),
    (2, 130, 112, 520),
    (3, 96, 20, 1000),
    # label axes of more than one slice of 112 positions: the slices add up in fp32, a window of
    # frames at a time, and each gradient entry is still rounded once
    (2, 40, 113, 24),
    (2, 70, 225, 520),
    (1, 33, 401, 40),
    (2, 300, 113, 40),  # two windows of frames (288 + 12)
    # vocabularies off the eight-element vector width: the rows are read element by element
    (1, 8, 3, 12),
    (2, 9, 4, 5),
    (2, 70, 20, 1001),
    (3, 40, 12, 515),
]


@pytest.mark.parametrize("kind", KIND_NAMES)
@pytest.mark.parametrize("B,T,U,V", SHAPES)
def test_16bit_against_the_fp32_entry_points_and_the_oracle(B, T, U, V, kind):
    LOWP_RTOL = RTOL + KINDS[kind][2]
    E, P, labels, il, ll = draw(B, T, U, V, seed=B * 1000 + T + U + V, kind=kind)
    deltas = torch.linspace(0.5, 2.0, B, device="cuda:0")
    costs, eg, pg = loss_16bit(E, P, labels, il, ll, deltas)
    c32, e32, p32 = loss_fp32(E, P, labels, il, ll, deltas)
    assert torch.equal(costs, c32)
    assert_rounds_the_fp32_result(eg, e32, "egrads", 0.999)
    assert_rounds_the_fp32_result(pg, p32, "pgrads", 0.999)
    # padding is exact zero
    for b in range(B):
        assert not eg[b, il[b]:].any() and not pg[b, ll[b] + 1:].any()
    want = oracle.loss_and_grads(E.float().cpu().numpy(), P.float().cpu().numpy(),
                                 labels.cpu().numpy(), il, ll)
    d = deltas.cpu().numpy()
    ve, _ = violations(costs.cpu().numpy(), want["costs"])
    assert ve == 0.0
    for got, ref, what in ((eg, want["egrads"], "egrads"), (pg, want["pgrads"], "pgrads")):
        ref = ref * d[:, None, None]
        frac, worst = violations(got.float().cpu().numpy(), ref, rtol=LOWP_RTOL, atol=ATOL)
        assert frac == 0.0, "%s: %.4g%% outside rtol=%g atol=%g (max abs err %g)" % (
            what, 100 * frac, LOWP_RTOL, ATOL, worst)


@pytest.mark.parametrize("kind", KIND_NAMES)
@pytest.mark.parametrize("off_e,off_p", [(200.0, -90.0), (-250.0, 0.0)])
def test_16bit_scores_far_from_zero(off_e, off_p, kind):
    """The same inputs with a large common offset (un-normalised logits; fp16 holds them up to
    65504, with a spacing of 0.125 at 200, which the oracle sees too since it is given the
    upcast arrays): the per-frame reference of the gradient kernels is then large, and the
    rounding of its product with log2(e) must not show in the gradients."""
    LOWP_RTOL = RTOL + KINDS[kind][2]
    E, P, labels, il, ll = draw(2, 80, 17, 640, seed=int(abs(off_e)), kind=kind)
    E = (E.float() + off_e).to(E.dtype)
    P = (P.float() + off_p).to(P.dtype)
    costs, eg, pg = loss_16bit(E, P, labels, il, ll)
    c32, e32, p32 = loss_fp32(E, P, labels, il, ll)
    assert torch.equal(costs, c32)
    assert_rounds_the_fp32_result(eg, e32, "egrads", 0.999)
    assert_rounds_the_fp32_result(pg, p32, "pgrads", 0.999)
    want = oracle.loss_and_grads(E.float().cpu().numpy(), P.float().cpu().numpy(),
                                 labels.cpu().numpy(), il, ll, precision="f64")
    for got, ref, what in ((eg, want["egrads"], "egrads"), (pg, want["pgrads"], "pgrads")):
        frac, worst = violations(got.float().cpu().numpy(), ref, rtol=LOWP_RTOL + 2e-4, atol=ATOL)
        assert frac == 0.0, "%s: %.4g%% outside (max abs err %g)" % (what, 100 * frac, worst)


@pytest.mark.parametrize("kind", KIND_NAMES)
def test_16bit_blank_not_zero_and_repeated_labels(kind):
    LOWP_RTOL = RTOL + KINDS[kind][2]
    B, T, U, V = 2, 40, 7, 24
    E, P, labels, il, ll = draw(B, T, U, V, seed=11, ragged=False, kind=kind)
    labels[:] = torch.tensor([[3, 3, 5, 5, 5, 0], [1, 1, 1, 2, 0, 0]], dtype=torch.int32)
    blank = 4
    costs, eg, pg = loss_16bit(E, P, labels, il, ll, blank=blank)
    c32, e32, p32 = loss_fp32(E, P, labels, il, ll, blank=blank)
    assert torch.equal(costs, c32)
    assert_rounds_the_fp32_result(eg, e32, "egrads", 0.999)
    assert_rounds_the_fp32_result(pg, p32, "pgrads", 0.999)
    want = oracle.loss_and_grads(E.float().cpu().numpy(), P.float().cpu().numpy(),
                                 labels.cpu().numpy(), il, ll, blank=blank)
    for got, ref in ((eg, want["egrads"]), (pg, want["pgrads"])):
        frac, _ = violations(got.float().cpu().numpy(), ref, rtol=LOWP_RTOL, atol=ATOL)
        assert frac == 0.0


@pytest.mark.parametrize("kind", KIND_NAMES)
def test_16bit_empty_utterances_and_empty_batch(kind):
    B, T, U, V = 3, 12, 4, 16
    E, P, labels, il, ll = draw(B, T, U, V, seed=5, kind=kind)
    il[1] = 0   # no frames: cost +inf, zero gradients (transducer_cpu.cpp:39-41)
    ll[2] = 0   # no labels
    costs, eg, pg = loss_16bit(E, P, labels, il, ll)
    c32, e32, p32 = loss_fp32(E, P, labels, il, ll)
    assert torch.equal(costs, c32) and bool(torch.isinf(costs[1]))
    assert not eg[1].any() and not pg[1].any()
    assert_rounds_the_fp32_result(eg, e32, "egrads", 0.999)
    assert_rounds_the_fp32_result(pg, p32, "pgrads", 0.999)
    # B == 0 and T == 0 are legal and touch nothing / clear the outputs
    sfx = KINDS[kind][1]
    capi.call("rnnt_hip_loss_forward" + sfx, None, None, None, None, None, None, None, 0,
              0, T, U, V, 0, None)
    eg0 = torch.full((2, 0, V), 1.0, device="cuda:0", dtype=KINDS[kind][0])
    pg0 = torch.full((2, U, V), 1.0, device="cuda:0", dtype=KINDS[kind][0])
    d_il, d_ll = dev(np.zeros(2, np.int32)), dev(np.zeros(2, np.int32))
    capi.call("rnnt_hip_loss_backward" + sfx, None, None, None, ptr(d_il), ptr(d_ll), None,
              ptr(eg0), ptr(pg0), None, 0, 2, 0, U, V, 0, None)
    torch.cuda.synchronize()
    assert not pg0.any()


@pytest.mark.parametrize("kind", KIND_NAMES)
@pytest.mark.parametrize("B,T,U,V,needle", [
    (1, 4, 1027, 8, "1025 label positions"),
])
def test_16bit_label_axes_past_the_folded_terms_limit_are_refused(B, T, U, V, needle, kind):
    dtype, sfx, _ = KINDS[kind]
    E = torch.zeros((B, T, V), device="cuda:0", dtype=dtype)
    P = torch.zeros((B, U, V), device="cuda:0", dtype=dtype)
    labels = torch.ones((B, U - 1), device="cuda:0", dtype=torch.int32)
    il, ll = dev(np.full(B, T, np.int32)), dev(np.full(B, U - 1, np.int32))
    nbytes = capi.load().rnnt_hip_loss_workspace_bytes(B, T, U, V)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0")
    costs = torch.zeros((B,), device="cuda:0")
    with pytest.raises(capi.RnntHipError, match=needle):
        capi.call("rnnt_hip_loss_forward" + sfx, ptr(E), ptr(P), ptr(labels), ptr(il), ptr(ll),
                  ptr(costs), ptr(ws), nbytes, B, T, U, V, 0, None)
    eg, pg = torch.zeros_like(E), torch.zeros_like(P)
    with pytest.raises(capi.RnntHipError, match=needle):
        capi.call("rnnt_hip_loss_backward" + sfx, ptr(E), ptr(P), ptr(labels), ptr(il), ptr(ll),
                  None, ptr(eg), ptr(pg), ptr(ws), nbytes, B, T, U, V, 0, None)


@pytest.mark.parametrize("kind", KIND_NAMES)
def test_16bit_through_the_torch_module(kind):
    from transducer_amd import TransducerLoss
    dtype = KINDS[kind][0]
    B, T, U, V = 3, 30, 6, 40
    E, P, labels, il, ll = draw(B, T, U, V, seed=21, kind=kind)
    d_il, d_ll = dev(il), dev(ll)
    with pytest.raises(TypeError, match="emissions must be torch.float32"):
        TransducerLoss()(E, P, labels, d_il, d_ll)  # the reference's behaviour stays the default
    with pytest.raises(TypeError, match="emissions must be torch.float32"):
        # the flag of the OTHER 16-bit type does not let this one in
        TransducerLoss(allow_bf16=kind != "bf16", allow_fp16=kind != "f16")(
            E, P, labels, d_il, d_ll)
    crit = TransducerLoss(allow_bf16=kind == "bf16", allow_fp16=kind == "f16")
    with pytest.raises(TypeError, match="predictions must be %s" % dtype):
        crit(E, P.float(), labels, d_il, d_ll)
    Et, Pt = E.clone().requires_grad_(True), P.clone().requires_grad_(True)
    costs = crit(Et, Pt, labels, d_il, d_ll)
    assert costs.dtype is torch.float32
    w = torch.linspace(1.0, 2.0, B, device="cuda:0")
    (costs * w).sum().backward()
    c, eg, pg = loss_16bit(E, P, labels, il, ll, w)
    assert torch.equal(costs.detach(), c)
    assert Et.grad.dtype is dtype and torch.equal(Et.grad, eg)
    assert torch.equal(Pt.grad, pg)
    # float32 tensors still take the fp32 path under the flag
    c32 = crit(E.float(), P.float(), labels, d_il, d_ll)
    assert torch.equal(c32, c)


@pytest.mark.parametrize("kind", KIND_NAMES)
def test_16bit_headline_configuration_against_the_fp32_path(kind):
    dtype = KINDS[kind][0]
    cfg = CONFIGS["cfg4"]
    from transducer_amd.synthetic import lengths
    g = torch.Generator(device="cuda:0")
    g.manual_seed(17)
    B, T, U, V = cfg.B, cfg.T, cfg.U + 1, cfg.V
    E = torch.randn((B, T, V), generator=g, device="cuda:0").to(dtype)
    P = torch.randn((B, U, V), generator=g, device="cuda:0").to(dtype)
    labels = torch.randint(1, V, (B, U - 1), generator=g, device="cuda:0", dtype=torch.int32)
    il, ll = lengths(cfg, np.random.Generator(np.random.Philox(key=17)))
    costs, eg, pg = loss_16bit(E, P, labels, il, ll)
    assert torch.isfinite(costs).all() and torch.isfinite(eg.float()).all()
    d_il, d_ll = dev(il), dev(ll)
    tmask = torch.arange(T, device="cuda:0")[None, :] >= d_il[:, None]
    umask = torch.arange(U, device="cuda:0")[None, :] > d_ll[:, None]
    assert not eg[tmask].any() and not pg[umask].any()
    c32, e32, p32 = loss_fp32(E, P, labels, il, ll)
    assert torch.equal(costs, c32)
    # both paths fold the sparse terms of egrads at this vocabulary: the same fp32 value, rounded
    assert torch.equal(eg, e32.to(dtype))
    assert_rounds_the_fp32_result(pg, p32, "pgrads", 0.9999)


# ------------------------------------------------------------------ best path
def decode_16bit(E, P, il, ll, blank=0):
    B, T, V = E.shape
    U = P.shape[1]
    out = torch.full((B, U - 1), -1, dtype=torch.int32, device="cuda:0")
    d_il, d_ll = dev(il), dev(ll)
    capi.call("rnnt_hip_viterbi_decode" + suffix_of(E), ptr(E), ptr(P), ptr(d_il), ptr(d_ll),
              ptr(out), B, T, U, V, blank, None)
    torch.cuda.synchronize()
    return out


def decode_fp32(E, P, il, ll, blank=0):
    E, P = E.float().contiguous(), P.float().contiguous()
    B, T, V = E.shape
    U = P.shape[1]
    out = torch.full((B, U - 1), -1, dtype=torch.int32, device="cuda:0")
    d_il, d_ll = dev(il), dev(ll)
    capi.call("rnnt_hip_viterbi_decode", ptr(E), ptr(P), ptr(d_il), ptr(d_ll), ptr(out),
              B, T, U, V, blank, None)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("kind", KIND_NAMES)
@pytest.mark.parametrize("B,T,U,V,blank", [(3, 37, 9, 64, 0), (2, 64, 33, 128, 5),
                                           (2, 300, 130, 40, 0), (4, 50, 11, 32, 31)])
def test_16bit_best_path_is_the_fp32_path_and_the_oracles(B, T, U, V, blank, kind):
    """16-bit scores are exact in fp32 and the decode has no rounding step of its own, so the
    path must be the fp32 decode's on the upcast scores, label for label; the oracle is fed the
    device's log-normaliser, as in the fp32 tests (the path is bit-exact GIVEN LN)."""
    E, P, _, il, ll = draw(B, T, U, V, seed=7 * B + T + U + V, kind=kind)
    ll = np.maximum(ll, 1).astype(np.int32)
    got = decode_16bit(E, P, il, ll, blank)
    ref = decode_fp32(E, P, il, ll, blank)
    assert torch.equal(got, ref)
    E32, P32 = E.float().contiguous(), P.float().contiguous()
    LN = torch.empty((B, T, U), device="cuda:0")
    d_il, d_ll = dev(il), dev(ll)
    capi.call("rnnt_hip_log_norms", ptr(E32), ptr(P32), ptr(LN), ptr(d_il), ptr(d_ll),
              B, T, U, V, None)
    want = oracle.viterbi(E32.cpu().numpy(), P32.cpu().numpy(), LN.cpu().numpy(), il, ll,
                          blank=blank)
    g = got.cpu().numpy()
    for b in range(B):
        assert np.array_equal(g[b, :ll[b]], want[b, :ll[b]])
        assert (g[b, ll[b]:] == -1).all()


@pytest.mark.parametrize("kind", KIND_NAMES)
def test_16bit_best_path_through_the_torch_module(kind):
    from transducer_amd import TransducerLoss
    B, T, U, V = 3, 40, 8, 48
    E, P, _, il, ll = draw(B, T, U, V, seed=3, kind=kind)
    d_il, d_ll = dev(il), dev(ll)
    with pytest.raises(TypeError, match="emissions must be torch.float32"):
        TransducerLoss().viterbi(E, P, d_il, d_ll)
    paths = TransducerLoss(allow_bf16=kind == "bf16", allow_fp16=kind == "f16").viterbi(
        E, P, d_il, d_ll)
    ref = decode_16bit(E, P, il, ll)
    for b in range(B):
        assert torch.equal(paths[b, :ll[b]], ref[b, :ll[b]])


def _loss_any(E, P, eg, pg, labels, il, ll, deltas):
    """Whole loss through the entry points of the tensors' type, on exactly these arrays."""
    sfx = "" if E.dtype is torch.float32 else suffix_of(E)
    B, T, V = E.shape
    U = P.shape[1]
    d_il, d_ll = dev(il), dev(ll)
    nbytes = capi.load().rnnt_hip_loss_workspace_bytes(B, T, U, V)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0")
    costs = torch.full((B,), float("nan"), device="cuda:0")
    capi.call("rnnt_hip_loss_forward" + sfx, ptr(E), ptr(P), ptr(labels), ptr(d_il), ptr(d_ll),
              ptr(costs), ptr(ws), nbytes, B, T, U, V, 0, None)
    capi.call("rnnt_hip_loss_backward" + sfx, ptr(E), ptr(P), ptr(labels), ptr(d_il), ptr(d_ll),
              ptr(deltas), ptr(eg), ptr(pg), ptr(ws), nbytes, B, T, U, V, 0, None)
    torch.cuda.synchronize()
    return costs


@pytest.mark.parametrize("kind", ["f32"] + KIND_NAMES)
@pytest.mark.parametrize("B,T,U,V", [(2, 40, 9, 24), (2, 70, 20, 1000), (3, 130, 33, 520)])
def test_arrays_that_start_off_a_16_byte_boundary_give_the_same_bits(B, T, U, V, kind):
    """The vocabulary allows 16-byte row loads but the arrays start one element past a 16-byte
    boundary (4-byte aligned fp32, 2-byte aligned 16-bit), as a view into a larger buffer does:
    rows then come in through the loads at the element's own alignment.  Only the loads differ,
    so costs, gradients and the best path are the aligned call's, bit for bit."""
    dtype = torch.float32 if kind == "f32" else KINDS[kind][0]
    E, P, labels, il, ll = draw(B, T, U, V, seed=B + T + U + V, kind="bf16" if kind == "f32" else kind)
    E, P = E.to(dtype), P.to(dtype)
    deltas = torch.tensor([0.5, 2.0, 1.0][:B], device="cuda:0")

    def shifted(x, fill):
        buf = torch.full((x.numel() + 16,), fill, device="cuda:0", dtype=x.dtype)
        view = buf[1:1 + x.numel()].view(x.shape)
        view.copy_(x)
        assert view.data_ptr() % 16 == x.element_size() and view.is_contiguous()
        return view

    eg, pg = torch.full_like(E, float("nan")), torch.full_like(P, float("nan"))
    costs = _loss_any(E, P, eg, pg, labels, il, ll, deltas)
    Es, Ps = shifted(E, float("nan")), shifted(P, float("nan"))
    egs, pgs = shifted(eg, float("nan")), shifted(pg, float("nan"))
    costs_s = _loss_any(Es, Ps, egs, pgs, labels, il, ll, deltas)
    assert torch.equal(costs, costs_s)
    assert torch.equal(eg.view(torch.uint8), egs.contiguous().view(torch.uint8))
    assert torch.equal(pg.view(torch.uint8), pgs.contiguous().view(torch.uint8))

    sfx = "" if kind == "f32" else KINDS[kind][1]
    d_il, d_ll = dev(il), dev(ll)
    paths = []
    for e, p in ((E, P), (Es, Ps)):
        out = torch.full((B, U - 1), -1, device="cuda:0", dtype=torch.int32)
        capi.call("rnnt_hip_viterbi_decode" + sfx, ptr(e), ptr(p), ptr(d_il), ptr(d_ll),
                  ptr(out), B, T, U, V, 0, None)
        torch.cuda.synchronize()
        paths.append(out)
    assert torch.equal(paths[0], paths[1])
