"""Shared helpers of the test suite: fixtures on disk, tolerance accounting, device plumbing."""
import ctypes
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")

# tolerance the loss and its gradients must meet against the reference in fp32
RTOL, ATOL = 1e-4, 1e-5


def reference_vectors():
    with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
        return json.load(f)


def vector_case(v):
    E = np.array(v["emissions"], np.float32)
    P = np.array(v["predictions"], np.float32)
    B, U = P.shape[0], P.shape[1]
    labels = np.array(v["labels"], np.int32).reshape(B, U - 1) if "costs" in v or U == 1 \
        else np.zeros((B, U - 1), np.int32)
    il = np.array(v["input_lengths"], np.int32)
    ll = np.array(v["label_lengths"], np.int32)
    return E, P, labels, il, ll


_ref_cases = None


def ref_cases():
    """{name: {array name: ndarray}} from tests/golden/ref_cases.npz (made by the reference's
    own compiled CPU sources, see tests/golden/make_golden.py)."""
    global _ref_cases
    if _ref_cases is None:
        z = np.load(os.path.join(GOLDEN, "ref_cases.npz"))
        out = {}
        for key in z.files:
            name, arr = key.split("/")
            out.setdefault(name, {})[arr] = z[key]
        _ref_cases = out
    return _ref_cases


def violations(got, want, rtol=RTOL, atol=ATOL):
    """fraction of entries with |got-want| > atol + rtol*|want|, and the largest |got-want|."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    err = np.abs(got - want)
    bad = err > atol + rtol * np.abs(want)
    bad |= np.isnan(got) != np.isnan(want)
    return float(bad.mean()) if bad.size else 0.0, float(np.nanmax(err)) if err.size else 0.0


def assert_close(got, want, rtol=RTOL, atol=ATOL, what=""):
    frac, worst = violations(got, want, rtol, atol)
    assert frac == 0.0, "%s: %.4g%% of entries outside rtol=%g atol=%g (max abs err %g)" % (
        what, 100 * frac, rtol, atol, worst)


def assert_same_bits(got, want, what=""):
    """Bit for bit, NaN patterns included (cells the library must leave untouched hold the NaN
    they were filled with on both sides)."""
    got = np.ascontiguousarray(got, np.float32).view(np.uint32)
    want = np.ascontiguousarray(want, np.float32).view(np.uint32)
    both_nan = np.isnan(got.view(np.float32)) & np.isnan(want.view(np.float32))
    diff = (got != want) & ~both_nan
    assert not diff.any(), "%s: %d of %d entries differ in their bits (%.4g%%)" % (
        what, int(diff.sum()), diff.size, 100.0 * diff.mean())


def check_close_reference(a, b, rtol=1e-6, atol=1e-5):
    """The reference's own comparison (transducer/test.h:19-29): threshold
    max(rtol*max(|a|,|b|), atol), infinities must match exactly."""
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    assert a.shape == b.shape
    inf = np.isinf(a) | np.isinf(b)
    assert np.array_equal(a[inf], b[inf])
    thr = np.maximum(rtol * np.maximum(np.abs(a), np.abs(b)), atol)
    ok = np.abs(a - b)[~inf] <= thr[~inf]
    assert ok.all(), "max abs err %g" % np.abs(a - b)[~inf].max()


# ------------------------------------------------------------------ device plumbing
def dev(a, device="cuda:0"):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


class DeviceCase(object):
    """Device copies of one problem plus the sizes the C interface wants."""

    def __init__(self, E, P, labels, il, ll):
        self.B, self.T, self.V = E.shape
        self.U = P.shape[1]
        self.E, self.P = dev(E), dev(P)
        self.labels = dev(labels.reshape(self.B, max(self.U - 1, 0)))
        self.il, self.ll = dev(il), dev(ll)

    @property
    def dims(self):
        return (self.B, self.T, self.U, self.V)


def gpu_forward(c, LN, blank=0):
    import torch
    from transducer_amd import capi
    B, T, U, V = c.dims
    costs = torch.full((B,), float("nan"), device=c.E.device)
    alphas = torch.full((B, T, U), float("nan"), device=c.E.device)
    dLN = dev(LN)
    capi.call("rnnt_hip_forward", ptr(c.E), ptr(c.P), ptr(costs), ptr(alphas), ptr(dLN),
              ptr(c.labels), ptr(c.il), ptr(c.ll), B, T, U, V, blank, None)
    torch.cuda.synchronize()
    return costs.cpu().numpy(), alphas.cpu().numpy()


def gpu_backward(c, alphas, LN, blank=0):
    import torch
    from transducer_amd import capi
    B, T, U, V = c.dims
    eg = torch.full_like(c.E, float("nan"))
    pg = torch.full_like(c.P, float("nan"))
    lng = torch.full((B, T, U), float("nan"), device=c.E.device)
    d_alphas, d_LN = dev(np.nan_to_num(alphas)), dev(LN)  # named: must outlive the launch
    capi.call("rnnt_hip_backward", ptr(c.E), ptr(c.P), ptr(eg), ptr(pg), ptr(lng),
              ptr(d_alphas), ptr(d_LN), ptr(c.labels), ptr(c.il), ptr(c.ll),
              B, T, U, V, blank, None)
    torch.cuda.synchronize()
    return eg.cpu().numpy(), pg.cpu().numpy(), lng.cpu().numpy()


def gpu_viterbi(c, LN, blank=0):
    import torch
    from transducer_amd import capi
    B, T, U, V = c.dims
    out = torch.full((B, max(U - 1, 0)), -1, dtype=torch.int32, device=c.E.device)
    d_LN = dev(LN)
    capi.call("rnnt_hip_viterbi", ptr(c.E), ptr(c.P), ptr(d_LN), ptr(out) if U > 1 else None,
              ptr(c.il), ptr(c.ll), B, T, U, V, blank, None)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def gpu_log_norms(c, with_lengths=True):
    import torch
    from transducer_amd import capi
    B, T, U, V = c.dims
    LN = torch.full((B, T, U), float("nan"), device=c.E.device)
    capi.call("rnnt_hip_log_norms", ptr(c.E), ptr(c.P), ptr(LN),
              ptr(c.il) if with_lengths else None, ptr(c.ll) if with_lengths else None,
              B, T, U, V, None)
    torch.cuda.synchronize()
    return LN.cpu().numpy()


def gpu_dense_grads(c, eg, pg, lng, LN, deltas=None):
    import torch
    from transducer_amd import capi
    B, T, U, V = c.dims
    deg, dpg = dev(eg), dev(pg)
    dd = dev(deltas) if deltas is not None else None
    d_lng, d_LN = dev(lng), dev(LN)
    capi.call("rnnt_hip_dense_grads", ptr(c.E), ptr(c.P), ptr(deg), ptr(dpg), ptr(d_lng),
              ptr(d_LN), ptr(dd), ptr(c.il), ptr(c.ll), B, T, U, V, None)
    torch.cuda.synchronize()
    return deg.cpu().numpy(), dpg.cpu().numpy()


def gpu_loss(c, deltas=None, blank=0):
    """whole loss through the C interface -> costs, egrads, pgrads (numpy)."""
    import torch
    from transducer_amd import capi
    B, T, U, V = c.dims
    nbytes = capi.load().rnnt_hip_loss_workspace_bytes(B, T, U, V)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=c.E.device)
    costs = torch.full((B,), float("nan"), device=c.E.device)
    eg = torch.full_like(c.E, float("nan"))
    pg = torch.full_like(c.P, float("nan"))
    dd = dev(deltas) if deltas is not None else None
    capi.call("rnnt_hip_loss_forward", ptr(c.E), ptr(c.P), ptr(c.labels), ptr(c.il), ptr(c.ll),
              ptr(costs), ptr(ws), nbytes, B, T, U, V, blank, None)
    capi.call("rnnt_hip_loss_backward", ptr(c.E), ptr(c.P), ptr(c.labels), ptr(c.il), ptr(c.ll),
              ptr(dd), ptr(eg), ptr(pg), ptr(ws), nbytes, B, T, U, V, blank, None)
    torch.cuda.synchronize()
    return costs.cpu().numpy(), eg.cpu().numpy(), pg.cpu().numpy()
