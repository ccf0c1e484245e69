#!/usr/bin/env python3
"""Benchmark of the RNN-T loss hot path on one MI355X.

A "step" is one forward+backward of the loss (log-normaliser, alpha recursion, dalpha recursion,
dense + sparse gradients) on one synthetic batch that is already resident in HBM, called through
the C interface of librnnt_hip.so.  Prints ONE JSON line:

  value / ms_per_step   milliseconds per fwd+bwd at the headline shape (lower is better)
  roofline              the slowest matrix-core kernel: algorithmic fp32 flops of one launch
                        (2 * V * sum_b T_b*(U_b+1), valid lattice cells only) over its mean
                        duration, measured with HIP events on the launch stream during the
                        timed steps, against the 157.3 TFLOP/s fp32 matrix peak (the kernels
                        form each fp32 product from six bf16 matrix products, so this fraction
                        may pass 1); "hbm" inside it prices the same launch against 8 TB/s with
                        the bytes the algorithm must move (valid rows of E and P read once,
                        the kernel's output written once)
  cpu_baseline          the CPU path (the OpenMP restatement in oracle/, which is checked bit for
                        bit against the reference's compiled sources) timed on the host cores
                        over a bounded sample of the same workload and scaled by lattice-cell
                        count; the lattice recursions are also timed through the reference's
                        own transducer_cpu.cpp build (oracle/_ref) when it is present
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "ms per fwd+bwd RNN-T loss, B=32 T=2000 U=100 V=10000; % of roofline"
PEAK_FP32_MATRIX_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch (fetched + written) from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this
# file, scaled by what the counters read for a plain copy of known size
# (profiles/cfg4_hbm_traffic_counters.md).  Recorded, not measured live: counters need rocprofv3.
RECORDED_TRAFFIC_BYTES = {"cfg4": {"lse": 2.546e9, "egrads": 5.633e9, "pgrads": 3.129e9}}

WORKLOADS = {
    # BASELINE configs[3]: the shape the metric is quoted on
    "cfg4": dict(B=32, T=2000, U=100, V=10000, sigma=1.0, ragged_T=(1500, 2000), ragged_U=(75, 100)),
    "cfg2": dict(B=8, T=2000, U=100, V=100, sigma=1.0, ragged_T=None, ragged_U=None),
    "cfg3a": dict(B=8, T=2000, U=100, V=1000, sigma=2.0, ragged_T=(1000, 2000), ragged_U=(50, 100)),
    "cfg3b": dict(B=8, T=2000, U=100, V=2000, sigma=2.0, ragged_T=(1000, 2000), ragged_U=(50, 100)),
    # BASELINE configs[4]: teacher-forced best path (log-normaliser + max-plus + lattice + backtrace)
    "cfg5": dict(B=32, T=2000, U=100, V=10000, sigma=1.0, ragged_T=(1500, 2000), ragged_U=(75, 100),
                 kind="viterbi"),
    "cfg5ties": dict(B=32, T=2000, U=100, V=10000, sigma=1.0, ragged_T=(1500, 2000),
                     ragged_U=(75, 100), kind="viterbi", near_ties=True),
    # the inputs of the reference's own benchmark script at the shape its README quotes 223.33 ms
    # for on an A100 (benchmarks/torch_benchmarks.py:26-35: uniform [0,1) scores, full lengths)
    "readme": dict(B=32, T=2000, U=100, V=10000, sigma=1.0, ragged_T=None, ragged_U=None,
                   uniform=True, published_ms=223.33),
    # the headline shape with bf16 scores and gradients (rnnt_hip_loss_*_bf16; not a reference
    # configuration: the reference takes float32 only)
    "cfg5bf16": dict(B=32, T=2000, U=100, V=10000, sigma=1.0, ragged_T=(1500, 2000),
                     ragged_U=(75, 100), kind="viterbi", io="bf16"),
    "cfg4bf16": dict(B=32, T=2000, U=100, V=10000, sigma=1.0, ragged_T=(1500, 2000),
                     ragged_U=(75, 100), io="bf16"),
    "cfg4f16": dict(B=32, T=2000, U=100, V=10000, sigma=1.0, ragged_T=(1500, 2000),
                    ragged_U=(75, 100), io="f16"),
}
PEAK_VALU_TLANEOPS = 256 * 64 * 2.4e9 / 1e12  # 256 CUs x 64 fp32 lanes x 2.4 GHz, one op per lane


def make_device_inputs(w, seed, device):
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    B, T, U, V = w["B"], w["T"], w["U"], w["V"]
    draw = torch.rand if w.get("uniform") else torch.randn
    E = draw((B, T, V), generator=g, device=device, dtype=torch.float32) * w["sigma"]
    P = draw((B, U + 1, V), generator=g, device=device, dtype=torch.float32) * w["sigma"]
    if w.get("near_ties"):  # a tenth of every frame's entries repeat another column's value
        for b in range(B):
            dst = torch.randint(1, V, (T, V // 10), generator=g, device=device)
            src = torch.randint(1, V, (T, V // 10), generator=g, device=device)
            E[b].scatter_(1, dst, E[b].gather(1, src))
    labels = torch.randint(1, V, (B, U), generator=g, device=device, dtype=torch.int32)
    rng = np.random.Generator(np.random.Philox(key=seed))
    il = np.full(B, T, np.int32)
    ll = np.full(B, U, np.int32)
    if w["ragged_T"]:
        il = rng.integers(w["ragged_T"][0], w["ragged_T"][1] + 1, B).astype(np.int32)
        il[0] = T
    if w["ragged_U"]:
        ll = rng.integers(w["ragged_U"][0], w["ragged_U"][1] + 1, B).astype(np.int32)
        ll[B - 1] = U
    return E, P, labels, torch.from_numpy(il).to(device), torch.from_numpy(ll).to(device), il, ll


def cpu_baseline(w, il, ll, seconds_budget=15.0):
    """Times the CPU path on a bounded sample of the workload and scales to the full batch.

    Full path = log-normaliser + alpha + dalpha + dense gradient accumulation, i.e. the
    torch-free end-to-end sequence of the reference's C++ tests (transducer/test.cpp:7-90), run
    by the OpenMP restatement in oracle/ (the reference's own LSE / dense-gradient helpers in
    test.h are single-threaded test code).  The lattice recursions alone are also timed through
    the reference's own transducer_cpu.cpp when oracle/_ref was built."""
    import oracle  # checker code, used here only as the timed CPU baseline
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    B, T, U, V = w["B"], w["T"], w["U"], w["V"]
    Bs = max(1, min(B, threads))
    rng = np.random.Generator(np.random.Philox(key=1234))
    P = rng.standard_normal((Bs, U + 1, V), dtype=np.float32) * np.float32(w["sigma"])
    labels = rng.integers(1, V, (Bs, U)).astype(np.int32)
    sll = ll[:Bs].astype(np.int32)

    def run(Ts):
        E = rng.standard_normal((Bs, Ts, V), dtype=np.float32) * np.float32(w["sigma"])
        sil = np.minimum(il[:Bs], Ts).astype(np.int32)
        sil[0] = Ts
        t0 = time.perf_counter()
        LN = oracle.log_norms_naive(E, P, sil, sll)
        t1 = time.perf_counter()
        costs, alphas = oracle.forward(E, P, LN, labels, sil, sll)
        eg, pg, lng = oracle.backward(E, P, np.nan_to_num(alphas), LN, labels, sil, sll)
        t2 = time.perf_counter()
        oracle.accumulate_grads(E, P, eg, pg, lng, LN, sil, sll)
        t3 = time.perf_counter()
        dp_ref = None
        if oracle.have_ref():
            r0 = time.perf_counter()
            _, ra = oracle.ref_forward(E, P, LN, labels, sil, sll)
            oracle.ref_backward(E, P, np.nan_to_num(ra), LN, labels, sil, sll)
            dp_ref = time.perf_counter() - r0
        cells = float(np.sum(sil.astype(np.int64) * (sll.astype(np.int64) + 1)))
        return (t1 - t0, t2 - t1, t3 - t2, dp_ref, cells)

    probe = run(min(T, 16))  # calibrates the sample size to the time budget
    per_frame = max(sum(probe[:3]) / min(T, 16), 1e-6)
    Ts = int(max(16, min(T, seconds_budget / per_frame)))
    lse_s, dp_s, acc_s, dp_ref_s, cells_sample = run(Ts)
    cells_full = float(np.sum(il.astype(np.int64) * (ll.astype(np.int64) + 1)))
    scale = cells_full / cells_sample
    out = {
        "value": round((lse_s + dp_s + acc_s) * 1e3 * scale, 1),
        "unit": "ms per fwd+bwd, scaled from the sample by lattice-cell count",
        "cores": threads,
        "kind": "port",
        "sample": "%d of %d utterances x first %d of %d frames, U=%d V=%d; naive LSE + alpha + "
                  "dalpha + dense gradient accumulation (OpenMP over utterances); measured %.2f s"
                  % (Bs, B, Ts, T, U, V, lse_s + dp_s + acc_s),
        "lse_ms": round(lse_s * 1e3 * scale, 1),
        "lattice_ms": round(dp_s * 1e3 * scale, 2),
        "dense_grads_ms": round(acc_s * 1e3 * scale, 1),
    }
    if dp_ref_s is not None:
        out["lattice_ms_reference_build"] = round(dp_ref_s * 1e3 * scale, 2)
    return out


def viterbi_main(args, w, capi, E, P, d_il, d_ll, il, ll):
    """--workload cfg5: one step = rnnt_hip_viterbi_decode (log-normaliser, best label per cell,
    best-path lattice, backtrace).  The dominant kernel is the max-plus scan, which has no
    matrix form: it is priced in vector lane-operations (one add and one compare/select per
    (t, u, v) of the valid lattice) against 256 CUs x 64 lanes x 2.4 GHz."""
    import torch
    B, T, U1, V = w["B"], w["T"], w["U"] + 1, w["V"]
    out_labels = torch.empty((B, U1 - 1), dtype=torch.int32, device=E.device)
    stream = ctypes.c_void_p(torch.cuda.current_stream(E.device).cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    io = w.get("io")
    bf16 = io is not None
    if bf16:
        dtype16 = {"bf16": torch.bfloat16, "f16": torch.float16}[io]
        E, P = E.to(dtype16), P.to(dtype16)
    entry = "rnnt_hip_viterbi_decode" + ("_" + io if bf16 else "")

    def step():
        capi.call(entry, p(E), p(P), p(d_il), p(d_ll), p(out_labels), B, T, U1, V, 0, stream)

    for _ in range(args.warmup):
        step()
        torch.cuda.synchronize()
    capi.profile_enable(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
        torch.cuda.synchronize()
    t1 = time.perf_counter()
    stages = capi.profile_read()
    capi.profile_enable(False)
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    per_launch = {k: (ms / n) for k, (ms, n) in stages.items() if n}
    per_step = {k: round(ms / args.steps, 4) for k, (ms, n) in stages.items() if n}
    cells = float(np.sum(il.astype(np.int64) * (ll.astype(np.int64) + 1)))
    lane_ops = 2.0 * (V - 1) * cells
    achieved = lane_ops / (per_launch["maxplus"] * 1e-3) / 1e12
    out = {
        "metric": "ms per teacher-forced viterbi decode, B=%d T=%d U=%d V=%d" % (B, T, w["U"], V),
        "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 arithmetic on %s scores" % io if bf16 else "f32", "data": "synthetic",
        "config": {"workload": "%s: B=%d T=%d U=%d V=%d blank=0, N(0,1) scores%s, input_lengths "
                               "U[%d,%d], label_lengths U[%d,%d]"
                               % ((args.workload, B, T, w["U"], V,
                                   ", a tenth of each frame's entries duplicated"
                                   if w.get("near_ties") else "") + w["ragged_T"] + w["ragged_U"]),
                   "seed": args.seed, "valid_lattice_cells": int(cells)},
        "roofline": {"bound": "valu", "kernel": "maxplus_kernel", "achieved": round(achieved, 2),
                     "peak": round(PEAK_VALU_TLANEOPS, 2), "unit": "Tlane-op/s",
                     "frac": round(achieved / PEAK_VALU_TLANEOPS, 4), "traffic": None,
                     "kernel_ms": round(per_launch["maxplus"], 4), "lane_ops_per_launch": lane_ops},
        "stage_ms_per_step": per_step,
    }
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg4", choices=sorted(WORKLOADS))
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain elementwise copy of the emissions array (B*T*V*4 "
                         "bytes read, as many written) so that a counter run can scale "
                         "FETCH_SIZE / WRITE_SIZE by what they read for a known transfer")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures the one-GPU hot path; --gpus %d is not supported "
                 "(the batch shards trivially, no multi-GPU code is part of this build)" % args.gpus)

    import torch
    from transducer_amd import capi

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device")
    capi.load()  # raises if librnnt_hip.so is not built: there is no fallback path
    device = torch.device("cuda:0")
    w = WORKLOADS[args.workload]
    B, T, U1, V = w["B"], w["T"], w["U"] + 1, w["V"]
    E, P, labels, d_il, d_ll, il, ll = make_device_inputs(w, args.seed, device)
    if w.get("kind") == "viterbi":
        return viterbi_main(args, w, capi, E, P, d_il, d_ll, il, ll)
    io = w.get("io")  # None (fp32), "bf16" or "f16"
    bf16 = io is not None
    if bf16:
        dtype16 = {"bf16": torch.bfloat16, "f16": torch.float16}[io]
        E, P = E.to(dtype16), P.to(dtype16)
    suffix, esize = ("_" + io, 2.0) if bf16 else ("", 4.0)
    costs = torch.empty(B, device=device)
    egrads = torch.empty_like(E)
    pgrads = torch.empty_like(P)
    deltas = torch.ones(B, device=device)
    nbytes = capi.load().rnnt_hip_loss_workspace_bytes(B, T, U1, V)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    stream = ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())

    def step():
        capi.call("rnnt_hip_loss_forward" + suffix, p(E), p(P), p(labels), p(d_il), p(d_ll),
                  p(costs), p(ws), nbytes, B, T, U1, V, 0, stream)
        capi.call("rnnt_hip_loss_backward" + suffix, p(E), p(P), p(labels), p(d_il), p(d_ll),
                  p(deltas), p(egrads), p(pgrads), p(ws), nbytes, B, T, U1, V, 0, stream)

    for _ in range(args.warmup):
        step()
        torch.cuda.synchronize()
    if args.copy_calibration:
        torch.mul(E, 1.0, out=egrads)  # vectorized_elementwise_kernel: reads E, writes egrads
        torch.cuda.synchronize()
    capi.profile_enable(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
        torch.cuda.synchronize()  # a device sync per call, as in benchmarks/torch_benchmarks.py:8-20
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    stages = capi.profile_read()
    capi.profile_enable(False)
    ms_per_step = (t1 - t0) * 1e3 / args.steps

    per_launch = {k: (ms / n) for k, (ms, n) in stages.items() if n}
    per_step = {k: round(ms / args.steps, 4) for k, (ms, n) in stages.items() if n}
    cells = float(np.sum(il.astype(np.int64) * (ll.astype(np.int64) + 1)))
    flops_one = 2.0 * V * cells  # one contraction over the valid lattice
    mfma_kernels = {k: per_launch[k] for k in ("lse", "egrads", "pgrads") if k in per_launch}
    dom = max(mfma_kernels, key=mfma_kernels.get)
    achieved = flops_one / (mfma_kernels[dom] * 1e-3) / 1e12
    flops_all = 3.0 * flops_one
    # bytes each contraction must move: valid rows of E and P in, its output out
    in_bytes = esize * V * (float(il.sum()) + float((ll + 1).sum()))
    out_bytes = {"lse": 4.0 * B * T * U1, "egrads": esize * B * T * V,
                 "pgrads": esize * B * U1 * V}
    hbm_gbs = (in_bytes + out_bytes[dom]) / (mfma_kernels[dom] * 1e-3) / 1e9
    out = {
        "metric": METRIC + (" (%s scores and gradients)" % io if bf16 else ""),
        "value": round(ms_per_step, 4),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": (round(ms_per_step / w["published_ms"], 5) if w.get("published_ms")
                        else None),
        "dtype": "f32 arithmetic on %s scores, %s gradients" % (io, io) if bf16 else "f32",
        "data": "synthetic",
        "config": {"workload": "%s: B=%d T=%d U=%d V=%d blank=0, %s scores, input_lengths "
                               "%s, label_lengths %s, deltas=1" %
                               (args.workload, B, T, w["U"], V,
                                "uniform [0,1)" if w.get("uniform") else "N(0,%g)" % w["sigma"],
                                "U[%d,%d]" % w["ragged_T"] if w["ragged_T"] else "=T",
                                "U[%d,%d]" % w["ragged_U"] if w["ragged_U"] else "=U"),
                   "seed": args.seed, "valid_lattice_cells": int(cells)},
        "roofline": {"bound": "mfma", "kernel": {"lse": "lse_stream_kernel",
                                                 "egrads": "egrads_stream_kernel",
                                                 "pgrads": "pgrads_stream_kernel"}[dom],
                     "achieved": round(achieved, 2), "peak": PEAK_FP32_MATRIX_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP32_MATRIX_TFLOPS, 4),
                     "traffic": RECORDED_TRAFFIC_BYTES.get(args.workload, {}).get(dom),
                     "kernel_ms": round(mfma_kernels[dom], 4),
                     "flops_per_launch": flops_one,
                     "hbm": {"achieved": round(hbm_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                             "frac": round(hbm_gbs / PEAK_HBM_GBS, 4),
                             "bytes_per_launch": in_bytes + out_bytes[dom]},
                     "all_kernels_frac_of_fp32_matrix_peak": {
                         k: round(flops_one / (v * 1e-3) / 1e12 / PEAK_FP32_MATRIX_TFLOPS, 4)
                         for k, v in mfma_kernels.items()}},
        "whole_step_frac_of_mfma_roofline": round(
            (flops_all / (PEAK_FP32_MATRIX_TFLOPS * 1e12)) / (ms_per_step * 1e-3), 4),
        "stage_ms_per_step": per_step,
    }
    if not args.no_cpu_baseline and not bf16:  # the CPU path has no bf16 form
        out["cpu_baseline"] = cpu_baseline(w, il, ll)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
