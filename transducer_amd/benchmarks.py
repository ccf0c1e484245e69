"""The reference's benchmark grid through the Python front end.

Same protocol as the reference's ``benchmarks/torch_benchmarks.py`` (:8-20 five untimed calls
then ten timed ones with a device synchronisation after each; :26-35 uniform [0,1) scores,
labels in [1,V), every utterance at full length; :100-105 B in {8,32}, T=2000, U=100,
V in {100,1000,2000,10000}), so its lines can be set beside the table in the reference's
README.  The backward figure repeats ``loss.backward(retain_graph=True)`` on one forward, as
the reference does.

    python -m transducer_amd.benchmarks [--json] [--viterbi]
"""
import argparse
import itertools
import json
import time

import torch

from . import TransducerLoss


def timefunc(fn, iters=10, warmup=5):
    for _ in range(warmup):
        fn()
        torch.cuda.synchronize()
    start = time.time()
    for _ in range(iters):
        fn()
        torch.cuda.synchronize()
    return (time.time() - start) * 1e3 / iters


def time_shape(B, T, U, V, viterbi=False):
    device = torch.device("cuda")
    emissions = torch.rand((B, T, V), device=device, dtype=torch.float32)
    predictions = torch.rand((B, U + 1, V), device=device, dtype=torch.float32)
    labels = torch.randint(low=1, high=V, size=(B, U), device=device, dtype=torch.int32)
    input_lengths = torch.full((B,), T, device=device, dtype=torch.int32)
    label_lengths = torch.full((B,), U, device=device, dtype=torch.int32)
    criterion = TransducerLoss()
    out = {"B": B, "T": T, "U": U, "V": V}

    out["forward_ms"] = timefunc(
        lambda: criterion(emissions, predictions, labels, input_lengths, label_lengths))
    if viterbi:
        out["viterbi_ms"] = timefunc(
            lambda: criterion.viterbi(emissions, predictions, input_lengths, label_lengths))

    emissions.requires_grad = True
    predictions.requires_grad = True
    loss = criterion(emissions, predictions, labels, input_lengths, label_lengths).sum()

    def backward():
        emissions.grad = None
        predictions.grad = None
        loss.backward(retain_graph=True)

    out["backward_ms"] = timefunc(backward)
    out["total_ms"] = out["forward_ms"] + out["backward_ms"]
    return out


def main():
    parser = argparse.ArgumentParser(description="Benchmark grid of the reference's README")
    parser.add_argument("--json", action="store_true", help="one JSON object per shape")
    parser.add_argument("--viterbi", action="store_true", help="also time criterion.viterbi")
    args = parser.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("transducer_amd.benchmarks needs a HIP device")
    for B, T, U, V in itertools.product([8, 32], [2000], [100], [100, 1000, 2000, 10000]):
        r = time_shape(B, T, U, V, viterbi=args.viterbi)
        if args.json:
            print(json.dumps(r), flush=True)
        else:
            print("Timing shape ({}, {}, {}, {})".format(B, T, U, V))
            line = "transducer: forward {:.3f}, backward {:.3f}, total {:.3f}".format(
                r["forward_ms"], r["backward_ms"], r["total_ms"])
            if args.viterbi:
                line += ", viterbi {:.3f}".format(r["viterbi_ms"])
            print(line, flush=True)


if __name__ == "__main__":
    main()
