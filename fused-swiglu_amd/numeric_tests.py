#!/usr/bin/env python3
"""Numerical check of `fused_mlp_module.fused_swiglu_bf16` against PyTorch's own bf16 formulation on the GPU.

Counterpart of the reference's numeric_tests.py: same sizes (M = N = K in 1024 ... 65536), same input law
(every element ~ U(-1/sqrt(K), +1/sqrt(K)), which is what kaiming_uniform_(a=sqrt(5)) leaves in a [rows, K] tensor,
numeric_tests.py:8-10,35-38), same three statistics per trial (max |d|, mean |d|, ||d||_F / ||ref||_F,
numeric_tests.py:49-52) and the same table of p20 / p80 / mean / std over the trials (numeric_tests.py:54-76).
Unlike the reference it can be seeded, sized from the command line, and it also reports the error against an
fp32 evaluation of the formulation (the bf16 torch result carries three roundings of its own).

  python numeric_tests.py                      # the reference's sweep, 100 trials per size
  python numeric_tests.py --sizes 1024 4096 --iterations 10 --seed 0
"""
import argparse
import math
import sys

import numpy as np
import torch
import torch.nn.functional as F

REFERENCE_SIZES = [1024, 2048, 4096, 8192, 16384, 32768, 65536]


def uniform_like_kaiming(rows, k, device, generator):
    bound = 1.0 / math.sqrt(k)  # gain sqrt(2 / (1 + 5)) * sqrt(3 / fan_in) with fan_in = K
    t = torch.empty((rows, k), device=device, dtype=torch.float32)
    t.uniform_(-bound, bound, generator=generator)
    return t.to(torch.bfloat16)


def torch_formulation(a, b, dtype=None):
    """C = A @ B.T; gated = C[:, ::2] * silu(C[:, 1::2]) at the tensors' own precision, or at `dtype`."""
    if dtype is not None:
        a, b = a.to(dtype), b.to(dtype)
    c = a @ b.T
    return c[:, ::2] * F.silu(c[:, 1::2])


def trial_stats(out, ref):
    diff = out.float() - ref.float()
    return diff.abs().max().item(), diff.abs().mean().item(), (diff.norm() / ref.float().norm()).item()


def run(sizes, iterations, seed=None, device="cuda:0", fp32_rows=512, out=sys.stdout):
    import fused_mlp_module
    gen = torch.Generator(device=device)
    if seed is not None:
        gen.manual_seed(seed)
    header = "%8s | %22s | %15s | %15s | %15s | %15s" % ("MNK", "Metric", "20th Percentile", "80th Percentile",
                                                        "Mean", "Std Dev")
    print(header, file=out)
    print("-" * len(header), file=out)
    results = {}
    for mnk in sizes:
        m = n = k = mnk
        cols = {"Max Abs Diff": [], "Mean Abs Diff": [], "Relative Diff": [], "Relative Diff vs fp32": []}
        for _ in range(iterations):
            a = uniform_like_kaiming(m, k, device, gen)
            b = uniform_like_kaiming(n, k, device, gen)
            mine = fused_mlp_module.fused_swiglu_bf16(a, b)
            theirs = torch_formulation(a, b)
            mx, mean, rel = trial_stats(mine, theirs)
            cols["Max Abs Diff"].append(mx)
            cols["Mean Abs Diff"].append(mean)
            cols["Relative Diff"].append(rel)
            rows = min(m, fp32_rows)  # fp32 evaluation on a row block keeps the 65536 case in memory
            exact = torch_formulation(a[:rows], b, torch.float32)
            cols["Relative Diff vs fp32"].append(trial_stats(mine[:rows], exact)[2])
            del a, b, mine, theirs, exact
        results[mnk] = {}
        for metric, values in cols.items():
            v = np.array(values)
            results[mnk][metric] = (np.percentile(v, 20), np.percentile(v, 80), v.mean(), v.std())
            print("%8d | %22s | %15.6e | %15.6e | %15.6e | %15.6e" % ((mnk, metric) + results[mnk][metric]), file=out)
    return results


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--sizes", type=int, nargs="+", default=REFERENCE_SIZES)
    ap.add_argument("--iterations", type=int, default=100)
    ap.add_argument("--seed", type=int, default=None, help="seed of the input generator (the reference is unseeded)")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        sys.exit("numeric_tests.py needs the GPU: the extension has no CPU path")
    run(args.sizes, args.iterations, args.seed)


if __name__ == "__main__":
    main()
