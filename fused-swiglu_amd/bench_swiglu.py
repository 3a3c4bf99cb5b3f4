#!/usr/bin/env python3
"""TFLOP/s of the fused gate/up SwiGLU kernel against a library GEMM followed by an eager gating kernel.

Counterpart of the reference's bench_swiglu.py: the "Gated MLP for Llama 70B" sweep (K = 8192, N = 2 * 28672,
Tokens in 512 ... 65536, bench_swiglu.py:52-60,84-86), bf16 randn inputs (:88-89), a [M, N] output buffer handed
to `swiglu_fwd_bf16` with ldC = N (:91,106), the FLOP convention M*N*(2K-1) + 6*M*N/2 (:112-117) and
median / p20 / p80 timing with the L2 defeated before every timed call (the semantics of the timer the reference
uses). The comparator here is hipBLASLt/rocBLAS through torch.mm plus an eager `C[:, :N/2] * silu(C[:, N/2:])`
(split halves, as the reference's comparator, :34-38); there is no Triton dependency and no plot, the table is
printed and optionally written as CSV.

  python bench_swiglu.py                         # full sweep
  python bench_swiglu.py --tokens 512 4096 --csv results.csv
  python bench_swiglu.py --forward --k 4096 --n 28672 --tokens 128 1024   # also the whole MLP forward (with the
                                                 # down projection [K, N/2]) against mm + eager gating + mm
"""
import argparse
import sys

import torch
import torch.nn.functional as F

REFERENCE_TOKENS = [512, 1024, 2048, 4096, 8192, 16384, 32768, 49152, 65536]
K_DEFAULT, N_DEFAULT = 8192, 28672 * 2


def reference_flops(m, n, k):
    return m * n * (2 * k - 1) + 6 * m * (n // 2)


def timed(fn, flush, warmup_ms=25.0, rep_ms=100.0):
    """Median, p20, p80 in ms over ~rep_ms of calls, each preceded by a write over `flush` (larger than the
    256 MB Infinity Cache) and bracketed by events."""
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        flush.zero_()
        fn()
    e1.record()
    torch.cuda.synchronize()
    est = max(e0.elapsed_time(e1) / 5, 1e-3)
    n_warm, n_rep = max(1, int(warmup_ms / est)), max(3, min(1000, int(rep_ms / est)))
    for _ in range(n_warm):
        fn()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
    for s, e in zip(starts, ends):
        flush.zero_()
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    t = torch.tensor([s.elapsed_time(e) for s, e in zip(starts, ends)], dtype=torch.float64)
    q = torch.quantile(t, torch.tensor([0.5, 0.2, 0.8], dtype=torch.float64))
    return q[0].item(), q[1].item(), q[2].item()


def run(tokens, k=K_DEFAULT, n=N_DEFAULT, device="cuda:0", out=sys.stdout, csv=None, forward=False):
    import fused_mlp_module
    flush = torch.empty(512 << 20, dtype=torch.uint8, device=device)
    rows = []
    print("%8s | %-18s | %10s | %10s | %10s | %10s" % ("Tokens", "provider", "ms", "TFLOP/s", "low", "high"), file=out)
    for m in tokens:
        a = torch.randn((m, k), dtype=torch.bfloat16, device=device)
        b = torch.randn((n, k), dtype=torch.bfloat16, device=device)
        c = torch.zeros((m, n), dtype=torch.bfloat16, device=device)
        c2 = torch.empty((m, n), dtype=torch.bfloat16, device=device)
        bt = b.T

        def fused():
            fused_mlp_module.swiglu_fwd_bf16(m, n, k, a, k, b, k, c, n)

        def library_plus_eager():
            torch.mm(a, bt, out=c2)
            return c2[:, : n // 2] * F.silu(c2[:, n // 2:])

        legs = [("hipBLASLt+eager", library_plus_eager, reference_flops(m, n, k)), ("Fused", fused, reference_flops(m, n, k))]
        if forward:
            w2 = torch.randn((k, n // 2), dtype=torch.bfloat16, device=device) / (n // 2) ** 0.5
            w2t = w2.T
            y = torch.empty((m, k), dtype=torch.bfloat16, device=device)
            fwd_flops = reference_flops(m, n, k) + m * k * (n - 1)

            def fused_forward():
                return fused_mlp_module.fused_swiglu_mlp_bf16(a, b, w2)

            def library_forward():
                torch.mm(a, bt, out=c2)
                return torch.mm(c2[:, : n // 2] * F.silu(c2[:, n // 2:]), w2t, out=y)

            legs += [("hipBLASLt forward", library_forward, fwd_flops), ("Fused forward", fused_forward, fwd_flops)]
        for name, fn, flops in legs:
            ms, lo, hi = timed(fn, flush)
            tf = lambda t: flops * 1e-12 / (t * 1e-3)
            rows.append((m, name, ms, tf(ms), tf(hi), tf(lo)))
            print("%8d | %-18s | %10.4f | %10.1f | %10.1f | %10.1f" % rows[-1], file=out)
        del a, b, c, c2, bt
    if csv:
        with open(csv, "w") as f:
            f.write("Tokens,provider,ms,tflops,tflops_low,tflops_high\n")
            for r in rows:
                f.write("%d,%s,%.6f,%.3f,%.3f,%.3f\n" % r)
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--tokens", type=int, nargs="+", default=REFERENCE_TOKENS)
    ap.add_argument("--k", type=int, default=K_DEFAULT)
    ap.add_argument("--n", type=int, default=N_DEFAULT, help="full N = 2 * ff")
    ap.add_argument("--csv", default=None)
    ap.add_argument("--forward", action="store_true", help="also time the whole forward, down projection included")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        sys.exit("bench_swiglu.py needs the GPU: the extension has no CPU path")
    run(args.tokens, args.k, args.n, csv=args.csv, forward=args.forward)


if __name__ == "__main__":
    main()
