#!/usr/bin/env python3
"""Benchmark of the MI355X fused SwiGLU MLP forward: one JSON line on stdout.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3] [--no-cpu] [--no-configs] ...

A step is one whole forward Y = (silu(X @ Wg) * (X @ Wu)) @ Wd over one batch of seeded synthetic input that is
already resident in HBM: the gated dual-GEMM kernel followed by the down-projection kernel, both launched
through the C ABI (libfsw_hip.so) on torch's current stream. `value` is 6*M*d*ff FLOPs per step over the wall
time of exactly K steps between two device synchronisations. The default workload is the headline configuration
(Llama-3-8B MLP prefill: M=8192, d=4096, ff=14336, bf16, seed 2).

Extra objects on the same line:
  roofline     — the gate/up kernel (2/3 of the FLOPs): algorithmic FLOPs / its average duration, measured with
                 HIP events recorded around that launch inside the timed steps, against the bf16 dense MFMA peak;
                 `traffic` is read from the committed counter profile named in `traffic_source`;
  configs      — all five configurations, each forward timed call by call (events around one fsw_mlp call, a
                 512 MiB cache-defeating write before every timed call): median / p20 / p80 and roofline fraction;
  comparator   — the vendor GEMM (torch.mm, hipBLASLt) on the gate/up and down shapes of the workload, same run;
  ceilings     — what this board sustains with nothing in the way: a register-only MFMA loop with random operands
                 and a plain streaming read (fsw_probe_mfma / fsw_probe_read of libfsw_probe.so);
  decode       — the M=16 weight-streaming configuration in GB/s against the HBM3E peak: `value` in steady state on
                 one set of weights, `cold` alternating three copies of the weights (1.06 GB, beyond every cache);
  cpu_baseline — the same formulation in fp32 PyTorch on this host's cores (oracle/, the checker): whole forwards
                 of the workload; its result is also the parity check of the GPU's Y over every row.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "fused-swiglu_amd"))

MFMA_PEAK_TFLOPS = 2516.6  # MI355X dense bf16/fp16: 256 CU x 2.4 GHz x 4096 flop/clk/CU
HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
DECODE_WARMUP = 500        # untimed forwards before the HBM-bound (M = 16) measurements, ~30 ms
SETTLE_MS = 200.0          # untimed forwards before the timed steps of the compute-bound legs, whatever --warmup says:
                           # after an idle period the board's clock needs ~50 ms of load to settle (the first 30
                           # forwards run 10 % slower), and on some boxes the step time keeps falling by another
                           # 0.5 % over the next 100 ms; the reference's timer (bench_swiglu.py:102-106) warms up too
FLUSH_BYTES = 512 << 20    # written before every timed call of the per-configuration leg (Infinity Cache: 256 MB)
# counter profiles (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measurable in-process) that hold the line
# `traffic_bytes_per_launch = N` for the dominant kernel of a workload
TRAFFIC_PROFILES = {"C3": "profiles/pair16_gateup_C3_hbm_traffic_pmc.md", "C4": "profiles/decode_C4_hbm_traffic_pmc.md"}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="C3", choices=["C1", "C2", "C3", "C4", "C5"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--cpu-passes", type=int, default=3, help="timed whole forwards of the cpu_baseline leg")
    ap.add_argument("--no-configs", action="store_true", help="skip the per-configuration leg")
    ap.add_argument("--no-comparator", action="store_true", help="skip the vendor GEMM leg")
    ap.add_argument("--no-ceilings", action="store_true", help="skip the MFMA / read probes")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one elementwise copy of 1 GiB (reads 1 GiB, writes 1 GiB): the known-size kernel "
                         "that FETCH_SIZE / WRITE_SIZE counter runs are scaled by")
    ap.add_argument("--no-decode", action="store_true", help="skip the M=16 decode leg")
    ap.add_argument("--no-prepacked", action="store_true", help="skip the leg with weights blocked offline")
    return ap.parse_args()


def traffic_from_profile(workload):
    """(bytes per launch, profile path) from the committed counter profile of this workload, or (None, None)."""
    rel = TRAFFIC_PROFILES.get(workload)
    if not rel:
        return None, None
    try:
        m = re.search(r"traffic_bytes_per_launch\s*=\s*(\d+)", open(os.path.join(ROOT, rel)).read())
    except OSError:
        return None, None
    return (int(m.group(1)), rel) if m else (None, None)


def run_steps(capi, torch, g, cfg, steps, warmup, fused_entry=False, prepacked=False, weight_sets=None, settle_ms=0.0):
    """Times exactly `steps` forwards between two device synchronisations.
    fused_entry=False: a step is the launch sequence fsw_mlp enqueues for this shape, issued through the
    per-step entry points so that HIP events can be recorded around each launch inside the timed region: in the
    large-tile regime fsw_gateup_hblocked -> fsw_down_blocked (X row-major, H blocked in the workspace), otherwise
    fsw_gateup -> fsw_down. prepacked=True passes weights blocked once, outside the timed region, by
    fsw_prepack_w13 / fsw_prepack_w2.
    fused_entry=True: a step is one fsw_mlp call and ONE event pair brackets the whole timed region (an event
    record costs the stream ~4 us, which is 6 % of a 64 us decode step but 0.2 % of a prefill step); the per-step
    kernel time is then the bracketed time / steps, inter-launch gaps included. weight_sets: a list of (W13, W2)
    pairs used round-robin, step by step.
    settle_ms: untimed steps are issued until at least this much device time has gone by (and at least `warmup`).
    Returns (wall seconds, [ms of gate/up], [ms of down], Y, [0.0], info) with info =
    {"settle_steps", "settle_ms", "step_ms": per-step device time from the step's first to its last event}."""
    import fsw_capi
    L = capi.lib()
    M, d, ff = cfg["M"], cfg["d"], cfg["ff"]
    code = fsw_capi.dtype_code(g["X"])
    Y = torch.empty((M, d), dtype=g["X"].dtype, device=g["X"].device)
    ws_bytes = L.fsw_mlp_workspace_bytes(code, M, d, ff)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=g["X"].device)
    h_bytes = (M * ff * 2 + 255) // 256 * 256
    hb_bytes = L.fsw_blocked_bytes(M, ff)
    blocked = (not fused_entry) and capi.variant_name(0, code, M, 2 * ff, d) == "pair16_256x256" and ws_bytes == hb_bytes
    stream = torch.cuda.current_stream().cuda_stream
    xp, wp, w2p, yp, wsp = (t.data_ptr() for t in (g["X"], g["W13"], g["W2"], Y, ws))
    sets = [(a.data_ptr(), b.data_ptr()) for a, b in weight_sets] if weight_sets else [(wp, w2p)]
    ldw, ldw2, wflag = d, ff, 0
    if prepacked:
        if not blocked:
            raise RuntimeError("prepacked weights are only used in the large-tile regime")
        w13b, w2b = capi.block_rows(g["W13"], "w13"), capi.block_rows(g["W2"], "w2")
        wp, w2p, ldw, ldw2, wflag = w13b.data_ptr(), w2b.data_ptr(), 0, 0, 1

    def step(ev, i):
        if fused_entry:
            a, b = sets[i % len(sets)]
            rc = L.fsw_mlp(code, M, d, ff, xp, d, a, d, b, ff, yp, d, wsp, ws_bytes, stream)
            rc2 = rc3 = 0
        elif blocked:
            ev[0].record()
            rc = L.fsw_gateup_hblocked(code, M, 2 * ff, d, xp, d, wp, ldw, wflag, wsp, stream)
            ev[1].record()
            rc2 = L.fsw_down_blocked(code, M, d, ff, wsp, w2p, ldw2, wflag, yp, d, stream)
            ev[2].record()
            rc3 = 0
        else:
            ev[0].record()
            rc = L.fsw_gateup(code, M, 2 * ff, d, xp, d, wp, d, wsp, ff, stream)
            ev[1].record()
            rc2 = L.fsw_down(code, M, d, ff, wsp, ff, w2p, ff, yp, d, wsp + h_bytes, ws_bytes - h_bytes, stream)
            ev[2].record()
            rc3 = 0
        if rc or rc2 or rc3:
            raise RuntimeError("fsw launch failed: %s / %s / %s" % (capi.strerror(rc), capi.strerror(rc2), capi.strerror(rc3)))

    events = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(steps + min(warmup, 16))]
    region = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    spare = events[steps:] or [[torch.cuda.Event(enable_timing=True) for _ in range(4)]]
    settle = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    settle[0].record()
    done, settled = 0, 0.0
    while done < warmup or settled < settle_ms:
        for _ in range(8 if done >= warmup else min(8, warmup - done)):
            step(spare[done % len(spare)], done)
            done += 1
        settle[1].record()
        settle[1].synchronize()
        settled = settle[0].elapsed_time(settle[1])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    region[0].record()
    for i in range(steps):
        step(events[i], i)
    region[1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    info = {"settle_steps": done, "settle_ms": round(settled, 2), "blocked": blocked}
    if fused_entry:
        return wall, [region[0].elapsed_time(region[1]) / steps], [0.0], Y, [0.0], info
    first = [e[0].elapsed_time(e[1]) for e in events[:steps]]
    second = [e[1].elapsed_time(e[2]) for e in events[:steps]]
    info["step_ms"] = [e[0].elapsed_time(e[2]) for e in events[:steps]]
    return wall, first, second, Y, [0.0], info


def quantiles(xs):
    s = sorted(xs)
    pick = lambda q: s[min(len(s) - 1, int(q * (len(s) - 1) + 0.5))]
    return pick(0.5), pick(0.2), pick(0.8)


def timed_calls(torch, fn, flush, min_calls=10, budget_ms=150.0):
    """ms per call (median, p20, p80) of `fn`, each call bracketed by events on the current stream and, when
    `flush` is a tensor, preceded by a write over it; the timing semantics of the reference's benchmark
    (bench_swiglu.py:102-106: one untimed call, an estimate from 5, then ~100 ms of timed calls)."""
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        fn()
    e1.record()
    torch.cuda.synchronize()
    est = max(e0.elapsed_time(e1) / 5, 1e-3)
    n = max(min_calls, min(400, int(budget_ms / est)))
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for a, b in pairs:
        if flush is not None:
            flush.zero_()
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return quantiles([a.elapsed_time(b) for a, b in pairs]) + (n,)


def device_inputs(torch, cfg_tuple, n_weight_sets=1):
    """Inputs of a configuration drawn on the device with the configuration's law (X ~ x_scale N(0,1),
    W ~ N(0,1) / sqrt(fan_in), packed as the reference packs them). For timing only: the seeded CPU inputs of the
    parity tests take minutes to draw for the largest configuration."""
    name, M, d, ff, dtype, seed, xs = cfg_tuple
    g = torch.Generator(device="cuda:0").manual_seed(seed)
    X = (torch.randn((M, d), device="cuda:0", generator=g) * xs).to(dtype)
    sets = []
    for _ in range(n_weight_sets):
        W13 = (torch.randn((2 * ff, d), device="cuda:0", generator=g) / d ** 0.5).to(dtype)
        W2 = (torch.randn((d, ff), device="cuda:0", generator=g) / ff ** 0.5).to(dtype)
        sets.append((W13, W2))
    return X, sets


def configs_leg(capi, torch, fsw_weights):
    """Every configuration: one fsw_mlp call per timed call, caches defeated before each. The two events that bracket
    a call cost the stream a few microseconds of their own (an EMPTY bracket behind the same flush is timed here and
    reported as `event_pair_overhead_ms`): nothing for a millisecond forward, 8 % of a 60 us decode forward. `ms_median`
    and `frac` are the raw bracket; `ms_net` / `frac_net` have the empty bracket's median subtracted."""
    out = {}
    flush = torch.empty(FLUSH_BYTES, dtype=torch.uint8, device="cuda:0")
    overhead = timed_calls(torch, lambda: None, flush, min_calls=100, budget_ms=1.0)[0]
    for tup in fsw_weights.CONFIGS:
        name, M, d, ff, dtype, seed, xs = tup
        X, sets = device_inputs(torch, tup)
        W13, W2 = sets[0]
        Y = torch.empty((M, d), dtype=dtype, device="cuda:0")
        ws = capi.mlp_workspace(X, ff)
        fn = lambda: capi.mlp(X, W13, W2, out=Y, workspace=ws)
        med, p20, p80, n = timed_calls(torch, fn, flush)
        flops, nbytes = fsw_weights.flops(M, d, ff), fsw_weights.hbm_bytes(M, d, ff)
        rec = {"M": M, "d": d, "ff": ff, "dtype": "bf16" if dtype == torch.bfloat16 else "fp16", "calls": n,
               "ms_median": round(med, 5), "ms_p20": round(p20, 5), "ms_p80": round(p80, 5),
               "tflops": round(flops / med / 1e9, 2), "gbs": round(nbytes / med / 1e6, 2),
               "kernels": "%s + %s" % (capi.variant_name(0, 0, M, 2 * ff, d), capi.variant_name(2, 0, M, d, ff))}
        net = max(med - overhead, 1e-6)
        rec["ms_net"] = round(net, 5)
        if name == "C4":
            rec.update(bound="hbm", frac=round(nbytes / med / 1e6 / HBM_PEAK_GBS, 4),
                       frac_net=round(nbytes / net / 1e6 / HBM_PEAK_GBS, 4))
        elif name == "C1":
            rec.update(bound="latency", frac=round(flops / med / 1e9 / MFMA_PEAK_TFLOPS, 4),
                       frac_net=round(flops / net / 1e9 / MFMA_PEAK_TFLOPS, 4))
        else:
            rec.update(bound="mfma", frac=round(flops / med / 1e9 / MFMA_PEAK_TFLOPS, 4),
                       frac_net=round(flops / net / 1e9 / MFMA_PEAK_TFLOPS, 4))
        out[name] = rec
        del X, sets, W13, W2, Y, ws
    out["event_pair_overhead_ms"] = round(overhead, 5)
    out["method"] = ("fsw_mlp, one call per timed call, events around the call, %d MiB written before each; inputs "
                     "drawn on the device with each configuration's law; ms_median / frac are the raw bracket, "
                     "ms_net / frac_net subtract the median of an empty bracket behind the same flush "
                     "(event_pair_overhead_ms)" % (FLUSH_BYTES >> 20))
    return out


def comparator_leg(torch, g, cfg, fsw_weights, steps, warmup, settle_ms):
    """hipBLASLt through torch.mm on the two GEMM shapes of the workload (no gating, C written at full width), timed
    the way `value` is: the same settling period and warm-up steps, then exactly `steps` back-to-back pairs of GEMMs
    between two device synchronisations, events around each GEMM inside the timed region."""
    M, d, ff = cfg["M"], cfg["d"], cfg["ff"]
    X, W13, W2 = g["X"], g["W13"], g["W2"]
    C = torch.empty((M, 2 * ff), dtype=X.dtype, device=X.device)
    H = torch.randn((M, ff), device=X.device).to(X.dtype)
    Y = torch.empty((M, d), dtype=X.dtype, device=X.device)
    w13t, w2t = W13.t(), W2.t()

    def step(ev):
        ev[0].record()
        torch.mm(X, w13t, out=C)
        ev[1].record()
        torch.mm(H, w2t, out=Y)
        ev[2].record()

    mk = lambda: [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    spare, settle = mk(), [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    settle[0].record()
    done, settled = 0, 0.0
    while done < warmup or settled < settle_ms:
        for _ in range(8 if done >= warmup else min(8, warmup - done)):
            step(spare)
            done += 1
        settle[1].record()
        settle[1].synchronize()
        settled = settle[0].elapsed_time(settle[1])
    events = [mk() for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for ev in events:
        step(ev)
    torch.cuda.synchronize()
    both = (time.perf_counter() - t0) / steps * 1e3
    gu = quantiles([e[0].elapsed_time(e[1]) for e in events])
    dn = quantiles([e[1].elapsed_time(e[2]) for e in events])
    return {"what": "torch.mm (hipBLASLt) on the gate/up [M,d]x[d,2ff] and down [M,ff]x[ff,d] shapes, no gating kernel; "
                    "timed like `value`: %.0f ms (%d steps) of settling, then %d back-to-back steps between two "
                    "synchronisations" % (settled, done, steps),
            "gateup_ms_median": round(gu[0], 5), "gateup_tflops": round(4 * M * d * ff / gu[0] / 1e9, 2),
            "down_ms_median": round(dn[0], 5), "down_tflops": round(2 * M * d * ff / dn[0] / 1e9, 2),
            "two_gemms_ms": round(both, 5), "two_gemms_tflops": round(fsw_weights.flops(M, d, ff) / both / 1e9, 2)}


def ceilings_leg(capi, torch):
    """Register-only MFMA loop (random bf16 operands) and a plain streaming read, through the measurement
    kernels of libfsw_probe.so (include/fsw_probe.h)."""
    L = capi.probe_lib()
    stream = torch.cuda.current_stream().cuda_stream
    ops = torch.randn(8192, device="cuda:0").to(torch.bfloat16)          # 16 KB of N(0,1) operands
    outb = torch.empty(256 * 256, dtype=torch.float32, device="cuda:0")
    iters = 20000                                                         # 256 x 4 waves x 20000 x 64 MFMAs ~ 12 ms
    fl = 256 * 4 * iters * 64 * 16384

    def mfma():
        capi.check(L.fsw_probe_mfma(0, iters, ops.data_ptr(), outb.data_ptr(), 256, stream))
    m = timed_calls(torch, mfma, None, min_calls=8, budget_ms=120.0)
    src = torch.empty(3 * (353 << 20), dtype=torch.uint8, device="cuda:0")  # 1.06 GB: beyond the Infinity Cache
    src.fill_(1)
    flag = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    warm_bytes = 353 << 20

    def read_warm():
        capi.check(L.fsw_probe_read(src.data_ptr(), warm_bytes, flag.data_ptr(), 2048, stream))

    def read_cold():
        capi.check(L.fsw_probe_read(src.data_ptr(), src.numel(), flag.data_ptr(), 2048, stream))
    for _ in range(100):
        read_warm()
    rw = timed_calls(torch, read_warm, None, min_calls=50, budget_ms=60.0)
    rc = timed_calls(torch, read_cold, None, min_calls=20, budget_ms=60.0)
    return {"mfma_sustained_tflops": round(fl / m[0] / 1e9, 1),
            "mfma_sustained_frac_of_peak": round(fl / m[0] / 1e9 / MFMA_PEAK_TFLOPS, 4),
            "mfma_probe": "register-only v_mfma_f32_16x16x32_bf16 loop, N(0,1) operands, 256 workgroups x 4 waves, "
                          "median of %d launches of %.1f ms" % (m[3], m[0]),
            "read_353MB_repeated_gbs": round(warm_bytes / rw[0] / 1e6, 1),
            "read_1059MB_gbs": round(src.numel() / rc[0] / 1e6, 1),
            "read_probe": "non-temporal 16-byte loads, 2048 workgroups; 353 MB re-read back to back, and 1059 MB "
                          "(beyond the 256 MB Infinity Cache) per launch"}


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(torch, inp, cfg, passes, y_gpu):
    """The fp32 PyTorch formulation on the host cores: one warm-up block, then `passes` whole forwards of the
    workload. The last result is the reference for a parity check of every row of the GPU's Y. `cores` is the
    number of threads torch actually runs (OMP_NUM_THREADS where the host sets it: a one-GPU share of a larger
    machine), `host_cpus` what the machine shows."""
    from oracle import oracle
    import fsw_weights
    M, d, ff = cfg["M"], cfg["d"], cfg["ff"]
    threads = torch.get_num_threads()
    X, W13f, W2f = inp["X"].float(), inp["W13"].float(), inp["W2"].float()  # upcast once, outside the timed passes
    oracle.ref_mlp(X[:64], W13f, W2f)  # warm-up
    times, Yref = [], None
    for _ in range(max(passes, 1)):
        t0 = time.perf_counter()
        Yref = oracle.ref_mlp(X, W13f, W2f)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    parity = oracle.error_metrics(y_gpu, Yref)
    parity["rows"] = M
    parity["pass"] = bool(oracle.passes(parity))
    base = {"value": round(fsw_weights.flops(M, d, ff) / med / 1e12, 4), "unit": "TFLOP/s", "cores": threads,
            "host_cpus": os.cpu_count(), "cpu_model": cpu_model(), "kind": "port",
            "sample": "%d whole forwards of %s (all %d rows) by the fp32 torch formulation, median %.2f s of %s" % (
                len(times), cfg["name"], M, med, ["%.2f" % t for t in times])}
    return base, parity


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus %d is not supported (the path shards over rows or "
              "over ff with one all-reduce, which is not part of this build)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    import fsw_capi as capi
    import fsw_weights
    capi.lib()
    torch.cuda.set_device(0)

    def load(name):
        inp = fsw_weights.make_config(name)
        g = {k: inp[k].to("cuda:0") for k in ("X", "W13", "W2")}
        return inp, g

    inp, g = load(args.workload)
    cfg = {k: inp[k] for k in ("name", "M", "d", "ff", "seed")}
    M, d, ff = cfg["M"], cfg["d"], cfg["ff"]
    dtype_name = "bf16" if inp["dtype"] == torch.bfloat16 else "fp16"
    hbm_bound = args.workload == "C4"
    # The HBM-bound workload is timed in steady state: after an idle period the first ~20 ms of forwards run
    # 3-5 % slower (measured: 61.8 us/step after 20 warm-up steps, 59.0 after 200, 58.4 after 1000), so its warm-up
    # is at least DECODE_WARMUP steps of ~60 us.
    if hbm_bound:
        args.warmup = max(args.warmup, DECODE_WARMUP)
    settle_ms = 0.0 if hbm_bound else SETTLE_MS
    wall, gu, dn, Y, pre, info = run_steps(capi, torch, g, cfg, args.steps, args.warmup, fused_entry=hbm_bound,
                                           settle_ms=settle_ms)
    pre_ms = sum(pre) / len(pre)
    blocked = info["blocked"]
    ms_per_step = wall / args.steps * 1e3
    tflops = fsw_weights.flops(M, d, ff) / (ms_per_step * 1e-3) / 1e12
    gu_ms, dn_ms = sum(gu) / len(gu), max(sum(dn) / len(dn), 1e-9)
    gu_tflops = fsw_weights.gateup_flops(M, d, ff) / (gu_ms * 1e-3) / 1e12
    dn_tflops = 0.0 if hbm_bound else 2 * M * d * ff / (dn_ms * 1e-3) / 1e12
    traffic, traffic_src = traffic_from_profile(args.workload)
    if hbm_bound:
        all_bytes = fsw_weights.hbm_bytes(M, d, ff)
        roofline = {"bound": "hbm", "kernel": "%s gate/up + %s down (whole forward, two launches)" % (
                        capi.variant_name(0, 0, M, 2 * ff, d), capi.variant_name(2, 0, M, d, ff)),
                    "achieved": round(all_bytes / (gu_ms * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(all_bytes / (gu_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                    "traffic": traffic, "traffic_source": traffic_src, "algorithmic_bytes": all_bytes,
                    "avg_kernel_ms": round(gu_ms, 5)}
    else:
        kname = capi.variant_name(0, 0, M, 2 * ff, d) + (" (v_mfma_f32_16x16x32), X row-major, H panel-blocked" if blocked else "")
        roofline = {"bound": "mfma", "kernel": kname + " (gate/up)",
                    "achieved": round(gu_tflops, 2), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(gu_tflops / MFMA_PEAK_TFLOPS, 4),
                    "traffic": traffic, "traffic_source": traffic_src,
                    "algorithmic_flops": fsw_weights.gateup_flops(M, d, ff),
                    "algorithmic_bytes": (2 * ff * d + M * d + M * ff) * 2, "avg_kernel_ms": round(gu_ms, 5),
                    "kernel_ms_median_p20_p80": [round(v, 5) for v in quantiles(gu)]}
    out = {
        "metric": "fused SwiGLU fwd TFLOP/s + %% bf16 MFMA peak (M=%d,d=%d,ff=%d)" % (M, d, ff),
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "ms_per_step_median": round(quantiles(info["step_ms"])[0], 5) if "step_ms" in info else round(ms_per_step, 5),
        "settle_ms": info["settle_ms"], "settle_steps": info["settle_steps"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype_name, "data": "synthetic",
        "config": {"workload": "%s: SwiGLU MLP forward M=%d d=%d ff=%d %s seed %d" % (
            cfg["name"], M, d, ff, dtype_name, cfg["seed"]), "M": M, "d": d, "ff": ff},
        "frac_of_mfma_peak": round(tflops / MFMA_PEAK_TFLOPS, 4),
        "kernels": {"gateup_ms": round(gu_ms, 5), "gateup_ms_median": round(quantiles(gu)[0], 5),
                    "gateup_tflops": round(gu_tflops, 2), "down_ms": round(dn_ms, 5),
                    "down_tflops": round(dn_tflops, 2),
                    "hbm_gbs": round(fsw_weights.hbm_bytes(M, d, ff) / (ms_per_step * 1e-3) / 1e9, 2)},
        "roofline": roofline,
    }

    if args.copy_probe:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst

    if not hbm_bound and not args.no_comparator:
        out["comparator"] = comparator_leg(torch, g, cfg, fsw_weights, args.steps, args.warmup, settle_ms)
        out["comparator"]["value_over_two_gemms"] = round(tflops / out["comparator"]["two_gemms_tflops"], 4)

    # decode leg: M = 16, weight streaming, judged in GB/s: steady state on one set of weights, and cold
    if args.workload != "C4" and not args.no_decode:
        tup = [c for c in fsw_weights.CONFIGS if c[0] == "C4"][0]
        X4, sets4 = device_inputs(torch, tup, n_weight_sets=3)
        c4 = {"name": "C4", "M": tup[1], "d": tup[2], "ff": tup[3], "seed": tup[5]}
        g4 = {"X": X4, "W13": sets4[0][0], "W2": sets4[0][1]}
        by4 = fsw_weights.hbm_bytes(c4["M"], c4["d"], c4["ff"])
        wall4, k4, _, _, _, _ = run_steps(capi, torch, g4, c4, 200, DECODE_WARMUP, fused_entry=True)
        wallc, kc, _, _, _, _ = run_steps(capi, torch, g4, c4, 201, DECODE_WARMUP, fused_entry=True, weight_sets=sets4)
        ms4, msc = wall4 / 200 * 1e3, wallc / 201 * 1e3
        k4_ms, kc_ms = sum(k4) / len(k4), sum(kc) / len(kc)
        traffic4, traffic4_src = traffic_from_profile("C4")
        kern4 = "%s gate/up + %s down" % (capi.variant_name(0, 0, c4["M"], 2 * c4["ff"], c4["d"]),
                                          capi.variant_name(2, 0, c4["M"], c4["d"], c4["ff"]))
        out["decode"] = {
            "workload": "C4: M=16 d=4096 ff=14336 bf16", "entry": "fsw_mlp (one call, two launches)",
            "warmup_steps": DECODE_WARMUP, "steps": 200,
            "ms_per_step": round(ms4, 5), "value": round(by4 / (ms4 * 1e-3) / 1e9, 2), "unit": "GB/s",
            "peak": HBM_PEAK_GBS, "frac": round(by4 / (ms4 * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "note": "steady state: the same 353 MB of weights every step (256 MB Infinity Cache: partly resident)",
            "roofline": {"bound": "hbm", "kernel": kern4, "achieved": round(by4 / (k4_ms * 1e-3) / 1e9, 2),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(by4 / (k4_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                         "traffic": traffic4, "traffic_source": traffic4_src, "avg_kernel_ms": round(k4_ms, 5)},
            "cold": {"weight_sets": 3, "working_set_bytes": 3 * (by4 - 2 * 16 * (c4["d"] + c4["ff"]) * 2),
                     "warmup_steps": DECODE_WARMUP, "steps": 201, "ms_per_step": round(msc, 5),
                     "value": round(by4 / (msc * 1e-3) / 1e9, 2), "unit": "GB/s",
                     "frac": round(by4 / (msc * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "kernel_frac": round(by4 / (kc_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "note": "three copies of W13 / W2 used round-robin: 1.06 GB between two uses of a byte, so no "
                             "cache level can serve the weights"}}
        del X4, sets4, g4

    if not args.no_ceilings:
        out["ceilings"] = ceilings_leg(capi, torch)
        if not hbm_bound:
            out["ceilings"]["gateup_kernel_over_mfma_sustained"] = round(gu_tflops / out["ceilings"]["mfma_sustained_tflops"], 4)

    # the same forward with the weights blocked once, offline (fsw_prepack_w13 / fsw_prepack_w2): reported beside
    # `value`, which stays on the reference's weight layout
    if blocked and not args.no_prepacked:
        wallp, gup, dnp, Yp, prep, _ = run_steps(capi, torch, g, cfg, args.steps, args.warmup, prepacked=True,
                                                 settle_ms=settle_ms)
        msp = wallp / args.steps * 1e3
        out["prepacked_weights"] = {
            "ms_per_step": round(msp, 5), "value": round(fsw_weights.flops(M, d, ff) / (msp * 1e-3) / 1e12, 2),
            "unit": "TFLOP/s", "gateup_ms": round(sum(gup) / len(gup), 5), "down_ms": round(sum(dnp) / len(dnp), 5),
            "max_abs_vs_row_major_weights": round((Yp.float() - Y.float()).abs().max().item(), 6)}

    if not args.no_configs:
        out["configs"] = configs_leg(capi, torch, fsw_weights)

    if not args.no_cpu:
        base, parity = cpu_baseline(torch, inp, cfg, args.cpu_passes, Y.cpu())
        out["cpu_baseline"] = base
        out["parity_check"] = {k: (round(v, 6) if isinstance(v, float) else v) for k, v in parity.items()}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
