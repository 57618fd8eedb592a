#!/usr/bin/env python3
"""Benchmark of the sampling hot path on one MI355X.

A "step" is one pass of the sampler over one batch of synthetic logits already resident in HBM:
batch 256 x vocab 128256, temperature 0.7, top-k 50, top-p 0.9, repetition penalty 1.15 over a
512-token Zipf(1.1) history per row, one seeded uniform per row (configuration 3 of BASELINE.json,
the one the metric is quoted on).  Prints ONE JSON line.

  value        sampled tokens/s of the whole step (one launch: topk_row_kernel reads every row once
               and finishes it; inputs resident in HBM, cycled through several buffers so that no
               step finds its logits in the Infinity Cache)
  roofline     that kernel: algorithmic bytes of one step divided by its average launch duration,
               measured here with HIP events on the launch stream over the timed region
  timing       W untimed warm-up steps, then exactly K timed steps between two events on the launch
               stream, a synchronisation on either side.  The spread measurement (30 groups of 10
               steps, its own figures) runs before the warm-up: a step is 27 us, W = 5 steps are
               0.14 ms, and a device that idled during the host's set-up is not at its working clocks
               after that little work
  cpu_baseline the CPU oracle's reference-arithmetic mode timed on this box's host, one thread,
               on a bounded sample of the same workload

The other configurations of BASELINE.json run through the same script for their own figures (never the
headline): --config C1 | C2 (multinomial) | C2g (greedy argmax) | C4 (speculative verify, 64 x 5 positions;
"tokens" are verified draft positions) | C5; and three sets of secondary timings at the C3 shape:
--config C3x (the step with min-p, with the frequency / presence penalties, with per-row arrays) | LP (token
log-probabilities) | GEN (the generation loop: embedding lookup, LM head, sampling, history append); and
--config OPS: the reference's operators on the path (softmax, log-softmax, argmax, token log-probabilities, conv2d,
matmul) at shapes from a classifier's ten classes to an LLM's vocabulary, each beside the vendor library's time
through torch.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C3|C1|C2|C2g|C4|C5|C3x|LP|GEN|OPS] [--no-cpu] [--no-producer]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_FP32_PEAK_TFLOPS = 157.3

# HBM bytes per launch of the dominant kernel, from hardware counters (not measurable from inside this
# script): two runs `rocprofv3 --pmc FETCH_SIZE --kernel-trace -- python3 bench.py --no-cpu --steps 20
# --warmup 5 --copy-probe` and the same with WRITE_SIZE; each counter's per-dispatch average for the
# kernel is scaled by what the same counter reads for the --copy-probe copy of one logits buffer
# (131 334 144 B read and written).  One entry per (configuration, kernel) that was measured, with the
# file under profiles/ that holds the counters; a run whose dominant kernel is not listed prints null.
PMC_TRAFFIC = {
    ("C3", "topk_row_kernel"): {
        "bytes": int(64680.2 * (128256 / 64139.6) * 1024 + 24.0 * 1024),
        "measured_on": "born::topk_row_kernel<true, false, 0>, workload C3",
        "source": "profiles/topk_row_kernel_c3_hbm_traffic.txt",
    },
    # (the probe of that run copied a C5 logits buffer: 608 256 KiB read and written)
    ("C5", "nucleus_row_kernel"): {
        "bytes": int(1013983.9 * (608256 / 304141.8) * 1024 + 102.9 * 1024),
        "measured_on": "born::nucleus_row_kernel<512, false, true>, workload C5 (what the L2s fetch, the Infinity Cache's share included)",
        "source": "profiles/nucleus_row_kernel_c5_counters.txt",
    },
}

METRIC = {
    "C3": "sampled tokens/s at batch 256 x vocab 128256 (top-k+top-p); achieved HBM GB/s",
    "C1": "sampled tokens/s at batch 1 x vocab 32000 (top-k+top-p, launch-latency bound); secondary configuration, not the headline",
    "C2": "sampled tokens/s at batch 64 x vocab 32000 (temperature-1 full-vocabulary multinomial); secondary configuration, not the headline",
    "C2g": "greedy tokens/s at batch 64 x vocab 32000 (argmax); secondary configuration, not the headline",
    "C4": "verified draft positions/s, speculative accept/reject at 64 sequences x 5 positions x vocab 32000; secondary configuration, not the headline",
    "C5": "sampled tokens/s at batch 1024 x vocab 152064 (top-p 0.99 without a top-k cut); secondary configuration, not the headline",
}


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform
    return platform.processor() or platform.machine()


def go_twin():
    """The Go twin of the CPU baseline (backend/rocm/cpu_ref_test.go), if this box has a Go toolchain: run in a child
    process of its own, reported with GOMAXPROCS.  No toolchain: says so."""
    import shutil
    import subprocess
    go = shutil.which("go")
    if not go:
        return {"go": "absent"}
    procs = os.environ.get("GOMAXPROCS") or str(len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1))
    try:
        r = subprocess.run([go, "test", "-run", "^$", "-bench", "CPURef", "-benchtime", "3x", "./backend/rocm"], cwd=ROOT, capture_output=True,
                           text=True, timeout=180, env=dict(os.environ, GOMAXPROCS=procs, GOFLAGS="-mod=mod"))
    except (OSError, subprocess.TimeoutExpired) as e:
        return {"go": go, "error": str(e)[:200]}
    out = {"go": go, "GOMAXPROCS": int(procs), "returncode": r.returncode}
    lines = [ln for ln in r.stdout.splitlines() if ln.startswith("Benchmark")]
    if lines:
        out["benchmarks"] = lines[:8]
    else:
        out["output_tail"] = (r.stdout + r.stderr)[-400:]
    return out


def parity_block(w, tokens_host, probs_host, rows=16):
    """The oracle as the checker on a slice of the batch, outside the timed region: how many of the sampled rows equal
    the fixed-point layer (must be all), how many the fp64 layer flags as lying within 1e-6 of a CDF step, how many
    differ from the fp64 layer (all of those must be flagged)."""
    from oracle import pyoracle
    B = w.logits.shape[0]
    idx = sorted(set(np.linspace(0, B - 1, num=min(rows, B)).astype(int).tolist()))
    x = np.ascontiguousarray(w.logits[idx])
    u = np.ascontiguousarray(w.uniforms[idx])
    h = None if w.history is None else np.ascontiguousarray(w.history[idx])
    fx = pyoracle.sample(x, u, w.temperature, w.top_k, w.top_p, w.rep, h, mode=pyoracle.MODE_FIXED)
    tr = pyoracle.sample(x, u, w.temperature, w.top_k, w.top_p, w.rep, h, mode=pyoracle.MODE_TRUTH)
    got, gp = tokens_host[idx], probs_host[idx]
    differ = got != tr["tokens"]
    same = ~differ & ~tr["near_cut"]
    rel = np.abs(gp[same].astype(np.float64) - tr["probs"][same]) / np.maximum(tr["probs"][same], 1e-300)
    return {"rows_checked": len(idx), "rows": idx,
            "tokens_equal_fixed_point_layer": int((got == fx["tokens"]).sum()),
            "probabilities_bit_equal_fixed_point_layer": int((gp.view(np.uint32) == fx["probs"].view(np.uint32)).sum()),
            "rows_flagged_within_1e-6_of_a_cdf_step": int(tr["near"].sum()),
            "tokens_differing_from_fp64_layer": int(differ.sum()),
            "of_those_not_flagged": int((differ & ~tr["near"]).sum()),
            "max_relative_probability_error_vs_fp64": float(rel.max()) if rel.size else 0.0,
            "checker": "oracle/born_oracle.c (fixed-point layer and fp64 layer), not part of the timed region"}


def cpu_baseline(w, seconds=12.0):
    """Times the oracle's reference-arithmetic mode (the checker, used here only as the CPU baseline)."""
    from oracle import pyoracle
    rows = min(16, w.logits.shape[0])
    x = np.ascontiguousarray(w.logits[:rows])
    u = w.uniforms[:rows]
    h = None if w.history is None else np.ascontiguousarray(w.history[:rows])
    pyoracle.sample(x, u, w.temperature, w.top_k, w.top_p, w.rep, h, mode=pyoracle.MODE_REF32)   # warm
    t0 = time.perf_counter()
    n = 0
    while time.perf_counter() - t0 < seconds:
        pyoracle.sample(x, u, w.temperature, w.top_k, w.top_p, w.rep, h, mode=pyoracle.MODE_REF32)
        n += rows
    dt = time.perf_counter() - t0
    out = {"value": n / dt, "unit": "tokens/s", "cores": 1, "kind": "port", "cpu_model": cpu_model(),
           "sample": f"{n} rows of the same workload ({rows}-row slices repeated for {dt:.1f} s), "
                     "C restatement of a Born-style scalar sampler (fp64 exp cast to fp32, sequential fp32 sums, heap top-k), 1 thread"}
    # The same port row-parallel over the host cores this process may use (rows are independent; the C call
    # releases the interpreter lock): the analogue of running the reference with one goroutine per core.
    from concurrent.futures import ThreadPoolExecutor
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = max(1, min(cores, 16))

    def worker(deadline):
        k = 0
        while time.perf_counter() < deadline:
            pyoracle.sample(x, u, w.temperature, w.top_k, w.top_p, w.rep, h, mode=pyoracle.MODE_REF32)
            k += rows
        return k

    t0 = time.perf_counter()
    with ThreadPoolExecutor(cores) as ex:
        done = sum(ex.map(worker, [t0 + seconds / 2] * cores))
    dt = time.perf_counter() - t0
    out["all_cores"] = {"value": done / dt, "unit": "tokens/s", "cores": cores,
                        "sample": f"{done} rows, {cores} threads each repeating the {rows}-row slice for {dt:.1f} s"}
    out["go_twin"] = go_twin()
    return out


def producer_leg(torch, dev, smp, sample_step, B, V, hidden, logits_all, stream, iters, fused_args=None):
    """The logits producer in front of the sampler: x[B, hidden] @ W[V, hidden]^T + b on the fp32 matrix cores
    (born_rocm_linear), written into the buffers the sampling step reads.  Random-init weights of the LM-head
    shape; reported beside the headline metric, never part of it."""
    from born_amd import linear as L
    g = torch.Generator(device=dev)
    g.manual_seed(20251125)
    x = torch.randn(B, hidden, device=dev, generator=g)
    wgt = torch.randn(V, hidden, device=dev, generator=g) * (1.5 / hidden ** 0.5)
    bias = torch.zeros(V, device=dev)
    layer = L.Linear(hidden, V, wgt, bias)
    scratch = torch.empty(B, V, device=dev)          # the logits the head produces and the chained sampling step reads

    def head():
        layer.Forward(x, (B, hidden), scratch, stream=stream)

    def timed(fn, k):
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(k):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / k

    for _ in range(10):
        head()
    ms_head = timed(head, iters)

    def both():
        head()
        sample_step(scratch)

    both()
    ms_both = timed(both, iters)
    flops = 2.0 * B * hidden * V
    tf = flops / (ms_head * 1e-3) / 1e12
    fused = None
    if fused_args is not None:
        # the same head with the sampling step in its epilogue (born_rocm_linear_sample): the logits are never written
        history, H, uniforms, tokens, probs = fused_args
        tok_ref = tokens.clone()                                     # tokens of the unfused pair on `scratch`

        def fused_step():
            L.ForwardSample(smp, layer, x, (B, hidden), history, None, uniforms, tokens, probs, hist_stride=H, stream=stream)

        fused_step()
        torch.cuda.synchronize()
        got = tokens.cpu().numpy()
        settled = got >= 0
        agree = bool((got[settled] == tok_ref.cpu().numpy()[settled]).all())
        if not settled.all():
            try:
                smp.Status(stream)
            except Exception:
                pass
        ms_fused = timed(fused_step, iters)
        fused = {"ms": ms_fused, "rows_settled": int(settled.sum()), "rows": int(B), "tokens_equal_the_unfused_pair": agree,
                 "logits_bytes_not_written": int(B) * int(V) * 4}
    return {"fused_head_and_sampling": fused, "kernel": "gemm_f32_dma_kernel", "workload": f"LM head: [{B}, {hidden}] @ [{V}, {hidden}]^T + bias, fp32 in / fp32 accumulate / fp32 out",
            "ms": ms_head, "roofline": {"bound": "mfma", "achieved": tf, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                                        "frac": tf / MFMA_FP32_PEAK_TFLOPS},
            "weight_stream_GBs": V * hidden * 4 / (ms_head * 1e-3) / 1e9,
            "ms_head_plus_sampling_step": ms_both, "tokens_per_s_head_plus_sampling": B / (ms_both * 1e-3), "iters": iters}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--config", default="C3")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--rotate", type=int, default=4,
                    help="number of distinct logits buffers cycled through, so that a step never finds its logits in a cache")
    ap.add_argument("--path", type=int, default=0, help="kernel selection of the sampler (0 = default; 1 = always the general kernel)")
    ap.add_argument("--no-producer", action="store_true",
                    help="skip the LM-head leg (hidden states -> logits on the device, then the same sampling step)")
    ap.add_argument("--hidden", type=int, default=4096, help="hidden size of the LM-head leg")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a few plain device-to-device copies of one logits buffer (a kernel of known traffic "
                         "for scaling the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; rows are independent, so more GPUs would each take a "
              "slice of the batch with no exchange. Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    from born_amd import sampler as S
    from born_amd import synth

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.config == "OPS":
        return main_ops(args, torch, S, dev)
    if args.config in ("C3x", "LP", "GEN"):
        return main_extras(args, torch, S, synth, dev)
    gen = {"C1": synth.c1, "C2": synth.c2, "C2g": synth.c2, "C3": synth.c3, "C4": synth.c4, "C5": synth.c5}[args.config]
    w = gen()
    if args.config in ("C2g", "C4"):
        return main_other(args, torch, S, synth, w, dev)
    B, V = w.logits.shape
    # Several copies of the logits at different addresses, used round-robin: together they exceed the 256 MB
    # Infinity Cache, so every step streams its logits from HBM as a fresh LM-head output would be.
    nrot = max(1, args.rotate)
    logits_all = [torch.from_numpy(w.logits).to(dev) for _ in range(nrot)]
    logits = logits_all[0]
    uniforms = torch.from_numpy(w.uniforms).to(dev)
    history = torch.from_numpy(w.history).to(dev) if w.history is not None else None
    H = 0 if history is None else history.shape[1]
    tokens = torch.empty(B, dtype=torch.int32, device=dev)
    probs = torch.empty(B, dtype=torch.float32, device=dev)

    smp = S.NewSampler(S.SamplerConfig(Temperature=w.temperature, TopK=w.top_k, TopP=w.top_p,
                                       RepetitionPenalty=w.rep), max_batch=B, max_vocab=V)
    smp.SetPath(args.path)
    stream = torch.cuda.current_stream().cuda_stream

    counter = [0]

    # One sampling step = one call of born_rocm_sample (the same C entry point Sampler.Sample makes, the same
    # arguments).  The calls are bound once, pointers and sizes already converted, so that the host side of a step is
    # the C call alone: with the Python wrapper's per-call conversions the host lags behind a 27 us kernel at the start
    # of a timed region, and that lag would be charged to the steps.
    from born_amd import _capi
    import functools
    lib = _capi.lib()

    def bind(lg):
        return functools.partial(lib.born_rocm_sample, smp._h, lg.data_ptr(), B, V, V, None if history is None else history.data_ptr(),
                                 None, H, uniforms.data_ptr(), tokens.data_ptr(), probs.data_ptr(), None, None, None, 0, stream)

    calls = [bind(lg) for lg in logits_all]
    smp.Sample(logits, B, V, history, None, uniforms, tokens, probs, hist_stride=H, stream=stream)   # the wrapper once: checks every argument

    def step(lg=None):
        if lg is None:
            rc = calls[counter[0] % nrot]()
            counter[0] += 1
        else:
            rc = bind(lg)()
        if rc:
            _capi.check(rc)

    def timed(k):
        """ms per step over exactly k steps, between two events on the launch stream, a synchronisation on either side."""
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(k):
            step()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / k

    # The literal reading of the flags first: W warm-up steps straight after the host's set-up (the device has idled),
    # then K timed steps.  Reported beside the headline as ms_per_step_idle_start.
    for _ in range(args.warmup):
        step()
    ms_idle_start = timed(args.steps)

    # The LM-head leg runs next (its own figures, never part of the headline): the W warm-up steps and the K timed
    # steps below then run on a device that is already at its working clocks, as in a serving loop.
    producer = None
    if not args.no_producer and args.config == "C3":
        producer = producer_leg(torch, dev, smp, step, B, V, args.hidden, logits_all, stream, max(5, args.steps // 10),
                                fused_args=(history, H, uniforms, tokens, probs))

    if args.copy_probe:
        dst = torch.empty_like(logits_all[0])
        for i in range(5):
            dst.copy_(logits_all[i % nrot])          # reads and writes logits.nbytes each
        torch.cuda.synchronize()
        del dst

    # spread of the step time: groups of 10 back-to-back steps, each group timed on its own (outside the headline figure).
    # Measured first: a step is 27 us, so W = 5 warm-up steps are 0.14 ms, and a device that idled while the host prepared
    # the run needs a few ms of work to be back at its working clocks (measured: the first 25 steps after a pause run
    # 1 % slower than the next 20 at C3, 8 % at C5).
    groups = sorted(timed(10) for _ in range(30))
    # W untimed warm-up steps, then exactly K timed steps
    for _ in range(args.warmup):
        step()
    ms = timed(args.steps)
    spread = {"median": groups[len(groups) // 2], "p10": groups[len(groups) // 10], "p90": groups[(9 * len(groups)) // 10],
              "sample": "30 groups of 10 steps, ms per step, measured before the warm-up and the timed region"}
    smp.Status(stream)
    counters = smp.Counters(stream)
    tok_host = tokens.cpu().numpy()
    assert tok_host.min() >= 0 and tok_host.max() < V

    # a step is a single launch, so the step time is the kernel's launch-to-launch duration (an upper bound of the
    # kernel's own duration, so a lower bound of the roofline fraction)
    ms_kernel = ms
    # the kernel the library selects for this configuration (born_amd/csrc/api.hip, sample_impl); the work counters
    # read back above confirm it: rows settled by the single-pass kernel, by its exact selection, by the other two
    kernel_name = ("topk_row_kernel" if 1 <= w.top_k <= 128 else "nucleus_row_kernel" if w.top_k == 0 else "sample_wide_kernel") \
        if args.path == 0 else "sample_wide_kernel"
    # (the checked call, the 30 groups, the warm-up, the timed region; the chained and the fused steps of the LM-head leg
    # count too)
    launches = 1 + 300 + 2 * (args.warmup + args.steps) + (0 if producer is None else 2 * (producer["iters"] + 1))
    warmup_effective = launches - args.steps - (0 if producer is None else producer["iters"] + 1)   # (the fused steps do not run this kernel)
    if kernel_name == "topk_row_kernel":
        confirmed = counters["topk_rows"] + counters["fallback_rows"] == B * launches and counters["general_rows"] == 0
    else:
        confirmed = counters["general_rows"] >= B * launches and counters["topk_rows"] == 0
    traffic = PMC_TRAFFIC.get((args.config, kernel_name))
    alg_bytes = w.algorithmic_bytes()
    achieved = alg_bytes / (ms_kernel * 1e-3) / 1e9

    out = {
        "metric": METRIC[args.config],
        "value": B / (ms * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "warmup_effective": warmup_effective,
        "ms_per_step": ms,
        "ms_per_step_idle_start": ms_idle_start,
        "ms_per_step_idle_start_note": "the same K steps behind the same W warm-up steps, taken straight after set-up, before anything else ran on the device",
        "ms_per_step_timing": "HIP events on the launch stream around exactly K steps, a synchronisation on either side, behind W warm-up steps; "
                              "the 30 groups of ms_per_step_spread run before the warm-up, so the device is at its working clocks",
        "ms_per_step_spread": spread,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{w.name}: batch {B} x vocab {V}, T={w.temperature}, top_k={w.top_k}, top_p={w.top_p}, "
                               f"repetition_penalty={w.rep}, history {H}/row, seeded uniforms; logits resident in HBM",
                   "seed": synth.BASE_SEED, "logits_buffers_rotated": nrot, "fallback_rows_per_step": counters["fallback_rows"] / max(1, launches)},
        "roofline": {"bound": "hbm", "kernel": kernel_name, "kernel_confirmed_by_work_counters": confirmed, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic["bytes"] if traffic else None,
                     "traffic_unit": "bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled by a copy of known size)",
                     "traffic_provenance": ({k: traffic[k] for k in ("measured_on", "source")} if traffic else None),
                     "algorithmic_bytes_per_launch": alg_bytes,
                     "kernel_ms": ms_kernel, "kernel_ms_kind": "step (launch-to-launch, HIP events over the timed region / steps)"},
    }
    if producer is not None:
        out["producer"] = producer
    if not args.no_cpu:
        out["parity"] = parity_block(w, tok_host, probs.cpu().numpy())
        out["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(out))


def main_ops(args, torch, S, dev):
    """The operators at several shapes, us per call through the C ABI with every buffer allocated beforehand (best of three
    regions of --steps calls), and the same operation through torch (the vendor libraries) beside it.  One JSON line."""
    import ctypes as C
    from born_amd import _capi
    lib = _capi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    steps = max(5, min(args.steps, 50))
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)

    def best(fn):
        res = []
        for _ in range(3):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            res.append(e0.elapsed_time(e1) / steps * 1e3)
        return min(res)

    def ptr(t):
        return C.c_void_p(t.data_ptr())

    out = {"metric": "operators of the path, us per call (not the headline)", "config": {"workload": "OPS"}, "n_gpus": 1, "steps": steps,
           "data": "synthetic", "dtype": "f32", "us": {}}
    smp = S.NewSampler(S.SamplerConfig(), max_batch=65536, max_vocab=152064)
    for rows, V in ((65536, 10), (8192, 1024), (4096, 4096), (1024, 32000), (256, 128256)):
        x = torch.randn(rows, V, device=dev, generator=gen) * 1.5
        y = torch.empty(rows, V, device=dev)
        tok = torch.randint(0, V, (rows,), device=dev, dtype=torch.int32)
        tok64 = tok.long()
        o32 = torch.empty(rows, dtype=torch.int32, device=dev)
        lp = torch.empty(rows, device=dev)
        shape = f"{rows} x {V}"
        out["us"][f"softmax {shape}"] = {"born": best(lambda: smp.Softmax(x, rows, V, y, stream=stream)),
                                         "torch": best(lambda: torch.softmax(x, dim=1, out=y))}
        out["us"][f"log_softmax {shape}"] = {"born": best(lambda: smp.Softmax(x, rows, V, y, stream=stream, log=True)),
                                             "torch": best(lambda: torch.log_softmax(x, dim=1, out=y))}
        out["us"][f"argmax {shape}"] = {"born": best(lambda: smp.Argmax(x, rows, V, o32, stream=stream)),
                                        "torch": best(lambda: torch.argmax(x, dim=1))}
        out["us"][f"token log-probabilities {shape}"] = {
            "born": best(lambda: smp.TokenLogprobs(x, rows, V, None, None, tok, lp, stream=stream)),
            "torch": best(lambda: torch.nn.functional.cross_entropy(x, tok64, reduction="none"))}
        del x, y
    smp.Close()
    for (m, k, n) in ((64, 784, 128), (64, 128, 10), (256, 784, 512), (1024, 1024, 1024), (512, 4096, 512), (4096, 4096, 4096)):
        a, b, c = torch.randn(m, k, device=dev, generator=gen), torch.randn(k, n, device=dev, generator=gen), torch.empty(m, n, device=dev)

        def mm():
            _capi.check(lib.born_rocm_matmul(ptr(a), ptr(b), ptr(c), m, k, n, k, n, n, None))
        out["us"][f"matmul [{m},{k}] @ [{k},{n}]"] = {"born": best(mm), "torch": best(lambda: torch.matmul(a, b, out=c))}
    for (m, k, n) in ((64, 784, 128), (64, 4096, 4096), (512, 4096, 512), (32, 4096, 128256)):
        x, w, b = torch.randn(m, k, device=dev, generator=gen), torch.randn(n, k, device=dev, generator=gen), torch.randn(n, device=dev, generator=gen)
        y = torch.empty(m, n, device=dev)

        def lin():
            _capi.check(lib.born_rocm_linear(ptr(x), m, k, k, ptr(w), n, k, ptr(b), ptr(y), n, None))
        out["us"][f"linear [{m},{k}] -> {n}"] = {"born": best(lin), "torch": best(lambda: torch.nn.functional.linear(x, w, b))}
        del x, w, y
    for (xs, ks, stride, pad) in (((64, 1, 28, 28), (32, 1, 5, 5), 1, 0), ((64, 32, 12, 12), (64, 32, 5, 5), 1, 0),
                                  ((256, 64, 56, 56), (64, 64, 3, 3), 1, 1)):
        x, w = torch.randn(*xs, device=dev, generator=gen), torch.randn(*ks, device=dev, generator=gen)
        ho, wo = (xs[2] + 2 * pad - ks[2]) // stride + 1, (xs[3] + 2 * pad - ks[3]) // stride + 1
        y = torch.empty(xs[0], ks[0], ho, wo, device=dev)
        xsa, ksa, osh = (C.c_int64 * 4)(*xs), (C.c_int64 * 4)(*ks), (C.c_int64 * 4)()

        def conv():
            _capi.check(lib.born_rocm_conv2d(ptr(x), xsa, ptr(w), ksa, stride, pad, ptr(y), osh, None))
        out["us"][f"conv2d {list(xs)} * {list(ks)} stride {stride} padding {pad}"] = {
            "born": best(conv), "torch": best(lambda: torch.nn.functional.conv2d(x, w, stride=stride, padding=pad))}
    print(json.dumps(out))


def main_extras(args, torch, S, synth, dev):
    """Secondary figures at the C3 shape (never the headline), one JSON line:
      C3x  the sampling step with min-p, with the frequency / presence penalties, and with per-row arrays
      LP   token log-probabilities (the cross-entropy forward term), plain and with history + penalty + temperature
      GEN  the generation loop (embedding lookup, LM head, sampling, history append) at three shapes"""
    stream = torch.cuda.current_stream().cuda_stream

    def timed(fn, k, warm):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(k):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / k * 1e3          # us per call

    out = {"metric": "secondary figures, us per step (not the headline)", "config": {"workload": args.config, "seed": synth.BASE_SEED},
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "data": "synthetic", "dtype": "f32", "us": {}}
    if args.config == "GEN":
        import time
        from born_amd import linear as L
        from born_amd.generate import Generator
        for (B, V, K) in [(1, 32000, 4096), (64, 32000, 4096), (256, 128256, 4096)]:
            E = torch.randn(V, K, device=dev) * 0.02
            W = torch.randn(V, K, device=dev) * 0.02
            smp = S.NewSampler(S.SamplerConfig(Temperature=0.8, TopK=40, TopP=0.95, RepetitionPenalty=1.1, Seed=1), max_batch=B, max_vocab=V)
            gen = Generator(E, V, K, L.Linear(K, V, W, None), smp, max_batch=B, max_len=1024)
            prompts = [[1, 2, 3]] * B
            gen.Generate(prompts, 8)
            n = min(200, args.steps)
            t0 = time.perf_counter()
            gen.Generate(prompts, n)
            dt = time.perf_counter() - t0
            out["us"][f"decode step (gather + LM head + sample + append), batch {B} x vocab {V} x hidden {K}"] = dt / n * 1e6
            smp.Close()
            del E, W
        print(json.dumps(out))
        return
    w = synth.c3()
    B, V = w.logits.shape
    lgs = [torch.from_numpy(w.logits).to(dev) for _ in range(max(1, args.rotate))]
    u = torch.from_numpy(w.uniforms).to(dev)
    h = torch.from_numpy(w.history).to(dev)
    H = h.shape[1]
    tok = torch.empty(B, dtype=torch.int32, device=dev)
    pr = torch.empty(B, device=dev)
    c = [0]

    def mk(top_k=None, **kw):
        return S.NewSampler(S.SamplerConfig(Temperature=w.temperature, TopK=w.top_k if top_k is None else top_k, TopP=w.top_p,
                                            RepetitionPenalty=w.rep, **kw), max_batch=B, max_vocab=V)

    def nxt():
        c[0] += 1
        return lgs[c[0] % len(lgs)]

    if args.config == "C3x":
        base, minp, fp = mk(), mk(MinP=0.05), mk(FrequencyPenalty=0.3, PresencePenalty=0.5)
        # penalties that raise logits (seen ids join the single-pass kernel's candidates from the history's hash)
        fneg = mk(FrequencyPenalty=-0.2, PresencePenalty=-0.1)
        rlow = S.NewSampler(S.SamplerConfig(Temperature=w.temperature, TopK=w.top_k, TopP=w.top_p, RepetitionPenalty=0.87), max_batch=B, max_vocab=V)
        k100, k128, k129, k256, k512, k513, k0 = mk(top_k=100), mk(top_k=128), mk(top_k=129), mk(top_k=256), mk(top_k=512), mk(top_k=513), mk(top_k=0)
        # rows whose large logits sit where a threshold drawn from the row's first logits does not look (same shape, same
        # history and uniforms): sorted ascending; a step up in the last tenth; a bump around the middle
        rng = np.random.default_rng(synth.BASE_SEED)
        i = np.arange(V, dtype=np.float64)
        shaped = {"ascending": np.tile(i / V * 20 - 10, (B, 1)) + rng.standard_normal((B, V)) * 1e-3,
                  "late_step": rng.standard_normal((B, V)), "mid_bump": rng.standard_normal((B, V))}
        shaped["late_step"][:, V - V // 10:] += 30
        shaped["mid_bump"][:, V // 2:V // 2 + V // 10] += 30
        shaped = {name: [torch.from_numpy(x.astype(np.float32)).to(dev) for _ in range(2)] for name, x in shaped.items()}

        def shaped_case(name, smp):
            def f():
                c[0] += 1
                smp.Sample(shaped[name][c[0] % 2], B, V, h, None, u, tok, pr, hist_stride=H, stream=stream)
            return f
        Ts = torch.full((B,), w.temperature, device=dev)
        ks = torch.full((B,), w.top_k, dtype=torch.int32, device=dev)
        ps = torch.full((B,), w.top_p, device=dev)
        rs = torch.full((B,), w.rep, device=dev)
        cases = {
            "C3": lambda: base.Sample(nxt(), B, V, h, None, u, tok, pr, hist_stride=H, stream=stream),
            "C3 shape, top_k 100": lambda: k100.Sample(nxt(), B, V, h, None, u, tok, pr, hist_stride=H, stream=stream),
            "C3 shape, top_k 128": lambda: k128.Sample(nxt(), B, V, h, None, u, tok, pr, hist_stride=H, stream=stream),
            "C3 shape, top_k 129": lambda: k129.Sample(nxt(), B, V, h, None, u, tok, pr, hist_stride=H, stream=stream),
            "C3 shape, top_k 256": lambda: k256.Sample(nxt(), B, V, h, None, u, tok, pr, hist_stride=H, stream=stream),
            "C3 shape, top_k 512": lambda: k512.Sample(nxt(), B, V, h, None, u, tok, pr, hist_stride=H, stream=stream),
            "C3 shape, top_k 513 (the general kernel)": lambda: k513.Sample(nxt(), B, V, h, None, u, tok, pr, hist_stride=H, stream=stream),
            "C3 settings, rows sorted ascending": shaped_case("ascending", base),
            "C3 settings, rows with a step up in their last tenth": shaped_case("late_step", base),
            "C3 settings, rows with a bump around their middle": shaped_case("mid_bump", base),
            "C3 settings, rows sorted ascending, top_k 512": shaped_case("ascending", k512),
            "C3 settings, rows with a step up in their last tenth, top_k 256": shaped_case("late_step", k256),
            "C3 shape, top_k 0 (top-p alone: the three-sweep kernel)": lambda: k0.Sample(nxt(), B, V, h, None, u, tok, pr, hist_stride=H, stream=stream),
            "C3 + min_p 0.05": lambda: minp.Sample(nxt(), B, V, h, None, u, tok, pr, hist_stride=H, stream=stream),
            "C3 + frequency 0.3 + presence 0.5": lambda: fp.Sample(nxt(), B, V, h, None, u, tok, pr, hist_stride=H, stream=stream),
            "C3 + frequency -0.2 + presence -0.1": lambda: fneg.Sample(nxt(), B, V, h, None, u, tok, pr, hist_stride=H, stream=stream),
            "C3 with repetition penalty 0.87 instead of 1.15": lambda: rlow.Sample(nxt(), B, V, h, None, u, tok, pr, hist_stride=H, stream=stream),
            "C3 with per-row arrays (same values in every row)":
                lambda: base.SampleRows(nxt(), B, V, h, None, u, Ts, ks, ps, rs, tok, pr, hist_stride=H, stream=stream),
            "C3 with per-row arrays and the promise that every row has a small top-k":
                lambda: base.SampleRows(nxt(), B, V, h, None, u, Ts, ks, ps, rs, tok, pr, hist_stride=H, stream=stream, rowKinds=1),
        }
    else:
        lp = torch.empty(B, device=dev)
        plain, full = S.NewSampler(S.SamplerConfig(), max_batch=B, max_vocab=V), mk()
        cases = {
            "token log-probabilities, plain (temperature 1, no history)":
                lambda: plain.TokenLogprobs(nxt(), B, V, None, None, tok, lp, stream=stream),
            "token log-probabilities, 512-token history + repetition penalty + T 0.7":
                lambda: full.TokenLogprobs(nxt(), B, V, h, None, tok, lp, hist_stride=H, stream=stream),
        }
        tok.zero_()
    for name, fn in cases.items():
        out["us"][name] = timed(fn, args.steps, args.warmup)
    if args.config == "C3x":
        # larger batches at the C3 settings: more rows than CUs run two rows to a CU at a time (512 threads per row)
        out["larger_batches"] = {}
        for rows in (512, 1024):
            wl = synth.c3(rows=rows)
            lg2 = [torch.from_numpy(wl.logits).to(dev) for _ in range(2)]
            u2, h2 = torch.from_numpy(wl.uniforms).to(dev), torch.from_numpy(wl.history).to(dev)
            t2, p2 = torch.empty(rows, dtype=torch.int32, device=dev), torch.empty(rows, device=dev)
            s2 = S.NewSampler(S.SamplerConfig(Temperature=wl.temperature, TopK=wl.top_k, TopP=wl.top_p, RepetitionPenalty=wl.rep),
                              max_batch=rows, max_vocab=V)

            def big():
                c[0] += 1
                s2.Sample(lg2[c[0] % 2], rows, V, h2, None, u2, t2, p2, hist_stride=H, stream=stream)
            us = timed(big, args.steps, args.warmup)
            out["larger_batches"][f"{rows} rows"] = {"us": us, "tokens_per_s": rows / us * 1e6,
                                                     "frac_of_8TBs": wl.algorithmic_bytes() / us / 1e3 / HBM_PEAK_GBS}
            s2.Close()
            del lg2
        # rows the single-pass kernel handed to its exact selection, over every step of every case above (0: none did)
        out["exact_selection_rows_total"] = {name: smp.Counters(stream)["fallback_rows"] for name, smp in
                                             (("handle of the C3 settings (all its cases)", base), ("top_k 256", k256), ("top_k 512", k512),
                                              ("frequency -0.2 + presence -0.1", fneg), ("repetition penalty 0.87", rlow))}
    out["algorithmic_bytes_per_step"] = w.algorithmic_bytes()
    print(json.dumps(out))


def main_other(args, torch, S, synth, w, dev):
    """C2g (greedy argmax over the C2 logits) and C4 (speculative verify): the same JSON shape, own figures."""
    stream = torch.cuda.current_stream().cuda_stream
    if args.config == "C2g":
        B, V = w.logits.shape
        logits = torch.from_numpy(w.logits).to(dev)
        tokens = torch.empty(B, dtype=torch.int32, device=dev)
        smp = S.NewSampler(max_batch=B, max_vocab=V)
        step = lambda: smp.Argmax(logits, B, V, tokens, stream=stream)
        units, alg_bytes, kernel_name = B, B * V * 4 + 4 * B, "argmax_partial_kernel"
        workload = f"C2 greedy: batch {B} x vocab {V}, argmax; logits resident in HBM"
    else:
        e = w.extra
        B, G, V = e["target"].shape
        t, d = torch.from_numpy(e["target"]).to(dev), torch.from_numpy(e["draft"]).to(dev)
        dt = torch.from_numpy(e["draft_tokens"]).to(dev)
        ua, ur = torch.from_numpy(e["u_acc"]).to(dev), torch.from_numpy(e["u_res"]).to(dev)
        na = torch.empty(B, dtype=torch.int32, device=dev)
        nt = torch.empty(B, dtype=torch.int32, device=dev)
        smp = S.NewSampler(S.SamplerConfig(Temperature=w.temperature), max_batch=B, max_vocab=V)
        step = lambda: smp.Verify(t, d, B, G, V, dt, ua, ur, na, nt, stream=stream)
        units, alg_bytes, kernel_name = B * G, 2 * B * G * V * 4 + 4 * B * G * 2 + 4 * B * 3, "spec_stats_kernel (+ residual, pick)"
        workload = f"C4: speculative verify, {B} sequences x {G} positions x vocab {V}, T={w.temperature}; \"tokens\" are verified draft positions"
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    smp.Status(stream)
    achieved = alg_bytes / (ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": METRIC[args.config], "value": units / (ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": workload, "seed": synth.BASE_SEED},
        "roofline": {"bound": "hbm", "kernel": kernel_name, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None, "traffic_provenance": None,
                     "algorithmic_bytes_per_launch": alg_bytes, "kernel_ms": ms,
                     "kernel_ms_kind": "step (all its launches, launch-to-launch, HIP events over the timed region / steps)"}}))


if __name__ == "__main__":
    main()
