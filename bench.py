#!/usr/bin/env python3
"""Benchmark of the fused P-partial reduce + residual-add + RMSNorm path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--sweep]

A step is one call of the fused op (one kernel launch) on one batch of synthetic
input that is already resident in HBM.  The default workload is the headline
configuration: one rank's shard of a Llama-70B TP=8 layer, P=8 partials of
[256, 8192] bf16 (a T=2048 batch).  Consecutive steps use different input sets,
cycling through 4 GiB of operands before any reuse.  The footprint is that large
on purpose: the kernel's streaming loads do not allocate in the 256 MB last-level
cache, so with a ~1 GiB rotation the lines WRITTEN by earlier steps (residual and
output) survive there until their set comes round again and inflate the figure by
up to 15 %.  Prints ONE JSON line on stdout; progress goes to stderr.

Fields beyond the usual ones:
  roofline      HBM roofline of the norm kernel: algorithmic bytes per launch
                divided by the mean launch duration, measured with HIP events that
                bracket the timed region's back-to-back launches on the launch stream.
  cpu_baseline  the CPU checker (oracle/, a port of the reference's
                csrc/cpu/layernorm.cpp extended to P partials) timed on this box's
                host cores on the same workload, for context only.
  sweep         (--sweep) µs/call and GB/s of every benchmark configuration, and the
                weave configuration's overlap figures.
"""
import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0       # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0
ROTATION_BYTES = 4 << 30      # distinct operand bytes cycled through before any reuse

# HBM bytes per launch read from the hardware counters (rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE, each scaled by the same counter's reading for the library's plain copy
# kernel of known size); the runs are summarised in
# profiles/row_norm_bf16_c2_T256_pmc_traffic.md.  Workloads without a counter run: None.
MEASURED_TRAFFIC_BYTES = {"c2_llama70b_tp8_shard@T256": 46366607}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="c2_llama70b_tp8_shard@T256")
    ap.add_argument("--max-ctas", type=int, default=0, help="grid cap (0 = library default)")
    ap.add_argument("--sweep", action="store_true", help="also time every configuration")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--weave-only", action="store_true",
                    help="time only the GEMM + norm weave of config 5 and print its figures (for profiling)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="after the timed region, run the library's plain copy kernel on "
                         "buffers of known size (reference traffic for rocprofv3 --pmc runs)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline")
    return ap.parse_args()


class NormRunner:
    """One bound call (tokenweave_amd.ops.BoundOp: arguments checked once, a single
    ctypes call per launch) for each input set, so that the host enqueues a step
    faster than the GPU runs it."""

    def __init__(self, cfg, nsets, max_ctas, device, epilogue="bf16"):
        import torch
        from tokenweave_amd import _custom_ops as ops
        from tokenweave_amd import _lib
        from tokenweave_amd import workloads as wl
        self.calls = []
        L = _lib.lib()
        for i in range(nsets):
            inp = wl.make_norm_inputs(cfg, device, seed_offset=i)
            if epilogue == "bf16":
                # y lands on this rank's staging rows (rank 0)
                op = ops.bind_reduce_add_rms_norm(inp.partials, inp.partials[0], inp.residual, inp.weight,
                                                  cfg.eps, max_ctas or None)
            else:
                op = self._bind_quant(ops, L, torch, cfg, epilogue, inp, max_ctas, device)
            op()  # one launch up front: a bad argument fails here, not in the timed loop
            self.calls.append(op)
        torch.cuda.synchronize()

    @staticmethod
    def _bind_quant(ops, L, torch, cfg, epilogue, inp, max_ctas, device):
        """The same reduction with a quantised output (one byte per element into its own
        buffer, a float per row for the dynamic kinds).  Checked once through the
        regular shim, then frozen."""
        qdtype = torch.int8 if epilogue == "int8_dynamic" else torch.float8_e4m3fn
        out = torch.empty(cfg.T, cfg.H, dtype=qdtype, device=device)
        scales = torch.full((max(cfg.T, 1), 1), 0.05, dtype=torch.float32, device=device)
        ptrs = (ctypes.c_void_p * cfg.P)(*[p.data_ptr() for p in inp.partials])
        keep = (inp, out, scales, ptrs)
        if epilogue == "fp8_static":
            ops.reduce_add_rms_norm_static_fp8_quant(inp.partials, out, inp.residual, inp.weight,
                                                     scales[:1].reshape(1), cfg.eps, max_ctas or None)
            args = (ptrs, cfg.P, out.data_ptr(), inp.residual.data_ptr(), inp.weight.data_ptr(),
                    scales.data_ptr(), cfg.T, cfg.H, max_ctas, cfg.eps)
            return ops.BoundOp(L.tw_reduce_add_rms_norm_static_fp8_quant, args, keep, out.device)
        ops.reduce_add_rms_norm_dynamic_per_token_quant(inp.partials, out, scales, inp.residual,
                                                        inp.weight, cfg.eps, None, max_ctas or None)
        args = (ptrs, cfg.P, out.data_ptr(), scales.data_ptr(), inp.residual.data_ptr(),
                inp.weight.data_ptr(), None, cfg.T, cfg.H, max_ctas, cfg.eps,
                1 if epilogue == "int8_dynamic" else 0)
        return ops.BoundOp(L.tw_reduce_add_rms_norm_dynamic_per_token_quant, args, keep, out.device)

    def step(self, i, stream):
        self.calls[i % len(self.calls)](stream)


def quant_bytes(cfg, epilogue):
    """Algorithmic bytes with a quantised output: one byte per element instead of two,
    plus one float per row for the dynamic kinds."""
    return cfg.bytes - cfg.T * cfg.H + (4 * cfg.T if epilogue.endswith("dynamic") else 4)


def time_norm(cfg, steps, warmup, max_ctas, device, epilogue="bf16"):
    """Returns dict(ms_per_step, gbps, kernel_us_mean): wall-clock per step between the
    two synchronisation points, and the mean launch duration from the HIP events that
    bracket the same `steps` back-to-back launches."""
    import torch
    nsets = max(2, min(256, -(-ROTATION_BYTES // cfg.bytes)))
    free, _ = torch.cuda.mem_get_info()
    set_bytes = (cfg.P + 1) * cfg.T * cfg.H * 2 + cfg.H * 2
    nsets = max(2, min(nsets, int(free * 0.6) // (set_bytes * 3)))  # fp32 staging while generating
    runner = NormRunner(cfg, nsets, max_ctas, device, epilogue)
    stream = torch.cuda.current_stream()
    for i in range(warmup):
        runner.step(i, stream)
    torch.cuda.synchronize()
    # timed region: exactly `steps` launches between two synchronisation points,
    # bracketed by HIP events on the launch stream
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for i in range(steps):
        runner.step(i, stream)
    e1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    res = {"ms_per_step": wall * 1e3 / steps, "gbps": cfg.bytes * steps / wall / 1e9,
           "nsets": nsets, "kernel_us_mean": e0.elapsed_time(e1) * 1e3 / steps}
    del runner
    torch.cuda.empty_cache()
    return res


CALIBRATION_COPY_BYTES = 256 << 20


def calibration_copies(device, n=8):
    """n launches of tw_copy_bytes, each reading and writing CALIBRATION_COPY_BYTES of
    memory that was not touched recently (4 source/destination pairs = 2 GiB)."""
    import torch
    from tokenweave_amd import _custom_ops as ops
    pairs = [(torch.ones(CALIBRATION_COPY_BYTES // 2, dtype=torch.bfloat16, device=device),
              torch.empty(CALIBRATION_COPY_BYTES // 2, dtype=torch.bfloat16, device=device))
             for _ in range(4)]
    torch.cuda.synchronize()
    for i in range(n):
        src, dst = pairs[i % 4]
        ops.copy_bytes(dst, src)
    torch.cuda.synchronize()


def time_norm_warm(cfg, steps, max_ctas, device):
    """Same call on ONE input set, so that after the first step the operands sit in
    the last-level cache (what a caller sees when the partials were just written)."""
    import torch
    runner = NormRunner(cfg, 1, max_ctas, device)
    stream = torch.cuda.current_stream()
    for i in range(10):
        runner.step(0, stream)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for i in range(steps):
        runner.step(0, stream)
    e1.record(stream)
    torch.cuda.synchronize()
    del runner
    torch.cuda.empty_cache()
    return e0.elapsed_time(e1) * 1e3 / steps


def cpu_baseline(cfg, budget_s):
    """Times the CPU checker on a bounded sample of the workload: the same shapes (rows
    capped at 1024), rotating through input sets of 1 GiB in total so that, like the GPU
    legs, every call reads memory and not a cache, repeated for `budget_s` seconds."""
    import numpy as np
    import torch
    from oracle import tw_oracle as O
    from tokenweave_amd import workloads as wl
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    rows = min(cfg.T, 1024)
    sample = cfg.with_tokens(rows)
    bits = lambda t: np.ascontiguousarray(t.contiguous().view(torch.int16).numpy().view(np.uint16))
    nsets = max(2, min(32, -(-(1 << 30) // sample.bytes)))
    sets = []
    for i in range(nsets):
        inp = wl.make_norm_inputs(sample, "cpu", seed_offset=i)
        r = bits(inp.residual)
        sets.append(([bits(p) for p in inp.partials], r, bits(inp.weight), np.empty_like(r)))
    for parts, r, w, y in sets[:2]:   # warm-up (page faults, thread pool)
        O.reduce_add_rms_norm(parts, r, w, cfg.eps, y=y)
    times, t_end = [], time.perf_counter() + budget_s
    while len(times) < 3 or time.perf_counter() < t_end:
        parts, r, w, y = sets[len(times) % nsets]
        t0 = time.perf_counter()
        O.reduce_add_rms_norm(parts, r, w, cfg.eps, y=y)
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    return {"value": round(sample.bytes / med / 1e9, 3), "unit": "GB/s", "cores": threads,
            "kind": "port",
            "sample": f"{len(times)} calls in {budget_s:.0f} s of P={sample.P} T={rows} H={sample.H} "
                      f"({sample.bytes} algorithmic bytes each) over {nsets} rotating input sets, "
                      f"median {med * 1e6:.0f} us/call, OpenMP over rows with {threads} threads"}


def time_weave(device, norm_cap, gemm_cap, steps=200):
    """Config 5: the bf16 MFMA GEMM of the 2458-row split (current stream) overlapped
    with the fused norm of the 1638-row split (second stream).  Every figure is the
    mean over `steps` back-to-back stages bracketed by HIP events; the norm inputs
    rotate through 8 sets (2.4 GB) so it reads cold HBM.  Calls are pre-bound ctypes
    calls (arguments validated once by the public shims) so that the host can enqueue
    a stage faster than the GPU runs it."""
    import torch
    from tokenweave_amd import _custom_ops as ops
    from tokenweave_amd import workloads as wl
    cfg, R = wl.C5_NORM, 8
    inps = [wl.make_norm_inputs(cfg, device, seed_offset=i) for i in range(R)]
    g = wl.make_gemm_inputs(device=device)
    Ta, K = g.a.shape
    N = g.b.shape[0]
    stages = [torch.zeros((Ta, N), dtype=torch.bfloat16, device=device) for _ in range(R)]
    main_s, side_s = torch.cuda.Stream(), torch.cuda.Stream()
    gemms, norms = {}, {}
    for cap in {0, gemm_cap}:
        gemms[cap] = [ops.bind_gemm_bf16_nt(stages[i], g.a, g.b, cap or None) for i in range(R)]
    for cap in {0, norm_cap}:
        norms[cap] = [ops.bind_reduce_add_rms_norm(inp.partials, inp.partials[0], inp.residual, inp.weight,
                                                   cfg.eps, cap or None) for inp in inps]
    pm, ps = main_s, side_s

    def gemm(i, cap, stream):
        gemms[cap][i % R](stream)

    def norm(i, cap, stream):
        norms[cap][i % R](stream)

    def weave(i):
        before = torch.cuda.Event()
        before.record(main_s)
        gemm(i, gemm_cap, pm)                 # GEMM first: it takes its CU budget ...
        side_s.wait_event(before)
        norm(i, norm_cap, ps)                 # ... and the norm fills the remaining CUs
        main_s.wait_stream(side_s)

    def timed(step):
        torch.cuda.synchronize()
        with torch.cuda.stream(main_s):
            for i in range(10):
                step(i)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(main_s)
            for i in range(steps):
                step(i)
            e1.record(main_s)
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / steps

    t_a = timed(lambda i: gemm(i, 0, pm))
    t_b = timed(lambda i: norm(i, 0, pm))
    t_ser = timed(lambda i: (gemm(i, 0, pm), norm(i, 0, pm)))
    t_ovl = timed(weave)
    flops = 2.0 * Ta * N * K
    return {"gemm_us": t_a, "norm_us": t_b, "serial_us": t_ser, "overlap_us": t_ovl,
            "speedup": t_ser / t_ovl, "overlap_eff": (t_ser - t_ovl) / min(t_a, t_b),
            "gemm_tflops_alone": flops / t_a / 1e6,
            "gemm_mfma_util_alone": flops / t_a / 1e6 / MFMA_BF16_PEAK_TFLOPS,
            "gemm_tflops_overlapped": flops / t_ovl / 1e6,
            "gemm_mfma_util_overlapped": flops / t_ovl / 1e6 / MFMA_BF16_PEAK_TFLOPS,
            "norm_gbps_alone": cfg.bytes / t_b / 1e3, "norm_gbps_overlapped": cfg.bytes / t_ovl / 1e3,
            "norm_cap": norm_cap, "gemm_cap": gemm_cap}


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one rank's work on ONE GPU; --gpus must be 1 "
                 "(this path has no collectives to scale across GPUs)")
    import torch
    from tokenweave_amd import workloads as wl
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    device = "cuda:0"
    torch.cuda.set_device(0)
    cfgs = wl.norm_configs()
    if args.workload not in cfgs:
        sys.exit(f"unknown workload {args.workload}; choose from {sorted(cfgs)}")
    cfg = cfgs[args.workload]
    if args.weave_only:
        w = time_weave(device, norm_cap=0, gemm_cap=128, steps=args.steps)
        print(json.dumps({"c5_weave": {k: (round(v, 4) if isinstance(v, float) else v) for k, v in w.items()}}),
              flush=True)
        return
    log(f"[bench] {torch.cuda.get_device_name(0)}; workload {cfg.name}: P={cfg.P} T={cfg.T} "
        f"H={cfg.H} bytes/call={cfg.bytes}")

    res = time_norm(cfg, args.steps, args.warmup, args.max_ctas, device)
    log(f"[bench] {res}")
    kernel_us = res["kernel_us_mean"]
    achieved = cfg.bytes / kernel_us / 1e3
    out = {
        "metric": "fused P-partial reduce+add+RMSNorm GB/s (% HBM peak), us/call, H=8192",
        "value": round(res["gbps"], 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(res["ms_per_step"], 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": cfg.name, "P": cfg.P, "T": cfg.T, "H": cfg.H, "eps": cfg.eps,
                   "bytes_per_call": cfg.bytes, "rotating_input_sets": res["nsets"],
                   "max_ctas": args.max_ctas},
        "pct_hbm_peak": round(100.0 * res["gbps"] / HBM_PEAK_GBPS, 2),
        "us_per_call": round(res["ms_per_step"] * 1e3, 3),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(cfg.name) if args.max_ctas == 0 else None,
                     "kernel": "row_norm_bf16_kernel<8,4,256,true,false,0>",
                     "kernel_us_mean": round(kernel_us, 3)},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, args.cpu_seconds)
        log(f"[bench] cpu_baseline {out['cpu_baseline']}")
    if args.calibration_copy:
        calibration_copies(device)
    if args.sweep:
        sweep = {}
        cfgs = dict(cfgs)
        cfgs["c2_unsharded@T2048"] = wl.C2.with_tokens(2048, "c2_unsharded@T2048")
        for name, c in cfgs.items():
            steps = max(50, min(2000, int(0.02 * 5e12 / c.bytes)))  # ~20 ms of kernel time
            r = time_norm(c, steps, max(5, steps // 10), args.max_ctas, device)
            warm_us = time_norm_warm(c, steps, args.max_ctas, device) if c.bytes < (200 << 20) else None
            sweep[name] = {"P": c.P, "T": c.T, "H": c.H, "bytes": c.bytes,
                           "us_per_call": round(r["ms_per_step"] * 1e3, 3),
                           "kernel_us": round(r["kernel_us_mean"], 3),
                           "kernel_us_cache_resident": None if warm_us is None else round(warm_us, 3),
                           "gbps": round(c.bytes / r["kernel_us_mean"] / 1e3, 1),
                           "pct_hbm_peak": round(c.bytes / r["kernel_us_mean"] / 1e3 / HBM_PEAK_GBPS * 100, 2)}
            log(f"[sweep] {name}: {sweep[name]}")
        # Grid-cap sweep of the headline shape (the reference's CTA sweep,
        # artifact/csvs/figure_10.csv: 2 ... 128 CTAs at 256 rows per GPU).
        c = cfgs["c2_llama70b_tp8_shard@T256"]
        cta = {}
        for cap in (2, 4, 8, 16, 32, 64, 128, 0):
            r = time_norm(c, 200, 20, cap, device)
            cta[str(cap or c.T)] = round(r["kernel_us_mean"], 2)
        sweep["c2_T256_us_by_max_ctas"] = cta
        log(f"[sweep] c2_T256_us_by_max_ctas: {cta}")
        # The reference's own microbenchmark grid for the P = 1 op (fused_add_rms_norm_cta,
        # H = 8192; artifact/csvs/figure_4.csv, one H100): context, not a baseline for the
        # headline metric, whose P = 8 form the reference does not publish.
        for rows, h100_us in ((64, 8.61), (256, 12.16), (1024, 29.92), (2048, 51.84), (4096, 96.51),
                              (32768, 712.4)):
            c = wl.C1.with_tokens(rows, f"p1_add_rms_norm@T{rows}")
            steps = max(50, min(2000, int(0.02 * 5e12 / c.bytes)))
            r = time_norm(c, steps, max(5, steps // 10), args.max_ctas, device)
            sweep[c.name] = {"P": 1, "T": rows, "H": c.H, "bytes": c.bytes,
                             "kernel_us": round(r["kernel_us_mean"], 3),
                             "gbps": round(c.bytes / r["kernel_us_mean"] / 1e3, 1),
                             "pct_hbm_peak": round(c.bytes / r["kernel_us_mean"] / 1e3 / HBM_PEAK_GBPS * 100, 2),
                             "reference_h100_us": h100_us}
            log(f"[sweep] {c.name}: {sweep[c.name]}")
        for name in ("c2_llama70b_tp8_shard@T256", "c2_unsharded@T2048"):
            c = cfgs[name]
            steps = max(50, min(2000, int(0.02 * 5e12 / c.bytes)))
            for epi in ("fp8_static", "fp8_dynamic", "int8_dynamic"):
                r = time_norm(c, steps, max(5, steps // 10), args.max_ctas, device, epi)
                b = quant_bytes(c, epi)
                sweep[f"{name}+{epi}"] = {"bytes": b, "kernel_us": round(r["kernel_us_mean"], 3),
                                          "gbps": round(b / r["kernel_us_mean"] / 1e3, 1),
                                          "pct_hbm_peak": round(b / r["kernel_us_mean"] / 1e3 / HBM_PEAK_GBPS * 100, 2)}
                log(f"[sweep] {name}+{epi}: {sweep[f'{name}+{epi}']}")
        w = time_weave(device, norm_cap=0, gemm_cap=128)
        sweep["c5_weave"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in w.items()}
        log(f"[sweep] c5_weave: {sweep['c5_weave']}")
        out["sweep"] = sweep
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
