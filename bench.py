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
  weave         config 5: GEMM of one token split (all eight partial sums, and one rank's)
                overlapped with the fused norm of the other split: alone, serial, overlapped.
  sweep         (--sweep) µs/call and GB/s of every benchmark configuration.
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
# kernel of known size), transcribed from the summary named beside each figure; this run
# does not measure them.  Workloads without a counter run: None.
MEASURED_TRAFFIC_BYTES = {
    "c2_llama70b_tp8_shard@T256": (46375250, "profiles/row_norm_bf16_c2_T256_pmc_traffic.md"),
}
# dominant kernel of a workload, as rocprofv3 names it
KERNEL_NAMES = {"c2_llama70b_tp8_shard@T256": "row_norm_bf16_kernel<8,4,256,true,false,0>"}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


_BENCH_LIB = None


def bench_lib():
    """benchlib/libtw_bench.so: measurement-only kernels (plain copy, row streams, empty
    kernel) and the norm kernels compiled with timeline stamps.  Built by `make -C
    benchlib`; the package neither builds nor loads it."""
    global _BENCH_LIB
    if _BENCH_LIB is None:
        path = os.path.join(ROOT, "benchlib", "libtw_bench.so")
        if not os.path.exists(path):
            sys.exit(f"{path} is missing: build it with `make -C benchlib`")
        L = ctypes.CDLL(path)
        vp, i64, ci, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
        L.twb_copy_bytes.argtypes = [vp, vp, i64, vp]
        L.twb_stream_rows.argtypes = [ctypes.POINTER(vp), vp, i64, i64, ci, vp]
        L.twb_trace_stream_rows.argtypes = [ctypes.POINTER(vp), vp, i64, i64, vp]
        L.twb_empty.argtypes = [ci, ci, vp]
        L.twb_clock_probe.argtypes = [vp, ci, vp]
        L.twb_touch_pages.argtypes = [vp, i64, vp, i64, ci, ci, vp, vp]
        L.twb_latency_chain.argtypes = [vp, i64, ci, i64, vp, vp, vp]
        L.twb_trace_reduce_add_rms_norm.argtypes = [ctypes.POINTER(vp), ci, vp, vp, vp, i64, i64, ci, f32, vp, vp]
        L.twb_gemm_loop.argtypes = [ci, ci, i64, vp, vp, vp, ci, vp]
        L.twb_lds_read_rate.argtypes = [ci, ci, ci, vp, vp, vp, ci, vp]
        L.twb_gemm_bf16_nt_tile.argtypes = [vp, vp, vp, i64, i64, i64, i64, ci, ci, vp]
        L.twb_last_error.restype = ctypes.c_char_p
        _BENCH_LIB = L
    return _BENCH_LIB


def bench_check(rc):
    if rc:
        raise RuntimeError(bench_lib().twb_last_error().decode())


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="c2_llama70b_tp8_shard@T256")
    ap.add_argument("--max-ctas", type=int, default=0, help="grid cap (0 = library default)")
    ap.add_argument("--sweep", action="store_true", help="also time every configuration")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-weave", action="store_true", help="leave the config 5 weave block out of the line")
    ap.add_argument("--gemm-only", action="store_true",
                    help="time only config 5's producer GEMM, one partial and all eight (for profiling)")
    ap.add_argument("--gemm-limits", action="store_true",
                    help="time the GEMM's k loop assembled from its parts (MFMAs, LDS fragment reads, operand "
                         "slabs global -> LDS) on L2-resident operands, and the LDS read rate, and print them")
    ap.add_argument("--gemm-scaling", action="store_true",
                    help="time the big GEMM kernel's 320 x 256 tile, one tile per compute unit, on 32 .. 256 "
                         "compute units (K = 1024 and 8192) with the shader clock rocm-smi reports meanwhile")
    ap.add_argument("--weave-only", action="store_true",
                    help="time only the GEMM + norm weave of config 5 and print its figures (for profiling)")
    ap.add_argument("--weave-power", action="store_true",
                    help="run every leg of config 5's stage for seconds each and print its time next to the "
                         "socket power, shader clock and memory-controller activity rocm-smi reports meanwhile")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="after the timed region, run the library's plain copy kernel on "
                         "buffers of known size (reference traffic for rocprofv3 --pmc runs)")
    ap.add_argument("--ceilings", action="store_true",
                    help="time the memory-system yardsticks (read-only row streams, the norm's traffic "
                         "without arithmetic, plain copy, empty kernel) at 256 and 2048 rows and print them")
    ap.add_argument("--host-cost", action="store_true",
                    help="measure the host time per call of the op's entry routes and print it")
    ap.add_argument("--timeline", action="store_true",
                    help="run the workload through the stamped build of the norm kernel and print the "
                         "per-workgroup timeline breakdown")
    ap.add_argument("--pretouch", type=int, default=0, metavar="STEP_BYTES",
                    help="before every launch, an untimed-by-itself helper kernel reads one dword per STEP_BYTES "
                         "of the launch's inputs from every XCD (address translations warm, data still cold); "
                         "for counter runs")
    ap.add_argument("--graph-replay", action="store_true",
                    help="time the workload under HIP-graph replay (two passes over the rotating input sets in "
                         "one graph) and print microseconds per launch")
    ap.add_argument("--tlb-latency", action="store_true",
                    help="measure the latency of dependent cold reads with and without a cached address "
                         "translation and print it")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline")
    return ap.parse_args()


class NormRunner:
    """One bound call (tokenweave_amd.ops.BoundOp: arguments checked once, a single
    ctypes call per launch) for each input set, so that the host enqueues a step
    faster than the GPU runs it."""

    def __init__(self, cfg, nsets, max_ctas, device, epilogue="bf16", split=None, pretouch=0):
        import torch
        from tokenweave_amd import _custom_ops as ops
        from tokenweave_amd import _lib
        from tokenweave_amd import workloads as wl
        self.calls = []
        self.inputs = []
        self.pretouch = pretouch
        self.sink = torch.zeros(256, dtype=torch.uint8, device=device) if pretouch else None
        L = _lib.lib()
        for i in range(nsets):
            inp = wl.make_norm_inputs(cfg, device, seed_offset=i)
            self.inputs.append(inp)
            if epilogue == "bf16":
                # y lands on this rank's staging rows (rank 0)
                op = ops.bind_reduce_add_rms_norm(inp.partials, inp.partials[0], inp.residual, inp.weight,
                                                  cfg.eps, max_ctas or None, split=split)
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

    def touch(self, i, stream, step_bytes):
        """Page-touch the inputs of step i: one dword per `step_bytes` of the P partial
        buffers and of the residual, read from every XCD."""
        inp = self.inputs[i % len(self.inputs)]
        st, r = inp.staging, inp.residual
        bench_check(bench_lib().twb_touch_pages(st.data_ptr(), st.numel() * 2, r.data_ptr(), r.numel() * 2,
                                                step_bytes, 4, self.sink.data_ptr(), stream.cuda_stream))

    def step(self, i, stream):
        if self.pretouch:
            self.touch(i, stream, self.pretouch)
        self.calls[i % len(self.calls)](stream)


def quant_bytes(cfg, epilogue):
    """Algorithmic bytes with a quantised output: one byte per element instead of two,
    plus one float per row for the dynamic kinds."""
    return cfg.bytes - cfg.T * cfg.H + (4 * cfg.T if epilogue.endswith("dynamic") else 4)


PREROLL_MS = 40.0   # untimed launches ahead of the warm-up: clocks ramped, queues and TLBs in steady state
REGIONS = 21        # timed regions of exactly `steps` launches each; the median region is reported


LEAD_IN = 40        # untimed launches ahead of an event bracket (the bracket starts in a busy queue)


def graph_replay_us(runner, launches, replays=5, brackets=7):
    """`launches` consecutive steps of `runner` captured into one HIP graph, replayed `replays`
    times per HIP-event bracket: microseconds per launch, median / min / max of `brackets`."""
    import torch
    main_s, _ = weave_streams()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=main_s):
        for i in range(launches):
            runner.step(i, main_s)
    ts = []
    with torch.cuda.stream(main_s):
        g.replay()
        torch.cuda.synchronize()
        for _ in range(brackets):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(main_s)
            for _ in range(replays):
                g.replay()
            e1.record(main_s)
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3 / (replays * launches))
    del g
    return statistics.median(ts), min(ts), max(ts)


def time_norm(cfg, steps, warmup, max_ctas, device, epilogue="bf16", regions=REGIONS, preroll_ms=PREROLL_MS,
              lead_in=LEAD_IN, split=None, pretouch=0, graph=False):
    """After an untimed pre-roll and `warmup` warm-up launches, times `regions` regions of
    exactly `steps` back-to-back launches twice over: by the wall clock between two device
    synchronisations (ms_per_step, gbps), and by HIP events on the launch stream around
    `steps` launches that follow `lead_in` untimed ones (event_us_per_launch: mean launch
    duration, gaps included).  Medians over the regions, plus the spread."""
    import torch
    nsets = max(2, min(256, -(-ROTATION_BYTES // cfg.bytes)))
    free, _ = torch.cuda.mem_get_info()
    set_bytes = (cfg.P + 1) * cfg.T * cfg.H * 2 + cfg.H * 2
    nsets = max(2, min(nsets, int(free * 0.6) // (set_bytes * 3)))  # fp32 staging while generating
    runner = NormRunner(cfg, nsets, max_ctas, device, epilogue, split, pretouch)
    stream = torch.cuda.current_stream()
    it = 0
    preroll_steps = max(warmup, int(preroll_ms * 1e3 / max(2.0, cfg.bytes / 6e6)))
    for _ in range(preroll_steps):
        runner.step(it, stream)
        it += 1
    torch.cuda.synchronize()
    for _ in range(warmup):
        runner.step(it, stream)
        it += 1
    # (a) wall clock: exactly `steps` launches between two synchronisations, from an idle queue
    walls = []
    for _ in range(regions):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            runner.step(it, stream)
            it += 1
        torch.cuda.synchronize()
        walls.append(time.perf_counter() - t0)
    # (b) launch duration: HIP events around exactly `steps` launches that follow `lead_in`
    # untimed launches on the same stream, so that the bracket starts in a busy queue (what
    # a per-kernel trace measures) and not with the idle-to-first-dispatch latency
    events = []
    for _ in range(regions):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        for _ in range(lead_in):
            runner.step(it, stream)
            it += 1
        e0.record(stream)
        for _ in range(steps):
            runner.step(it, stream)
            it += 1
        e1.record(stream)
        torch.cuda.synchronize()
        events.append(e0.elapsed_time(e1) * 1e-3)
    wall, ev = statistics.median(walls), statistics.median(events)
    res = {"ms_per_step": wall * 1e3 / steps, "gbps": cfg.bytes * steps / wall / 1e9,
           "nsets": nsets, "event_us_per_launch": ev * 1e6 / steps,
           "event_us_per_launch_min": min(events) * 1e6 / steps,
           "event_us_per_launch_max": max(events) * 1e6 / steps,
           "regions": regions, "preroll_steps": preroll_steps, "lead_in_steps": lead_in}
    if graph:
        # (c) the same launches with no host in the loop: two passes over the input sets in one graph
        res["graph_replay_us_per_launch"], _, _ = graph_replay_us(runner, 2 * nsets)
    del runner
    torch.cuda.empty_cache()
    return res


def time_tlb_latency(device):
    """What an address-translation miss costs a cold read.  One lane reads dwords one after
    the other (each waits for the one before) from two 4 GiB regions A and B, always from
    cache lines that nothing has read since they were written (cold data):
      pass 1  A, one read per 2 MiB                      (translations as the fill left them)
      pass 2  B likewise                                 (pushes A's translations out of any TLB
                                                          that cannot hold 2 x 2048 of them)
      pass 3  A again, other lines of the same pages     (warm only if the TLBs reach > 8 GiB)
      pass 4  A again, other lines, right after pass 3   (translations warm, data cold)
      pass 5  A, 32 reads per 64 KiB inside 2 MiB pages  (same page back to back: the floor)
    Microseconds per read: median and 90th percentile."""
    import numpy as np
    import torch
    L = bench_lib()
    sp = torch.cuda.current_stream().cuda_stream
    size = 4 << 30
    A = torch.empty(size, dtype=torch.uint8, device=device)
    B = torch.empty(size, dtype=torch.uint8, device=device)
    A.random_(0, 200)
    B.random_(0, 200)
    torch.cuda.synchronize()
    n = size // (2 << 20)
    out = torch.zeros(n * 4, dtype=torch.int32, device=device)
    sink = torch.zeros(4, dtype=torch.int32, device=device)

    def chain(buf, stride, count, offset):
        bench_check(L.twb_latency_chain(buf.data_ptr(), stride, count, offset, out.data_ptr(), sink.data_ptr(), sp))
        torch.cuda.synchronize()
        t = out[:count].cpu().numpy().astype(np.float64) * 0.01
        return {"reads": count, "median_us": round(float(np.median(t)), 3), "p10_us": round(float(np.percentile(t, 10)), 3),
                "p90_us": round(float(np.percentile(t, 90)), 3)}

    res = {"region_bytes": size, "page_stride_bytes": 2 << 20}
    res["pass1_A_first_touch"] = chain(A, 2 << 20, n, 0)
    res["pass2_B_first_touch"] = chain(B, 2 << 20, n, 0)
    res["pass3_A_after_B_other_lines"] = chain(A, 2 << 20, n, 8192)
    res["pass4_A_again_other_lines"] = chain(A, 2 << 20, n, 16384)
    res["pass5_A_64KiB_steps_inside_pages"] = chain(A, 64 << 10, 4096, 32768)
    res["pass6_A_first_256_pages_again"] = chain(A, 2 << 20, 256, 24576)
    res["pass7_A_first_256_pages_again"] = chain(A, 2 << 20, 256, 28672)
    for k, v in res.items():
        log(f"[tlb-latency] {k}: {v}")
    return res


def time_graph_replay(cfg, max_ctas, device, cycles=2, replays=5, brackets=7):
    """The workload under HIP-graph replay: `cycles` passes over the rotating input sets
    (4 GiB, cold data) captured into one graph, timed per launch by HIP events around
    `replays` replays (median of `brackets`): the launches back to back with no host in the
    loop — what is left of the launch-to-launch gap when the host is out of the picture."""
    import torch
    nsets = max(2, min(256, -(-ROTATION_BYTES // cfg.bytes)))
    runner = NormRunner(cfg, nsets, max_ctas, device)
    med, lo, hi = graph_replay_us(runner, cycles * nsets, replays, brackets)
    out = {"workload": cfg.name, "launches_per_graph": cycles * nsets, "rotating_input_sets": nsets,
           "replays_per_bracket": replays, "brackets": brackets,
           "us_per_launch": round(med, 3), "min": round(lo, 3), "max": round(hi, 3)}
    del runner
    torch.cuda.empty_cache()
    return out


CALIBRATION_COPY_BYTES = 256 << 20


def calibration_copies(device, n=8):
    """n launches of tw_copy_bytes, each reading and writing CALIBRATION_COPY_BYTES of
    memory that was not touched recently (4 source/destination pairs = 2 GiB)."""
    import torch
    L = bench_lib()
    pairs = [(torch.ones(CALIBRATION_COPY_BYTES // 2, dtype=torch.bfloat16, device=device),
              torch.empty(CALIBRATION_COPY_BYTES // 2, dtype=torch.bfloat16, device=device))
             for _ in range(4)]
    torch.cuda.synchronize()
    sp = torch.cuda.current_stream().cuda_stream
    for i in range(n):
        src, dst = pairs[i % 4]
        bench_check(L.twb_copy_bytes(dst.data_ptr(), src.data_ptr(), CALIBRATION_COPY_BYTES, sp))
    torch.cuda.synchronize()


def event_time(fn, steps, stream, warm=20, regions=5):
    """Median over `regions` of the HIP-event bracket around `steps` back-to-back calls of
    fn(i), in microseconds per call."""
    import torch
    it = 0
    for _ in range(warm):
        fn(it)
        it += 1
    out = []
    for _ in range(regions):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(steps):
            fn(it)
            it += 1
        e1.record(stream)
        torch.cuda.synchronize()
        out.append(e0.elapsed_time(e1) * 1e3 / steps)
    return statistics.median(out)


def time_ceilings(device):
    """What the memory system gives kernels with the norm kernel's launch shape (one
    256-lane workgroup per 16 KiB row, nine input streams, 4 GiB of rotating operands so
    every launch reads cold HBM), at 256 and 2048 rows of hidden size 8192."""
    import torch
    from tokenweave_amd import _lib
    from tokenweave_amd import workloads as wl
    L, TL = bench_lib(), _lib.lib()
    stream = torch.cuda.current_stream()
    sp = stream.cuda_stream
    vp = ctypes.c_void_p
    sink = torch.zeros(4096, dtype=torch.uint8, device=device)
    out = {}
    for rows in (256, 2048):
        cfg = wl.C2.with_tokens(rows)
        nsets = max(2, min(256, -(-ROTATION_BYTES // cfg.bytes)))
        sets = []
        for i in range(nsets):
            inp = wl.make_norm_inputs(cfg, device, seed_offset=i)
            ptrs = (vp * 9)(*([p.data_ptr() for p in inp.partials] + [inp.residual.data_ptr()]))
            sets.append((inp, ptrs))
        steps = max(50, min(2000, int(0.02 * 5e12 / cfg.bytes)))
        read_bytes = 9 * rows * cfg.H * 2
        traffic_bytes = read_bytes + 2 * rows * cfg.H * 2
        res = {}

        def streams(write):
            def fn(i):
                inp, ptrs = sets[i % nsets]
                bench_check(L.twb_stream_rows(ptrs, sink.data_ptr(), rows, cfg.H, write, sp))
            return event_time(fn, steps, stream)

        us = streams(0)
        res["read_only_9_streams"] = {"bytes": read_bytes, "us": round(us, 3), "gbps": round(read_bytes / us / 1e3, 1)}
        us = streams(1)
        res["norm_traffic_no_arithmetic"] = {"bytes": traffic_bytes, "us": round(us, 3),
                                             "gbps": round(traffic_bytes / us / 1e3, 1)}
        us = streams(2)
        res["write_only_2_streams"] = {"bytes": traffic_bytes - read_bytes, "us": round(us, 3),
                                       "gbps": round((traffic_bytes - read_bytes) / us / 1e3, 1)}
        # plain copy moving the same number of bytes in total (half read, half written)
        half = (traffic_bytes // 2) // 16 * 16
        srcs = [inp.staging.view(-1).view(torch.uint8) for inp, _ in sets]
        dsts = [torch.empty(half, dtype=torch.uint8, device=device) for _ in range(min(nsets, 8))]

        def copy(i):
            bench_check(L.twb_copy_bytes(dsts[i % len(dsts)].data_ptr(), srcs[i % nsets].data_ptr(), half, sp))
        us = event_time(copy, steps, stream)
        res["plain_copy_same_total_bytes"] = {"bytes": 2 * half, "us": round(us, 3),
                                              "gbps": round(2 * half / us / 1e3, 1)}

        def norm(i):
            inp, ptrs = sets[i % nsets]
            rc = TL.tw_reduce_add_rms_norm(ctypes.cast(ptrs, ctypes.POINTER(vp)), cfg.P, inp.partials[0].data_ptr(),
                                           inp.residual.data_ptr(), inp.weight.data_ptr(), cfg.T, cfg.H, 0,
                                           cfg.eps, sp)
            if rc:
                _lib.check(rc)
        us = event_time(norm, steps, stream)
        res["norm_kernel"] = {"bytes": cfg.bytes, "us": round(us, 3), "gbps": round(cfg.bytes / us / 1e3, 1)}
        us = event_time(lambda i: bench_check(L.twb_empty(rows, 256, sp)), 2000, stream)
        res["empty_kernel_same_grid"] = {"us": round(us, 3)}
        out[f"rows{rows}"] = res
        log(f"[ceilings] rows={rows}: {res}")
        del sets, srcs, dsts
        torch.cuda.empty_cache()
    return out


def time_timeline(cfg, device, launches=200, burst=6):
    """Runs the stamped build of the norm kernel in `launches` bursts of `burst` back-to-back launches on
    rotating inputs, keeps the stamps of each burst's last launch (a launch that starts on an idle GPU
    begins 0.4 - 0.7 us later on half of the XCCs; one that follows another does not) and reduces the
    per-row stamps (wall clock, 10 ns units) to a breakdown of one launch: microseconds;
    `min`/`median`/`max` are over the rows of a launch, each then the median over launches."""
    import numpy as np
    import torch
    from tokenweave_amd import workloads as wl
    L = bench_lib()
    stream = torch.cuda.current_stream()
    sp = stream.cuda_stream
    vp = ctypes.c_void_p
    nsets = max(2, min(256, -(-ROTATION_BYTES // cfg.bytes)))
    sets = []
    for i in range(nsets):
        inp = wl.make_norm_inputs(cfg, device, seed_offset=i)
        sets.append((inp, (vp * cfg.P)(*[p.data_ptr() for p in inp.partials])))
    slot = torch.zeros((cfg.T, 8), dtype=torch.int64, device=device)
    trace = torch.zeros((launches, cfg.T, 8), dtype=torch.int64, device=device)

    def call(i):
        inp, ptrs = sets[i % nsets]
        bench_check(L.twb_trace_reduce_add_rms_norm(ptrs, cfg.P, inp.partials[0].data_ptr(),
                                                    inp.residual.data_ptr(), inp.weight.data_ptr(), cfg.T, cfg.H,
                                                    0, cfg.eps, slot.data_ptr(), sp))
    for i in range(50):
        call(i)
    torch.cuda.synchronize()
    n, event_ms = 50, []
    for s in range(launches):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        call(n)
        e0.record(stream)
        for i in range(1, burst):
            call(n + i)
        e1.record(stream)
        n += burst
        torch.cuda.synchronize()
        event_ms.append(e0.elapsed_time(e1) / (burst - 1))
        trace[s].copy_(slot)
    bench_check(L.twb_trace_end())   # later launches write no stamps: `slot` may be freed
    event_us = sorted(event_ms)[len(event_ms) // 2] * 1e3
    t = trace.cpu().numpy()
    st = t[:, :, :6].astype(np.float64) * 0.01          # 100 MHz wall clock -> us
    xcc = (t[:, :, 6] >> 32) & 0xf
    rel = st - st[:, :, 0].min(axis=1)[:, None, None]   # relative to the launch's first row begin

    def med(a):
        return float(np.median(a))

    def rows_stat(a):
        return {"min": round(med(a.min(axis=1)), 2), "median": round(med(np.median(a, axis=1)), 2),
                "max": round(med(a.max(axis=1)), 2)}
    span = rel[:, :, 5].max(axis=1)
    out = {
        "workload": cfg.name, "launches": launches, "burst": burst,
        "event_us_per_launch_with_stamps": round(event_us, 3),
        "first_row_begin_to_last_ack_us": {"median": round(med(span), 2), "min": round(float(span.min()), 2),
                                           "max": round(float(span.max()), 2)},
        "launch_to_launch_minus_span_us": round(event_us - med(span), 2),
        "row_begin_after_first_row_us": rows_stat(rel[:, :, 0]),
        "loads_returned_after_row_begin_us": rows_stat(st[:, :, 1] - st[:, :, 0]),
        "loads_returned_after_first_row_us": rows_stat(rel[:, :, 1]),
        "residual_stores_issued_after_loads_us": rows_stat(st[:, :, 2] - st[:, :, 1]),
        "row_sum_after_residual_stores_us": rows_stat(st[:, :, 3] - st[:, :, 2]),
        "y_stores_issued_after_row_sum_us": rows_stat(st[:, :, 4] - st[:, :, 3]),
        "stores_acknowledged_after_y_issue_us": rows_stat(st[:, :, 5] - st[:, :, 4]),
        "row_end_after_first_row_us": rows_stat(rel[:, :, 5]),
        "rows_per_xcc_first_launch": [int((xcc[0] == x).sum()) for x in range(8)],
        "median_row_begin_by_xcc_us": [round(med(rel[:, :, 0][xcc == x]), 2) if (xcc == x).any() else None
                                       for x in range(8)],
        "median_loads_returned_by_xcc_us": [round(med(rel[:, :, 1][xcc == x]), 2) if (xcc == x).any() else None
                                            for x in range(8)],
        "median_row_end_by_xcc_us": [round(med(rel[:, :, 5][xcc == x]), 2) if (xcc == x).any() else None
                                     for x in range(8)],
    }
    return out


def time_arrivals(cfg, device, launches=100):
    """The stand-in kernel (the norm's traffic, no arithmetic) with a stamp after each of
    the nine streams has returned: when, after the launch's first row begins, the data
    of a row arrives.  Microseconds; min / median / max over the rows of a launch, each
    the median over launches."""
    import numpy as np
    import torch
    from tokenweave_amd import workloads as wl
    L = bench_lib()
    stream = torch.cuda.current_stream()
    sp = stream.cuda_stream
    vp = ctypes.c_void_p
    nsets = max(2, min(256, -(-ROTATION_BYTES // cfg.bytes)))
    sets = []
    for i in range(nsets):
        inp = wl.make_norm_inputs(cfg, device, seed_offset=i)
        sets.append((inp, (vp * 9)(*([p.data_ptr() for p in inp.partials] + [inp.residual.data_ptr()]))))
    trace = torch.zeros((launches, cfg.T, 16), dtype=torch.int64, device=device)
    for i in range(launches + 20):
        inp, ptrs = sets[i % nsets]
        bench_check(L.twb_trace_stream_rows(ptrs, trace[max(0, i - 20)].data_ptr(), cfg.T, cfg.H, sp))
    torch.cuda.synchronize()
    st = trace.cpu().numpy()[:, :, :12].astype(np.float64) * 0.01
    rel = st - st[:, :, 0].min(axis=1)[:, None, None]
    names = ["row_begins"] + [f"stream_{s}_returned" for s in range(9)] + ["stores_issued", "stores_acknowledged"]
    out = {"workload": cfg.name, "launches": launches}
    for j, n in enumerate(names):
        a = rel[:, :, j]
        out[n] = {"min": round(float(np.median(a.min(axis=1))), 2),
                  "median": round(float(np.median(np.median(a, axis=1))), 2),
                  "max": round(float(np.median(a.max(axis=1))), 2)}
    return out


def host_cost(device, calls=3000):
    """Host time per call (the loop's wall time without a device synchronisation; the GPU
    queue is deep enough not to block it) of the ways into the op, on a decode-size batch
    (8 rows, P = 8, H = 8192), with torch.add as the yardstick.  Microseconds."""
    import torch
    import tokenweave_amd as tw
    from tokenweave_amd import _custom_ops as ops
    T, H, P = 8, 8192, 8
    buf = tw.PartialsBuffer(P, T, H, rank=0, device=device)
    buf.storage.normal_()
    res = torch.randn(T, H, device=device).bfloat16()
    layer = tw.RMSNorm(H, eps=1e-5, dtype=torch.bfloat16).to(device)
    hs = buf.hidden_states(T)
    parts = [buf.slot(p)[:T] for p in range(P)]
    w = layer.weight.data
    x = torch.randn(T, H, device=device).bfloat16()
    bound = ops.bind_reduce_add_rms_norm(parts, parts[0], res, w, 1e-5)
    st = torch.cuda.current_stream()
    mc = buf.multicast_ptr
    ways = {
        "BoundOp(stream)": lambda: bound(st),
        "ops.fused_add_rms_norm": lambda: ops.fused_add_rms_norm(hs, res, w, 1e-5),
        "torch.ops.tokenweave_amd.fused_add_rms_norm": lambda: torch.ops.tokenweave_amd.fused_add_rms_norm(hs, res, w, 1e-5),
        "ops.via_ctypes.fused_add_rms_norm": lambda: ops.via_ctypes.fused_add_rms_norm(hs, res, w, 1e-5),
        "ops.fused_rs_ln_ag_cta": lambda: ops.fused_rs_ln_ag_cta(hs, res, w, mc, 0, 0, P, 0, 1e-5),
        "ops.via_ctypes.fused_rs_ln_ag_cta": lambda: ops.via_ctypes.fused_rs_ln_ag_cta(hs, res, w, mc, 0, 0, P, 0, 1e-5),
        "ops.reduce_add_rms_norm(8 tensors)": lambda: ops.reduce_add_rms_norm(parts, parts[0], res, w, 1e-5),
        "RMSNorm(x, residual)": lambda: layer(hs, res),
        "RMSNorm(x, residual, fused_ar=True, ...)": lambda: layer(hs, res, MAX_CTAS=None, fused_ar=True,
                                                                   symm_mem_hdl=buf, rank=0, world_size=P, offset=0),
        "fused_allreduce_layernorm": lambda: tw.fused_allreduce_layernorm(layer, hs, res, buf, T // P, 0, P, 0),
        "torch.add(x, x, out=x)": lambda: torch.add(x, x, out=x),
    }
    out = {"compiled_binding": bool(ops.COMPILED_BINDING), "calls": calls}
    for name, fn in ways.items():
        for _ in range(200):
            fn()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            t0 = time.perf_counter()
            for _ in range(calls):
                fn()
            t1 = time.perf_counter()
            torch.cuda.synchronize()
            us = (t1 - t0) * 1e6 / calls
            best = us if best is None else min(best, us)
        out[name] = round(best, 2)
        log(f"[host] {name}: {best:.2f} us")
    return out


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


def host_cpu():
    """(model string, physical cores, logical CPUs) of the host, from /proc/cpuinfo."""
    model, cores, logical = "unknown", set(), 0
    try:
        phys = core = None
        with open("/proc/cpuinfo") as f:
            for line in f:
                key, _, val = line.partition(":")
                key, val = key.strip(), val.strip()
                if key == "model name":
                    model = val
                elif key == "processor":
                    logical += 1
                elif key == "physical id":
                    phys = val
                elif key == "core id":
                    core = val
                elif not key and phys is not None and core is not None:
                    cores.add((phys, core))
                    phys = core = None
        if phys is not None and core is not None:
            cores.add((phys, core))
    except OSError:
        pass
    return model, len(cores) or None, logical or (os.cpu_count() or 1)


def cpu_baseline(cfg, budget_s):
    """Times the CPU checker on a bounded sample of the workload: the same shapes (rows
    capped at 1024), rotating through input sets of 1 GiB in total so that, like the GPU
    legs, every call reads memory and not a cache.  Two legs: OpenMP over rows with all the
    threads this process is given (OMP_NUM_THREADS, else the logical CPUs) for two thirds of
    `budget_s` seconds -> value, cores; and one thread for the rest -> single_thread."""
    import numpy as np
    import torch
    from oracle import tw_oracle as O
    from tokenweave_amd import workloads as wl
    model, physical, logical = host_cpu()
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or logical
    rows = min(cfg.T, 1024)
    sample = cfg.with_tokens(rows)
    bits = lambda t: np.ascontiguousarray(t.contiguous().view(torch.int16).numpy().view(np.uint16))
    nsets = max(2, min(32, -(-(1 << 30) // sample.bytes)))
    sets = []
    for i in range(nsets):
        inp = wl.make_norm_inputs(sample, "cpu", seed_offset=i)
        r = bits(inp.residual)
        sets.append(([bits(p) for p in inp.partials], r, bits(inp.weight), np.empty_like(r)))
    O.lib()
    gomp = ctypes.CDLL("libgomp.so.1")   # the OpenMP runtime the checker is linked against

    def leg(nthreads, seconds):
        gomp.omp_set_num_threads(nthreads)
        for parts, r, w, y in sets[:2]:   # warm-up (page faults, thread pool)
            O.reduce_add_rms_norm(parts, r, w, cfg.eps, y=y)
        times, t_end = [], time.perf_counter() + seconds
        while len(times) < 3 or time.perf_counter() < t_end:
            parts, r, w, y = sets[len(times) % nsets]
            t0 = time.perf_counter()
            O.reduce_add_rms_norm(parts, r, w, cfg.eps, y=y)
            times.append(time.perf_counter() - t0)
        return statistics.median(times), len(times)

    med, n = leg(threads, budget_s * 2.0 / 3.0)
    med1, n1 = leg(1, budget_s / 3.0)
    gomp.omp_set_num_threads(threads)
    return {"value": round(sample.bytes / med / 1e9, 3), "unit": "GB/s", "cores": threads,
            "kind": "port", "cpu_model": model, "physical_cores": physical, "logical_cpus": logical,
            "single_thread": {"value": round(sample.bytes / med1 / 1e9, 3), "unit": "GB/s", "cores": 1,
                              "us_per_call": round(med1 * 1e6, 1), "calls": n1},
            "sample": f"{n} calls in {budget_s * 2 / 3:.0f} s of P={sample.P} T={rows} H={sample.H} "
                      f"({sample.bytes} algorithmic bytes each) over {nsets} rotating input sets, "
                      f"median {med * 1e6:.0f} us/call, OpenMP over rows with {threads} threads; then "
                      f"{n1} calls in {budget_s / 3:.0f} s with one thread, median {med1 * 1e6:.0f} us/call"}


def weave_streams():
    """The two streams of every weave measurement, created once (the tuner's pair: HIP spreads
    streams over a few hardware queues, 4 by default, in creation order, and two streams that
    land on one queue run their kernels one after the other)."""
    from tokenweave_amd.tune_weave import weave_streams as pair
    return pair()


WEAVE_REGIONS = 11   # rounds in which the legs of a weave measurement take turns


def time_weave(device, form="eight_partials", gemm_caps=(128,), norm_cap=0, steps=20, regions=WEAVE_REGIONS):
    """Config 5: the bf16 MFMA GEMM of the 2458-row split on the current stream overlapped with
    the fused norm of the 1638-row split on a second stream.  form "eight_partials": the
    producer of all P = 8 row-parallel partial sums of the split (one launch,
    tw_gemm_bf16_nt_partials, into the 8 staging slots); "one_partial": one rank's GEMM.

    The legs — GEMM alone, norm alone, both on one stream (serial), and the two-stream stage
    for every GEMM compute-unit budget in `gemm_caps` — take turns region by region
    (`regions` rounds; in each, every leg runs 2 untimed and `steps` timed stages between
    HIP events), and each figure is the median over the rounds: every leg sees the same
    mix of clock and power states, where back-to-back legs of seconds each would not.  A
    one-wave clock probe follows each leg's timed stages and reads the shader clock the
    leg left behind.  The serial leg is also timed with an event between its two kernels
    (`*_us_in_serial`).  The norm inputs rotate through 8 sets (2.4 GB) so it reads cold HBM, the GEMM
    outputs through as many staging buffers.  Calls are pre-bound (arguments validated once
    by the public shims) so that the host enqueues a stage faster than the GPU runs it."""
    import torch
    from tokenweave_amd import _custom_ops as ops
    from tokenweave_amd import workloads as wl
    from tokenweave_amd.tune_weave import interleaved_medians
    cfg = wl.C5_NORM
    P = 8 if form == "eight_partials" else 1
    R = 4 if P == 8 else 8
    inps = [wl.make_norm_inputs(cfg, device, seed_offset=i) for i in range(8)]
    gs = wl.make_partials_gemm_inputs(P, device=device)
    Ta, K = gs[0].a.shape
    N = gs[0].b.shape[0]
    stages = [torch.zeros((P, Ta, N), dtype=torch.bfloat16, device=device) for _ in range(R)]
    main_s, side_s = weave_streams()

    def bind_gemm(i, cap):
        if P == 1:
            return ops.bind_gemm_bf16_nt(stages[i][0], gs[0].a, gs[0].b, cap or None)
        return ops.bind_gemm_bf16_nt_partials([stages[i][p] for p in range(P)], [g.a for g in gs],
                                              [g.b for g in gs], cap or None)
    gemms = {cap: [bind_gemm(i, cap) for i in range(R)] for cap in {0, *gemm_caps}}
    norms = {cap: [ops.bind_reduce_add_rms_norm(inp.partials, inp.partials[0], inp.residual, inp.weight,
                                                cfg.eps, cap or None) for inp in inps] for cap in {0, norm_cap}}

    def gemm(i, cap, stream):
        gemms[cap][i % R](stream)

    def norm(i, cap, stream):
        norms[cap][i % 8](stream)

    def weave(cap):
        def stage(i):
            before = torch.cuda.Event()
            before.record(main_s)
            gemm(i, cap, main_s)                  # GEMM first: it takes its CU budget ...
            side_s.wait_event(before)
            norm(i, norm_cap, side_s)             # ... and the norm fills the remaining CUs
            main_s.wait_stream(side_s)
        return stage

    legs = {"gemm": lambda i: gemm(i, 0, main_s), "norm": lambda i: norm(i, 0, main_s),
            "serial": lambda i: (gemm(i, 0, main_s), norm(i, 0, main_s))}
    for cap in gemm_caps:
        legs[f"weave/{cap}"] = weave(cap)

    # shader clock right after each leg's timed stages
    BL = bench_lib()
    probe_out = torch.zeros((len(legs) * regions, 2), dtype=torch.int64, device=device)
    probes = {name: [] for name in legs}

    def probe(name):
        k = sum(len(v) for v in probes.values())
        bench_check(BL.twb_clock_probe(probe_out[k].data_ptr(), 20, main_s.cuda_stream))
        probes[name].append(k)

    res = interleaved_medians(legs, main_s, steps, regions=regions, after_region=probe)
    pr = probe_out.cpu().numpy().astype(float)
    clock = {name: round(statistics.median(pr[k, 0] / max(pr[k, 1], 1.0) / 10.0 for k in ks), 3)
             for name, ks in probes.items()}   # cycles per 10 ns tick -> GHz

    # the serial stage with an event between its kernels: what each takes inside the serial stage
    g_in, n_in = [], []
    with torch.cuda.stream(main_s):
        it = 0
        for _ in range(regions):
            evs = []
            for _ in range(steps):
                e = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
                e[0].record(main_s)
                gemm(it, 0, main_s)
                e[1].record(main_s)
                norm(it, 0, main_s)
                e[2].record(main_s)
                evs.append(e)
                it += 1
            torch.cuda.synchronize()
            g_in.append(statistics.mean(e[0].elapsed_time(e[1]) for e in evs[2:]) * 1e3)
            n_in.append(statistics.mean(e[1].elapsed_time(e[2]) for e in evs[2:]) * 1e3)

    t_a, t_b, t_ser = res["gemm"]["us"], res["norm"]["us"], res["serial"]["us"]
    by_cap = {cap: res[f"weave/{cap}"]["us"] for cap in gemm_caps}
    best_cap = min(by_cap, key=by_cap.get)
    t_ovl = by_cap[best_cap]
    flops = 2.0 * P * Ta * N * K
    # serial is two kernels that cannot overlap: it cannot undercut the longer one, and it
    # should be the sum of the two alone up to what the different duty cycle does to the clock
    consistent = t_ser >= max(t_a, t_b) * 0.995 and abs(t_ser - (t_a + t_b)) <= 0.05 * (t_a + t_b)
    out = {"form": form, "gemm_us": t_a, "norm_us": t_b, "serial_us": t_ser, "overlap_us": t_ovl,
           "speedup": t_ser / t_ovl,
           "overlap_eff": (t_ser - t_ovl) / min(t_a, t_b) if consistent else None,
           "legs_consistent": consistent,
           "serial_vs_sum_of_alone": t_ser / (t_a + t_b),
           "gemm_us_in_serial": statistics.median(g_in), "norm_us_in_serial": statistics.median(n_in),
           "us_min_max": {k: [round(v["min"], 2), round(v["max"], 2)] for k, v in res.items()},
           "shader_clock_ghz_after_leg": clock,
           "gemm_tflops_alone": flops / t_a / 1e6,
           "gemm_mfma_util_alone": flops / t_a / 1e6 / MFMA_BF16_PEAK_TFLOPS,
           "gemm_mfma_util_in_stage": flops / t_ovl / 1e6 / MFMA_BF16_PEAK_TFLOPS,
           "norm_gbps_alone": cfg.bytes / t_b / 1e3, "norm_gbps_in_stage": cfg.bytes / t_ovl / 1e3,
           "norm_cap": norm_cap, "gemm_cus": best_cap, "stages_per_region": steps, "regions": regions,
           "overlap_us_by_gemm_cus": {str(c): round(v, 2) for c, v in by_cap.items()}}
    del gemms, norms, stages, inps, gs
    torch.cuda.empty_cache()
    return {k: (round(v, 4) if isinstance(v, float) else v) for k, v in out.items()}


def time_gemm_only(device, steps=200):
    """Config 5's producer GEMM by itself, both forms, for profiling: [2458, 1024] x [8192, 1024]^T
    into rotating staging buffers, `steps` launches of one partial and steps / 4 of all eight."""
    import torch
    from tokenweave_amd import _custom_ops as ops
    from tokenweave_amd import workloads as wl
    stream = torch.cuda.current_stream()
    out = {}
    for form, P, R, n in (("one_partial", 1, 8, steps), ("eight_partials", 8, 4, max(10, steps // 4))):
        gs = wl.make_partials_gemm_inputs(P, device=device)
        Ta, K = gs[0].a.shape
        N = gs[0].b.shape[0]
        stages = [torch.zeros((P, Ta, N), dtype=torch.bfloat16, device=device) for _ in range(R)]
        if P == 1:
            calls = [ops.bind_gemm_bf16_nt(stages[i][0], gs[0].a, gs[0].b) for i in range(R)]
        else:
            calls = [ops.bind_gemm_bf16_nt_partials([stages[i][p] for p in range(P)], [g.a for g in gs],
                                                    [g.b for g in gs]) for i in range(R)]
        us = event_time(lambda i: calls[i % R](stream), n, stream, warm=10, regions=3)
        flops = 2.0 * P * Ta * N * K
        out[form] = {"us": round(us, 2), "tflops": round(flops / us / 1e6, 1),
                     "mfma_util": round(flops / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
        del calls, stages, gs
        torch.cuda.empty_cache()
    return out


def time_gemm_limits(device):
    """What the big GEMM kernel's k loop can reach by itself on this GPU: the loop of the 320 x 256 tile
    put together from its parts, every compute unit busy, operands served by the L2s, no tile prologue
    or epilogue.  TFLOP/s from HIP events around the launch; cycles and clock from the kernel's own stamps.
    Also the rate at which 1 .. 16 waves of a compute unit get the loop's 16-byte LDS reads through."""
    import numpy as np
    import torch
    L = bench_lib()
    stream = torch.cuda.current_stream()
    sp = stream.cuda_stream
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    window = 4 << 20
    src = torch.randint(0, 255, (8 * window + (128 << 10),), dtype=torch.uint8, device=device)
    stamps = torch.zeros((cus, 2), dtype=torch.int64, device=device)
    sink = torch.zeros(1024, dtype=torch.float32, device=device)
    slabs = 8192
    flops = cus * 8 * slabs * 40 * 32768.0   # 8 waves x 40 MFMAs of 32 x 32 x 16 per slab
    loop = {}
    for name, parts in (("mfma", 0), ("mfma+lds_reads", 1), ("mfma+slab_loads", 2), ("full_loop", 3),
                        ("full_loop_loads_spread", 7)):
        ms = []
        for _ in range(4):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            bench_check(L.twb_gemm_loop(slabs, parts, window, src.data_ptr(), stamps.data_ptr(), sink.data_ptr(),
                                        cus, sp))
            e1.record(stream)
            torch.cuda.synchronize()
            ms.append(e0.elapsed_time(e1))
        st = stamps.cpu().numpy().astype(np.float64)
        cyc, wall_us = float(np.median(st[:, 0])), float(np.median(st[:, 1])) / 100.0
        t = sorted(ms[1:])[1] * 1e-3
        loop[name] = {"cycles_per_slab": round(cyc / slabs), "mfma_issue_share": round(2560.0 * slabs / cyc, 3),
                      "shader_clock_ghz": round(cyc / wall_us / 1e3, 2), "tflops": round(flops / t / 1e12, 1),
                      "share_of_2.5_pflops": round(flops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 3)}
        # socket power while the same launch repeats for two seconds
        samples, t_end = [], time.perf_counter() + 2.0
        while time.perf_counter() < t_end:
            for _ in range(8):
                bench_check(L.twb_gemm_loop(slabs, parts, window, src.data_ptr(), stamps.data_ptr(),
                                            sink.data_ptr(), cus, sp))
            samples.append(board_metrics())   # taken while the queued launches run
            torch.cuda.synchronize()
        watts = [x["watts"] for x in samples[2:] if "watts" in x]
        loop[name]["socket_watts"] = round(statistics.median(watts)) if watts else None
        log(f"[gemm-limits] {name}: {loop[name]}")
    lds = {}
    iters = 2000
    cyc_out = torch.zeros(cus, dtype=torch.int64, device=device)
    usink = torch.zeros(1024, dtype=torch.int32, device=device)
    for waves in (1, 2, 4, 8, 16):
        for dma in (0, 1):
            for _ in range(2):
                bench_check(L.twb_lds_read_rate(iters, waves, dma, src.data_ptr(), cyc_out.data_ptr(), usink.data_ptr(),
                                                cus, sp))
                torch.cuda.synchronize()
            cyc = float(np.median(cyc_out.cpu().numpy()))
            lds[f"waves{waves}" + ("+slab_loads" if dma else "")] = {
                "read_bytes_per_cycle": round(waves * iters * 28 * 1024 / cyc, 1),
                "cycles_per_read_per_wave": round(cyc / (iters * 28), 1)}
    return {"definitions": "loop: the k loop of the 320 x 256 x 64 tile (8 waves, 40 MFMAs of 32 x 32 x 16 and 28 "
                           "16-byte LDS reads per wave and slab, 72 KiB per slab global -> LDS) with wait + barrier "
                           "per slab, on all compute units, operands in a 4 MiB window per XCD; mfma_issue_share "
                           "= 2560 MFMA cycles per slab / measured cycles per slab; lds: 16-byte reads with the "
                           "fragment addressing",
            "loop": loop, "lds_read_rate": lds}


def time_gemm_scaling(device, seconds=2.0):
    """How the big GEMM kernel's speed per compute unit depends on how many compute units run it.
    [320 c / 32, K] x [8192, K]^T with the grid capped at c workgroups is c tiles of 320 x 256, one per
    compute unit, a single round — the same work per compute unit for every c.  Each point runs for
    `seconds` of back-to-back launches (HIP events, median) while a thread samples `rocm-smi
    --showclocks`; sclk is the median shader clock it reported.  Per compute unit the nominal peak is
    2500 / 256 = 9.77 TFLOP/s at 2.4 GHz."""
    import re
    import subprocess
    import threading
    import torch
    from tokenweave_amd import _custom_ops as ops
    from tokenweave_amd import workloads as wl
    stream = torch.cuda.current_stream()

    def sclk_mhz():
        try:
            txt = subprocess.run(["rocm-smi", "--showclocks", "--json"], capture_output=True, text=True,
                                 timeout=10).stdout
            card = json.loads(txt)
            card = card[sorted(card)[0]]
            for k, v in card.items():
                if k.startswith("sclk clock speed"):
                    m = re.search(r"([0-9.]+)", str(v))
                    return float(m.group(1)) if m else None
        except Exception:   # no rocm-smi, no permission, other output: the clock column stays empty
            return None
        return None

    out = {"definitions": "one 320 x 256 tile per compute unit on `cus` compute units (grid cap), N = 8192; "
                          "tflops_per_cu against a nominal 9.77; sclk_mhz = median of rocm-smi samples during the run"}
    for K in (1024, 8192):
        rows = []
        for cus in (32, 64, 128, 192, 224, 256):
            M = 320 * cus // 32
            g = wl.make_gemm_inputs(M, 8192, K, device)
            outs = [torch.zeros((M, 8192), dtype=torch.bfloat16, device=device) for _ in range(4)]
            calls = [ops.bind_gemm_bf16_nt(o, g.a, g.b, cus) for o in outs]
            for i in range(20):
                calls[i % 4](stream)
            torch.cuda.synchronize()
            samples, stop = [], threading.Event()

            def sampler():
                while not stop.is_set():
                    samples.append(sclk_mhz())
                    time.sleep(0.05)
            th = threading.Thread(target=sampler)
            th.start()
            ts, t_end = [], time.perf_counter() + seconds
            while time.perf_counter() < t_end:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for i in range(200):
                    calls[i % 4](stream)
                e1.record(stream)
                torch.cuda.synchronize()
                ts.append(e0.elapsed_time(e1) * 1e3 / 200)
            stop.set()
            th.join()
            us = statistics.median(ts)
            tf = 2.0 * M * 8192 * K / us / 1e6
            clk = [c for c in samples[2:] if c]
            rows.append({"cus": cus, "M": M, "us": round(us, 2), "tflops": round(tf, 1),
                         "tflops_per_cu": round(tf / cus, 2),
                         "share_of_nominal_per_cu": round(tf / cus / (MFMA_BF16_PEAK_TFLOPS / 256), 3),
                         "sclk_mhz": round(statistics.median(clk)) if clk else None})
            log(f"[gemm-scaling] K={K}: {rows[-1]}")
            del outs, calls, g
            torch.cuda.empty_cache()
        out[f"K{K}"] = rows
    return out


def board_metrics():
    """Socket power (W), shader clock (MHz) and memory-controller activity (%) as
    `rocm-smi --showmetrics` reports them right now; {} where the tool or a field is missing."""
    import re
    import subprocess
    out = {}
    try:
        txt = subprocess.run(["rocm-smi", "--showmetrics"], capture_output=True, text=True, timeout=10).stdout
    except Exception:
        return out
    for key, name in (("current_socket_power (W):", "watts"), ("current_gfxclk (MHz):", "sclk_mhz"),
                      ("average_umc_activity (%):", "umc_pct")):
        m = re.search(re.escape(key) + r"\s*([0-9.]+)\s*$", txt, re.M)
        if m:
            out[name] = float(m.group(1))
    return out


def time_weave_power(device, seconds=2.5):
    """What the board draws while each leg of config 5's stage runs back to back for `seconds`:
    socket power, shader clock and memory-controller activity (medians of `rocm-smi
    --showmetrics` samples during the leg), the stage time (HIP events), and their product,
    the energy one stage takes.  Legs per form (one rank's GEMM / all eight partial sums):
    GEMM alone, norm alone, both on one stream, the two-stream stage at the GEMM budgets
    128 and 240 compute units; for one rank's GEMM also the big kernel forced to its 192 x 256
    and 128 x 256 tiles (164 and 124 registers per lane: a norm workgroup fits beside two of
    its waves on every SIMD) alone and beside the uncapped norm on the second stream."""
    import threading
    import torch
    from tokenweave_amd import _custom_ops as ops
    from tokenweave_amd import workloads as wl
    BL = bench_lib()
    cfg = wl.C5_NORM
    inps = [wl.make_norm_inputs(cfg, device, seed_offset=i) for i in range(8)]
    norms = [ops.bind_reduce_add_rms_norm(inp.partials, inp.partials[0], inp.residual, inp.weight, cfg.eps, None)
             for inp in inps]
    main_s, side_s = weave_streams()
    idle = board_metrics()
    out = {"definitions": "us = stage time by HIP events; watts / sclk_mhz / umc_pct = medians of rocm-smi "
                          "--showmetrics samples (current_socket_power, current_gfxclk, average_umc_activity) "
                          "while the leg runs for `seconds`; mJ = watts x us",
           "seconds": seconds, "idle": idle}

    def run_leg(fn):
        for i in range(10):
            fn(i)
        torch.cuda.synchronize()
        samples, stop = [], threading.Event()

        def sampler():
            while not stop.is_set():
                samples.append(board_metrics())
                time.sleep(0.05)
        th = threading.Thread(target=sampler)
        th.start()
        ts, t_end = [], time.perf_counter() + seconds
        while time.perf_counter() < t_end:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(main_s)
            for i in range(100):
                fn(i)
            e1.record(main_s)
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3 / 100)
        stop.set()
        th.join()
        row = {"us": round(statistics.median(ts), 2)}
        for k in ("watts", "sclk_mhz", "umc_pct"):
            v = [x[k] for x in samples[2:] if k in x]
            row[k] = round(statistics.median(v), 1) if v else None
        row["mJ"] = round(row["watts"] * row["us"] * 1e-3, 1) if row["watts"] else None
        return row

    def norm(i, stream):
        norms[i % 8](stream)

    def two_streams(gemm):
        def stage(i):
            before = torch.cuda.Event()
            before.record(main_s)
            gemm(i, main_s)
            side_s.wait_event(before)
            norm(i, side_s)
            main_s.wait_stream(side_s)
        return stage

    for form, P in (("one_partial", 1), ("eight_partials", 8)):
        gs = wl.make_partials_gemm_inputs(P, device=device)
        Ta, K = gs[0].a.shape
        N = gs[0].b.shape[0]
        R = 4
        stages = [torch.zeros((P, Ta, N), dtype=torch.bfloat16, device=device) for _ in range(R)]

        def bind(cap):
            if P == 1:
                return [ops.bind_gemm_bf16_nt(st[0], gs[0].a, gs[0].b, cap or None) for st in stages]
            return [ops.bind_gemm_bf16_nt_partials([st[p] for p in range(P)], [g.a for g in gs],
                                                   [g.b for g in gs], cap or None) for st in stages]
        gemms = {cap: bind(cap) for cap in (0, 128, 240)}
        legs = {"gemm": lambda i: gemms[0][i % R](main_s),
                "norm": lambda i: norm(i, main_s),
                "serial": lambda i: (gemms[0][i % R](main_s), norm(i, main_s))}
        for cap in (128, 240):
            legs[f"gemm/{cap}"] = (lambda c: lambda i: gemms[c][i % R](main_s))(cap)
            legs[f"weave/{cap}"] = two_streams((lambda c: lambda i, s: gemms[c][i % R](s))(cap))
        if P == 1:
            for tm in (3, 2):
                def forced(i, stream, tm=tm):
                    bench_check(BL.twb_gemm_bf16_nt_tile(stages[i % R][0].data_ptr(), gs[0].a.data_ptr(),
                                                         gs[0].b.data_ptr(), Ta, N, K, N, tm, 2,
                                                         stream.cuda_stream))
                legs[f"gemm_tile{64 * tm}x256"] = (lambda f: lambda i: f(i, main_s))(forced)
                legs[f"same_units/tile{64 * tm}x256"] = two_streams(forced)
        rows = {}
        for name, fn in legs.items():
            rows[name] = run_leg(fn)
            log(f"[weave-power] {form} {name}: {rows[name]}")
        out[form] = rows
        del gemms, stages, gs
        torch.cuda.empty_cache()
    return out


def weave_block(device, steps):
    """Both forms of config 5 for the JSON line."""
    caps = (128, 160, 176, 192, 208, 224, 240)
    return {"workload": "c5 token weave: GEMM [2458, 1024] x [8192, 1024]^T of one split || fused P=8 norm of "
                        "the 1638-row split, H=8192",
            "definitions": "serial = both kernels on one stream; overlap = GEMM capped to gemm_cus compute "
                           "units on the current stream, norm on a second stream; speedup = serial/overlap; "
                           "overlap_eff = (serial - overlap)/min(gemm, norm), null unless serial >= max(gemm, "
                           "norm) and |serial - (gemm + norm)| <= 5 %; every leg is the median of "
                           "`regions` interleaved regions of `stages_per_region` stages; MFMA utilisation "
                           "against 2.5 PFLOP/s dense bf16",
            "eight_partials": time_weave(device, "eight_partials", caps, steps=steps),
            "one_partial": time_weave(device, "one_partial", caps, steps=steps)}


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
    if args.ceilings:
        print(json.dumps({"ceilings": time_ceilings(device)}), flush=True)
        return
    if args.host_cost:
        print(json.dumps({"host_us_per_call": host_cost(device)}), flush=True)
        return
    if args.tlb_latency:
        print(json.dumps({"tlb_latency": time_tlb_latency(device)}), flush=True)
        return
    if args.graph_replay:
        print(json.dumps({"graph_replay": time_graph_replay(cfg, args.max_ctas, device)}), flush=True)
        return
    if args.timeline:
        print(json.dumps({"timeline": time_timeline(cfg, device), "arrivals": time_arrivals(cfg, device)}),
              flush=True)
        return
    if args.gemm_only:
        print(json.dumps({"c5_gemm": time_gemm_only(device, min(args.steps, 200))}), flush=True)
        return
    if args.gemm_limits:
        print(json.dumps({"gemm_limits": time_gemm_limits(device)}), flush=True)
        return
    if args.gemm_scaling:
        print(json.dumps({"gemm_scaling": time_gemm_scaling(device)}), flush=True)
        return
    if args.weave_only:
        print(json.dumps({"weave": weave_block(device, 20)}), flush=True)
        return
    if args.weave_power:
        print(json.dumps({"weave_power": time_weave_power(device)}), flush=True)
        return
    log(f"[bench] {torch.cuda.get_device_name(0)}; workload {cfg.name}: P={cfg.P} T={cfg.T} "
        f"H={cfg.H} bytes/call={cfg.bytes}")

    res = time_norm(cfg, args.steps, args.warmup, args.max_ctas, device, pretouch=args.pretouch,
                    graph=not args.pretouch)
    log(f"[bench] {res}")
    kernel_us = res["event_us_per_launch"]
    traffic = MEASURED_TRAFFIC_BYTES.get(cfg.name, (None, None)) if args.max_ctas == 0 else (None, None)
    achieved = cfg.bytes / kernel_us / 1e3
    out = {
        "metric": "fused P-partial reduce+add+RMSNorm GB/s (% HBM peak), us/call, H=8192",
        "value": round(res["gbps"], 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(res["ms_per_step"], 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": cfg.name, "P": cfg.P, "T": cfg.T, "H": cfg.H, "eps": cfg.eps,
                   "bytes_per_call": cfg.bytes, "rotating_input_sets": res["nsets"],
                   "max_ctas": args.max_ctas, "timed_regions": res["regions"],
                   "region_reported": "median", "preroll_steps": res["preroll_steps"]},
        "pct_hbm_peak": round(100.0 * res["gbps"] / HBM_PEAK_GBPS, 2),
        "us_per_call": round(res["ms_per_step"] * 1e3, 3),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic[0], "traffic_source": traffic[1],
                     "kernel": KERNEL_NAMES.get(cfg.name),
                     "duration_source": "HIP-event bracket around each region's `steps` launches on the "
                                        "launch stream, after `lead_in_steps` untimed launches (launch gaps "
                                        "included), median region",
                     "lead_in_steps": res["lead_in_steps"],
                     "event_us_per_launch": round(kernel_us, 3),
                     "graph_replay_us_per_launch": (round(res["graph_replay_us_per_launch"], 3)
                                                    if "graph_replay_us_per_launch" in res else None),
                     "event_us_per_launch_min_max": [round(res["event_us_per_launch_min"], 3),
                                                     round(res["event_us_per_launch_max"], 3)]},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, args.cpu_seconds)
        log(f"[bench] cpu_baseline {out['cpu_baseline']}")
    if not args.no_weave:
        out["weave"] = weave_block(device, 20)
        log(f"[bench] weave {out['weave']}")
    if args.calibration_copy:
        calibration_copies(device)
    if args.sweep:
        sweep = {}
        cfgs = dict(cfgs)
        cfgs["c2_unsharded@T2048"] = wl.C2.with_tokens(2048, "c2_unsharded@T2048")
        for name, c in cfgs.items():
            steps = max(50, min(2000, int(0.02 * 5e12 / c.bytes)))  # ~20 ms of kernel time
            r = time_norm(c, steps, max(5, steps // 10), args.max_ctas, device, regions=5, preroll_ms=10.0)
            warm_us = time_norm_warm(c, steps, args.max_ctas, device) if c.bytes < (200 << 20) else None
            one_wg = None
            if c.P > 1 and c.T <= 48:   # decode sizes: the same call without the split-row kernel
                one_wg = time_norm(c, steps, max(5, steps // 10), args.max_ctas, device, regions=5, preroll_ms=10.0,
                                   split=False)["event_us_per_launch"]
            sweep[name] = {"P": c.P, "T": c.T, "H": c.H, "bytes": c.bytes,
                           "kernel_us_one_workgroup_per_row": None if one_wg is None else round(one_wg, 3),
                           "us_per_call": round(r["ms_per_step"] * 1e3, 3),
                           "kernel_us": round(r["event_us_per_launch"], 3),
                           "kernel_us_cache_resident": None if warm_us is None else round(warm_us, 3),
                           "gbps": round(c.bytes / r["event_us_per_launch"] / 1e3, 1),
                           "pct_hbm_peak": round(c.bytes / r["event_us_per_launch"] / 1e3 / HBM_PEAK_GBPS * 100, 2)}
            log(f"[sweep] {name}: {sweep[name]}")
        # Grid-cap sweep of the headline shape (the reference's CTA sweep,
        # artifact/csvs/figure_10.csv: 2 ... 128 CTAs at 256 rows per GPU).
        c = cfgs["c2_llama70b_tp8_shard@T256"]
        cta = {}
        for cap in (2, 4, 8, 16, 32, 64, 128, 0):
            r = time_norm(c, 200, 20, cap, device, regions=5, preroll_ms=10.0)
            cta[str(cap or c.T)] = round(r["event_us_per_launch"], 2)
        sweep["c2_T256_us_by_max_ctas"] = cta
        log(f"[sweep] c2_T256_us_by_max_ctas: {cta}")
        # The reference's own microbenchmark grid for the P = 1 op (fused_add_rms_norm_cta,
        # H = 8192; artifact/csvs/figure_4.csv, one H100): context, not a baseline for the
        # headline metric, whose P = 8 form the reference does not publish.
        for rows, h100_us in ((64, 8.61), (256, 12.16), (1024, 29.92), (2048, 51.84), (4096, 96.51),
                              (32768, 712.4)):
            c = wl.C1.with_tokens(rows, f"p1_add_rms_norm@T{rows}")
            steps = max(50, min(2000, int(0.02 * 5e12 / c.bytes)))
            r = time_norm(c, steps, max(5, steps // 10), args.max_ctas, device, regions=5, preroll_ms=10.0)
            sweep[c.name] = {"P": 1, "T": rows, "H": c.H, "bytes": c.bytes,
                             "kernel_us": round(r["event_us_per_launch"], 3),
                             "gbps": round(c.bytes / r["event_us_per_launch"] / 1e3, 1),
                             "pct_hbm_peak": round(c.bytes / r["event_us_per_launch"] / 1e3 / HBM_PEAK_GBPS * 100, 2),
                             "reference_h100_us": h100_us}
            log(f"[sweep] {c.name}: {sweep[c.name]}")
        for name in ("c2_llama70b_tp8_shard@T256", "c2_unsharded@T2048"):
            c = cfgs[name]
            steps = max(50, min(2000, int(0.02 * 5e12 / c.bytes)))
            for epi in ("fp8_static", "fp8_dynamic", "int8_dynamic"):
                r = time_norm(c, steps, max(5, steps // 10), args.max_ctas, device, epi, regions=5, preroll_ms=10.0)
                b = quant_bytes(c, epi)
                sweep[f"{name}+{epi}"] = {"bytes": b, "kernel_us": round(r["event_us_per_launch"], 3),
                                          "gbps": round(b / r["event_us_per_launch"] / 1e3, 1),
                                          "pct_hbm_peak": round(b / r["event_us_per_launch"] / 1e3 / HBM_PEAK_GBPS * 100, 2)}
                log(f"[sweep] {name}+{epi}: {sweep[f'{name}+{epi}']}")
        out["sweep"] = sweep
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
