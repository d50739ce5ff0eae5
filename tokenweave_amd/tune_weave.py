"""Measures, on the GPU it runs on, the weave budgets for one model shape and
writes a table in the layout `load_config` reads.

    python -m tokenweave_amd.tune_weave --hidden 8192 --k 1024 --k-mlp 3584 --world-size 8 \\
        --out tokenweave_amd/tokenweave_configs/llama_config_8.json

The shipped tables (`tokenweave_configs/`, the reference's five: vllm/tokenweave_configs/*.json):
llama_config_8 (hidden 8192, K 1024 / 3584), llama_config_4 (2048 / 7168), qwen2_config_8 (1024 / 3696),
qwen2_config_4 (2048 / 7392), mixtral_config_8 (hidden 6144, K 768 / 2048).

For every token count N and split offset (the reference's five, artifact/figure_9/bench.py:107)
it times the two stages the reference overlaps per block (tokenweave_utils.py:236-260): the
row-parallel GEMM [split, K] x [hidden, K]^T of the first token split on the current stream
while the fused P-partial norm of the second split runs on a second stream, and the same
with the splits exchanged — over a grid of GEMM compute-unit budgets and norm grid caps —
and the same kernels on one stream.  All legs of one (N, offset, block) are timed
interleaved, region by region, and compared by their medians, so that every leg sees the
same mix of power states.  One offset is chosen per token count: the one whose attention
and MLP stages together take the least time; the budgets and the "overlap" flag (1 when the
weave is at least 2 % faster than one stream at that offset) are the ones measured there.
The role of artifact/configs_generator/generator.py in the reference, which picks the
minimum-latency row of its benchmark sweep.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import statistics
import sys
from typing import Callable, Dict, List, Sequence

import torch

from . import _custom_ops as ops
from . import _lib
from . import workloads as wl
from .tokenweave_utils import tokenweave_split_size

REFERENCE_SPLIT_OFFSETS = (0, 64, 128, 192, 256)   # artifact/figure_9/bench.py:107

_STREAMS = None


def weave_streams():
    """The two streams of every timed stage, created once: HIP spreads streams over a few
    hardware queues in creation order, and two streams that share a queue run their
    kernels one after the other."""
    global _STREAMS
    if _STREAMS is None:
        _STREAMS = (torch.cuda.Stream(), torch.cuda.Stream())
    return _STREAMS


def interleaved_medians(legs: Dict[str, Callable[[int], None]], stream: torch.cuda.Stream, steps: int,
                        regions: int = 11, lead_in: int = 2,
                        after_region: Callable[[str], None] = None) -> Dict[str, Dict[str, float]]:
    """Times every leg (`fn(i)` enqueues one stage; its work must be ordered after and
    before `stream`) in `regions` rounds: in each round every leg in turn runs `lead_in`
    untimed stages and then `steps` stages bracketed by HIP events on `stream`.  Because
    the legs alternate every few milliseconds, clock and power state are shared by all of
    them instead of belonging to whichever ran last.  `after_region(name)` is called after a
    leg's timed stages have been enqueued (before the synchronisation), e.g. to enqueue a
    clock probe.  Returns per leg: median, min and max microseconds per stage over the
    rounds."""
    samples: Dict[str, List[float]] = {name: [] for name in legs}
    it = 0
    with torch.cuda.stream(stream):
        for name, fn in legs.items():      # one untimed pass: first-launch costs
            fn(it)
            it += 1
        torch.cuda.synchronize()
        for _ in range(regions):
            for name, fn in legs.items():
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                for _ in range(lead_in):
                    fn(it)
                    it += 1
                e0.record(stream)
                for _ in range(steps):
                    fn(it)
                    it += 1
                e1.record(stream)
                if after_region is not None:
                    after_region(name)
                torch.cuda.synchronize()
                samples[name].append(e0.elapsed_time(e1) * 1e3 / steps)
    return {name: {"us": statistics.median(v), "min": min(v), "max": max(v)} for name, v in samples.items()}


class _Stage:
    """One GEMM [rows_gemm, K] x [hidden, K]^T and one fused norm of rows_norm rows, with the
    C-ABI calls for: both on one stream, and the weave (GEMM capped on the main stream, norm
    on the side stream behind an event, the main stream waiting for it afterwards)."""

    def __init__(self, L, rows_gemm, rows_norm, hidden, k, world_size, device):
        self.L = L
        self.g = wl.make_gemm_inputs(rows_gemm, hidden, k, device)
        self.out = torch.empty((rows_gemm, hidden), dtype=torch.bfloat16, device=device)
        cfg = wl.NormConfig("tune", P=world_size, T=rows_norm, H=hidden, eps=1e-5, seed=77,
                            partial_std=world_size ** -0.5)
        nsets = max(2, min(8, (1 << 31) // cfg.bytes))
        self.keep, self.sets = [], []
        for i in range(nsets):
            inp = wl.make_norm_inputs(cfg, device, seed_offset=i)
            ops.reduce_add_rms_norm(inp.partials, inp.partials[0], inp.residual, inp.weight, cfg.eps)
            ptrs = (ctypes.c_void_p * cfg.P)(*[p.data_ptr() for p in inp.partials])
            self.keep.append((inp, ptrs))
            self.sets.append((ptrs, cfg.P, inp.partials[0].data_ptr(), inp.residual.data_ptr(),
                              inp.weight.data_ptr(), cfg.T, cfg.H, cfg.eps))
        ops.gemm_bf16_nt(self.out, self.g.a, self.g.b)
        self.gargs = (self.out.data_ptr(), self.g.a.data_ptr(), self.g.b.data_ptr(), rows_gemm, hidden, k)
        self.main_s, self.side_s = weave_streams()
        self.pm = ctypes.c_void_p(self.main_s.cuda_stream)
        self.ps = ctypes.c_void_p(self.side_s.cuda_stream)

    def _check(self, rc):
        if rc:
            raise RuntimeError(_lib.last_error())

    def serial(self, i):
        out, a, b, M, N, K = self.gargs
        rc = self.L.tw_gemm_bf16_nt(out, a, b, M, N, K, N, 0, self.pm)
        ptrs, P, y, r, w, T, H, eps = self.sets[i % len(self.sets)]
        rc |= self.L.tw_reduce_add_rms_norm(ptrs, P, y, r, w, T, H, 0, eps, self.pm)
        self._check(rc)

    def weave(self, gemm_cus, norm_ctas):
        out, a, b, M, N, K = self.gargs

        def stage(i):
            before = torch.cuda.Event()
            before.record(self.main_s)
            rc = self.L.tw_gemm_bf16_nt(out, a, b, M, N, K, N, gemm_cus, self.pm)   # GEMM first: it takes its budget
            self.side_s.wait_event(before)
            ptrs, P, y, r, w, T, H, eps = self.sets[i % len(self.sets)]
            rc |= self.L.tw_reduce_add_rms_norm(ptrs, P, y, r, w, T, H, norm_ctas, eps, self.ps)
            self.main_s.wait_stream(self.side_s)
            self._check(rc)
        return stage


def tune(hidden, k, world_size, tokens, offsets: Sequence[int] = REFERENCE_SPLIT_OFFSETS, device="cuda:0",
         log=print, k_mlp=None, regions=7, stage_budget_us=3000.0):
    """One table.  Per token count and split offset two blocks are timed: the attention
    block's row-parallel GEMM (inner dimension `k`, the rank's slice of the attention
    output) beside the norm -> `attention_ctas`, `gemm_cus`; and the MLP's (`k_mlp`, the
    rank's slice of the intermediate size) -> `mlp_ctas`, `mlp_gemm_cus`.  Without `k_mlp`
    the MLP entries repeat the attention ones.  Each block is two stages (the GEMM of one
    split beside the norm of the other, both ways round); budgets are compared by the sum
    of the two stages' median times.  `regions` rounds per leg, each of as many stages as
    fit `stage_budget_us` (3 .. 20)."""
    L = _lib.lib()
    cus = ops.num_compute_units(device)
    gemm_grid = sorted({0} | {int(cus * f) // 8 * 8 for f in (0.5, 0.625, 0.75, 0.875)})
    norm_grid = (0, cus // 2)
    kinds = [("attention", k)] + ([("mlp", k_mlp)] if k_mlp is not None else [])
    table = {}
    for n in tokens:
        by_offset = {}
        for off in offsets:
            split = min(tokenweave_split_size(n, off), n)
            rest = n - split
            if split == 0 or rest == 0:
                continue
            found = {}
            for kind, kk in kinds:
                stages = [_Stage(L, split, rest, hidden, kk, world_size, device),
                          _Stage(L, rest, split, hidden, kk, world_size, device)]
                legs = {}
                for s, st in enumerate(stages):
                    legs[f"serial{s}"] = st.serial
                    for gc in gemm_grid:
                        for nc in norm_grid:
                            legs[f"weave{s}/{gc}/{nc}"] = st.weave(gc, nc)
                main_s = stages[0].main_s
                with torch.cuda.stream(main_s):   # size the regions by one serial stage
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    stages[0].serial(0)
                    e0.record(main_s)
                    stages[0].serial(1)
                    e1.record(main_s)
                    torch.cuda.synchronize()
                steps = max(3, min(20, int(stage_budget_us / max(1.0, e0.elapsed_time(e1) * 1e3))))
                res = interleaved_medians(legs, main_s, steps, regions=regions)
                serial = res["serial0"]["us"] + res["serial1"]["us"]
                best = None
                for gc in gemm_grid:
                    for nc in norm_grid:
                        us = res[f"weave0/{gc}/{nc}"]["us"] + res[f"weave1/{gc}/{nc}"]["us"]
                        if best is None or us < best[0]:
                            best = (us, gc, nc)
                found[kind] = {"us": best[0], "gemm_cus": best[1], "ctas": best[2], "serial": serial}
                log(f"tokens={n} offset={off} {kind} (K={kk}, {split}+{rest} rows): both stages {best[0]:.1f} us "
                    f"with gemm_cus={best[1]} norm_ctas={best[2]} (one stream: {serial:.1f} us, "
                    f"speedup {serial / best[0]:.3f}; {steps} stages x {regions} regions per leg)")
                del stages, legs
                torch.cuda.empty_cache()
            by_offset[off] = found
        if not by_offset:
            continue
        # one offset per token count: attention and MLP stages together, absolute time (every
        # offset does the same total work)
        def total(f, key):
            return sum(f[kind][key] for kind in f)
        off = min(by_offset, key=lambda o: total(by_offset[o], "us"))
        f = by_offset[off]
        a = f["attention"]
        m = f.get("mlp", a)
        stage_us, serial_us = total(f, "us"), total(f, "serial")
        table[str(n)] = {"attention_ctas": a["ctas"], "mlp_ctas": m["ctas"], "split_offset": off,
                         "gemm_cus": a["gemm_cus"], "mlp_gemm_cus": m["gemm_cus"],
                         "overlap": int(stage_us < 0.98 * serial_us)}
        log(f"tokens={n}: split_offset={off}, weave {stage_us:.1f} us vs one stream {serial_us:.1f} us "
            f"(speedup {serial_us / stage_us:.3f}) -> {table[str(n)]}")
    return table


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--hidden", type=int, default=8192)
    ap.add_argument("--k", type=int, default=1024,
                    help="inner dimension of the attention block's row-parallel GEMM (per rank)")
    ap.add_argument("--k-mlp", type=int, default=None,
                    help="inner dimension of the MLP's row-parallel GEMM (per rank); default: not tuned apart")
    ap.add_argument("--world-size", type=int, default=8)
    ap.add_argument("--tokens", type=int, nargs="+", default=[1024, 2048, 4096, 8192, 16384, 32768, 65536])
    ap.add_argument("--offsets", type=int, nargs="+", default=list(REFERENCE_SPLIT_OFFSETS))
    ap.add_argument("--regions", type=int, default=7)
    ap.add_argument("--out", required=True)
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        sys.exit("tune_weave needs the GPU it tunes for")
    table = tune(args.hidden, args.k, args.world_size, args.tokens, args.offsets,
                 log=lambda m: print(m, file=sys.stderr, flush=True), k_mlp=args.k_mlp, regions=args.regions)
    with open(args.out, "w") as f:
        json.dump(table, f, indent=2)
        f.write("\n")
    print(args.out)


if __name__ == "__main__":
    main()
