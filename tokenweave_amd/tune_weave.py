"""Measures, on the GPU it runs on, the weave budgets for one model shape and
writes a table in the layout `load_config` reads.

    python -m tokenweave_amd.tune_weave --hidden 8192 --k 1024 --k-mlp 3584 --world-size 8 \\
        --out tokenweave_amd/tokenweave_configs/llama_config_8.json

The shipped tables (`tokenweave_configs/`, the reference's five: vllm/tokenweave_configs/*.json):
llama_config_8 (hidden 8192, K 1024 / 3584), llama_config_4 (2048 / 7168), qwen2_config_8 (1024 / 3696),
qwen2_config_4 (2048 / 7392), mixtral_config_8 (hidden 6144, K 768 / 2048).

For every token count N and split offset it times the stage the reference overlaps
(tokenweave_utils.py:236-260): the row-parallel GEMM [split, K] x [hidden, K]^T of one
token split on the current stream while the fused P-partial norm of the other split
runs on a second stream, over a grid of GEMM compute-unit budgets and norm grid caps,
and keeps the fastest; the same two kernels are also timed on one stream, and an entry
whose best weave is not at least 2 % faster gets "overlap": 0 (no weave at that size).  The role of artifact/configs_generator/generator.py in the
reference, which picks the minimum-latency row of its benchmark sweep.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import sys

import torch

from . import _custom_ops as ops
from . import _lib
from . import workloads as wl
from .tokenweave_utils import tokenweave_split_size


_STREAMS = None


def _streams():
    """The two streams of every timed stage, created once: HIP spreads streams over a few
    hardware queues in creation order, and two streams that share a queue run their
    kernels one after the other."""
    global _STREAMS
    if _STREAMS is None:
        _STREAMS = (torch.cuda.Stream(), torch.cuda.Stream())
    return _STREAMS


def time_stage(L, gemm_args, norm_sets, gemm_cus, norm_ctas, steps=40):
    main_s, side_s = _streams()
    pm, ps = ctypes.c_void_p(main_s.cuda_stream), ctypes.c_void_p(side_s.cuda_stream)
    out, a, b, M, N, K = gemm_args

    def stage(i):
        before = torch.cuda.Event()
        before.record(main_s)
        rc = L.tw_gemm_bf16_nt(out, a, b, M, N, K, N, gemm_cus, pm)
        side_s.wait_event(before)
        ptrs, P, y, r, w, T, H, eps = norm_sets[i % len(norm_sets)]
        rc |= L.tw_reduce_add_rms_norm(ptrs, P, y, r, w, T, H, norm_ctas, eps, ps)
        main_s.wait_stream(side_s)
        if rc:
            raise RuntimeError(_lib.last_error())

    with torch.cuda.stream(main_s):
        for i in range(5):
            stage(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(main_s)
        for i in range(steps):
            stage(i)
        e1.record(main_s)
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / steps


def time_serial(L, gemm_args, norm_sets, steps=40):
    """The same two kernels one after the other on one stream, both uncapped."""
    s = _streams()[0]
    sp = ctypes.c_void_p(s.cuda_stream)
    out, a, b, M, N, K = gemm_args

    def stage(i):
        rc = L.tw_gemm_bf16_nt(out, a, b, M, N, K, N, 0, sp)
        ptrs, P, y, r, w, T, H, eps = norm_sets[i % len(norm_sets)]
        rc |= L.tw_reduce_add_rms_norm(ptrs, P, y, r, w, T, H, 0, eps, sp)
        if rc:
            raise RuntimeError(_lib.last_error())

    with torch.cuda.stream(s):
        for i in range(5):
            stage(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(s)
        for i in range(steps):
            stage(i)
        e1.record(s)
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / steps


def tune(hidden, k, world_size, tokens, offsets, device="cuda:0", log=print, k_mlp=None):
    """One table.  Two kinds of stage are timed per token count: the norm beside the
    attention block's row-parallel GEMM (inner dimension `k`, the rank's slice of the
    attention output) -> `attention_ctas`, `gemm_cus`; and beside the MLP's (`k_mlp`, the
    rank's slice of the intermediate size) -> `mlp_ctas`, `mlp_gemm_cus`.  Without `k_mlp`
    the MLP entries repeat the attention ones."""
    L = _lib.lib()
    cus = ops.num_compute_units(device)
    gemm_grid = sorted({0} | {int(cus * f) // 8 * 8 for f in (0.5, 0.625, 0.75, 0.875)})
    norm_grid = (0, cus // 2)
    table = {}
    for n in tokens:
        best = {}
        for kind, kk in (("attention", k), ("mlp", k_mlp)):
            if kk is None:
                continue
            for off in offsets:
                split = min(tokenweave_split_size(n, off), n)
                rest = n - split
                if split == 0 or rest == 0:
                    continue
                g = wl.make_gemm_inputs(split, hidden, kk, device)
                out = torch.empty((split, hidden), dtype=torch.bfloat16, device=device)
                cfg = wl.NormConfig("tune", P=world_size, T=rest, H=hidden, eps=1e-5, seed=77,
                                    partial_std=world_size ** -0.5)
                nsets = max(2, min(8, (1 << 31) // cfg.bytes))
                keep, sets = [], []
                for i in range(nsets):
                    inp = wl.make_norm_inputs(cfg, device, seed_offset=i)
                    ops.reduce_add_rms_norm(inp.partials, inp.partials[0], inp.residual, inp.weight, cfg.eps)
                    ptrs = (ctypes.c_void_p * cfg.P)(*[p.data_ptr() for p in inp.partials])
                    keep.append((inp, ptrs))
                    sets.append((ptrs, cfg.P, inp.partials[0].data_ptr(), inp.residual.data_ptr(),
                                 inp.weight.data_ptr(), cfg.T, cfg.H, cfg.eps))
                ops.gemm_bf16_nt(out, g.a, g.b)
                gargs = (out.data_ptr(), g.a.data_ptr(), g.b.data_ptr(), split, hidden, kk)
                serial = time_serial(L, gargs, sets)
                for gc in gemm_grid:
                    for nc in norm_grid:
                        us = time_stage(L, gargs, sets, gc, nc)
                        # a table has one split offset: compare offsets by the stage's gain over
                        # its own serial time
                        if kind not in best or us / serial < best[kind][0] / best[kind][4]:
                            best[kind] = (us, off, gc, nc, serial)
                del keep, sets, g, out
                torch.cuda.empty_cache()
            us, off, gc, nc, serial = best[kind]
            log(f"tokens={n} {kind} (K={kk}): best stage {us:.1f} us with split_offset={off} gemm_cus={gc} "
                f"norm_ctas={nc} (one stream: {serial:.1f} us, speedup {serial / us:.2f})")
        a = best["attention"]
        m = best.get("mlp", a)
        stage_us, serial_us = a[0] + m[0], a[4] + m[4]
        table[str(n)] = {"attention_ctas": a[3], "mlp_ctas": m[3], "split_offset": a[1], "gemm_cus": a[2],
                         "mlp_gemm_cus": m[2], "overlap": int(stage_us < 0.98 * serial_us)}
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
    ap.add_argument("--offsets", type=int, nargs="+", default=[0, 256])
    ap.add_argument("--out", required=True)
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        sys.exit("tune_weave needs the GPU it tunes for")
    table = tune(args.hidden, args.k, args.world_size, args.tokens, args.offsets,
                 log=lambda m: print(m, file=sys.stderr, flush=True), k_mlp=args.k_mlp)
    with open(args.out, "w") as f:
        json.dump(table, f, indent=2)
        f.write("\n")
    print(args.out)


if __name__ == "__main__":
    main()
