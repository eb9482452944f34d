#!/usr/bin/env python3
"""Benchmark of the cross-submesh reshard on one MI355X.

A step is one reshard (one pass of the hot path over one batch of synthetic
input).  The default workload is configuration 2 of BASELINE.json, the one the
metric is quoted on: a bf16 [8, 4096, 8192] activation resharded from
hidden-sharded 8 ways (devices 0-7) to sequence-sharded 4 ways (devices 8-11),
all twelve shard buffers resident in this GPU's HBM before the timed region
starts.  Prints one JSON line.

No torch in this process: PyTorch's wheel bundles its own HIP runtime and two
HIP runtimes cannot both drive the GPU.  The library owns its stream and its
device memory, and raises if no GPU is present (there is no CPU fallback).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak


def cpu_baseline(arrays, gs, seconds=12.0):
    """The C restatement of the reference reshard (oracle/reshard_cpu.c) timed on
    this box's host cores over the same workload; a reported baseline only."""
    import numpy as np
    from oracle import reshard_cpu, reshard_oracle as ro
    from helpers import oracle_shape, raw_global
    from multimesh_jax_amd import workloads

    threads = min(len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", "16") or 16), 64)
    a, g = arrays[0], gs[0]
    so, do = oracle_shape(a["type"], a["src"]), oracle_shape(a["type"], a["dst"])
    shards = ro.make_shards(raw_global(a, g), so, a["src"].get("minor_to_major"))
    n = int(np.prod(ro.shard_shape(do)))
    out = {d: np.empty(n, dtype=ro.raw_dtype(a["type"])) for d in range(do.dev_start, do.dev_start + do.dev_count)}
    alg = workloads.algorithmic_bytes(arrays)

    def timed(nthreads, budget):
        reshard_cpu.reshard(shards, so, do, out, nthreads=nthreads)  # warm-up, page in
        reps, t0 = 0, time.perf_counter()
        while True:
            reshard_cpu.reshard(shards, so, do, out, nthreads=nthreads)
            reps += 1
            dt = time.perf_counter() - t0
            if dt >= budget:
                return alg * reps / dt / 1e9, reps, dt

    one, reps1, dt1 = timed(1, seconds * 0.3)
    many, reps, dt = timed(threads, seconds * 0.7)
    return {"value": round(many, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "single_thread_value": round(one, 2),
            "sample": "configuration 2 at full size: %d repetitions in %.1f s on %d pthreads (and %d repetitions in "
                      "%.1f s on 1 thread); C restatement of the reference reshard, one memcpy per contiguous run"
                      % (reps, dt, threads, reps1, dt1)}, out


def measure(ctx, mm, workloads, args, config, with_parity=True):
    """Creates the stores of one configuration, checks the result against the
    oracle, times `args.steps` reshards.  Returns (result dict, arrays, gs, first destination stores)."""
    from gpu_helpers import make_stores, read_all
    from helpers import oracle_outputs

    arrays = workloads.config(config, args.scale)
    if args.name:
        arrays = [a for a in arrays if args.name in a["name"]]
    gs = [workloads.generate(a) for a in arrays]
    alg_bytes = workloads.algorithmic_bytes(arrays)
    # Buffer sets rotated between steps: at least `--sets`, and enough of them that 768 MiB of other buffers are
    # touched before a set comes round again - the 256 MB Infinity Cache must not serve a small configuration's reads
    # (an explicit --sets 1 or 2 is a probing run and is taken as given).
    n_sets = max(1, args.sets)
    if args.sets >= 3:
        n_sets = max(n_sets, -(-(768 << 20) // max(alg_bytes, 1)) + 1)
    sets = [make_stores(ctx, arrays, gs, poison=None) for _ in range(n_sets)]

    def step(i):
        srcs, dsts = sets[i % len(sets)]
        if len(srcs) == 1:
            ctx.Reshard(srcs[0], dsts[0])
        elif args.unbatched:  # one call and one launch per array, as the reference's schedule loop issues them
            for s_, d_ in zip(srcs, dsts):
                ctx.Reshard(s_, d_)
        else:
            ctx.ReshardBatch(srcs, dsts)

    before = ctx.stats
    step(0)
    ctx.Sync()
    launches = ctx.stats["kernel_launches"] - before["kernel_launches"]
    if with_parity and alg_bytes <= (2 << 30):  # parity before timing: bit for bit against the oracle
        for a, g, d in zip(arrays, gs, sets[0][1]):
            expect = oracle_outputs(a, g)
            got = read_all(ctx, d)
            for dev in expect:
                if got[dev].tobytes() != expect[dev].tobytes():
                    sys.exit("bench.py: GPU result differs from the oracle (array %s, device %d)" % (a["name"], dev))

    for i in range(args.warmup):
        step(i)
    ctx.Sync()
    # timed region: exactly K steps, wall clock bracketed by synchronisation;
    # HIP events on the library's own stream give the kernel time inside it
    t0 = time.perf_counter()
    ctx.StartTimer()
    for i in range(args.steps):
        step(i)
    kernel_ms = ctx.StopTimer()
    ctx.Sync()
    wall_s = time.perf_counter() - t0

    batched = len(arrays) > 1 and not getattr(args, "unbatched", False)
    plan = (ctx.plan_stats(sets[0][0][0], sets[0][1][0]) if len(arrays) == 1 else
            ctx.batch_plan_stats(sets[0][0], sets[0][1]) if batched else None)
    # cold plan construction (host only, excluded from the steady-state figure: plans are cached per descriptor pair)
    from helpers import lib_shape
    src_shapes = [lib_shape(a["type"], a["src"]) for a in arrays]
    dst_shapes = [lib_shape(a["type"], a["dst"]) for a in arrays]
    tp = time.perf_counter()
    cold = mm.Plan(src_shapes, dst_shapes, args.chunk_bytes, args.order, args.xcd_mode)
    plan_build_ms = (time.perf_counter() - tp) * 1e3
    table_bytes = cold.stats["table_bytes"]
    del cold
    generic = plan is not None and plan["n_copy_generic_chunks"] > plan["n_copy16_chunks"]
    res = {
        "alg_bytes": alg_bytes,
        "ms_per_step": wall_s * 1e3 / args.steps,
        "value": alg_bytes / (wall_s / args.steps) / 1e9,
        "kernel_ms": kernel_ms / args.steps,
        "achieved": alg_bytes / (kernel_ms / args.steps * 1e-3) / 1e9,
        "launches": launches,
        "plan": plan,
        "plan_build_ms": plan_build_ms,
        "plan_table_bytes": table_bytes,
        "kernel": ("mmr_transpose_kernel" if plan is not None and plan["n_transpose_chunks"] > 0 else
                   "mmr_copy_generic_kernel" if generic or config in (5, 6) else "mmr_copy16_kernel"),
        "n_arrays": len(arrays),
        "sets": len(sets),
    }
    first_dsts = sets[0][1]
    for srcs, dsts in sets[1:]:
        for s in srcs + dsts:
            ctx.Free(s)
    return res, arrays, gs, first_dsts, sets[0][0]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2, help="BASELINE.json configuration (1-5); 2 is the headline")
    ap.add_argument("--sets", type=int, default=3, help="independent buffer sets rotated between steps")
    ap.add_argument("--all", action="store_true", help="also measure configurations 1, 3, 4 and 5 (adds minutes)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--unbatched", action="store_true",
                    help="multi-array configurations: one Reshard call per array instead of one batched call (probing)")
    # plan options (0 = library default) and probing switches
    ap.add_argument("--chunk-bytes", type=int, default=0)
    ap.add_argument("--order", type=int, default=0)
    ap.add_argument("--xcd-mode", type=int, default=0)
    ap.add_argument("--flags", type=int, default=0)
    ap.add_argument("--name", type=str, default="", help="only the arrays whose name contains this")
    ap.add_argument("--scale", type=int, default=1, help="divide the large extents (probing only)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every logical device of both submeshes is a buffer in one "
                 "MI355X's HBM and nothing here uses a second GPU (got --gpus %d)" % args.gpus)

    import multimesh_jax_amd as mm
    from multimesh_jax_amd import workloads
    from gpu_helpers import read_all

    ctx = mm.ReshardContext(0)
    if args.chunk_bytes or args.order or args.xcd_mode or args.flags:
        ctx.set_plan_options(args.chunk_bytes, args.order, args.xcd_mode, args.flags)

    res, arrays, gs, first_dsts, first_srcs = measure(ctx, mm, workloads, args, args.config)

    traffic = None
    tpath = os.path.join(ROOT, "profiles", "traffic_config%d.json" % args.config)
    if os.path.exists(tpath) and args.scale == 1 and not args.name:
        with open(tpath) as f:
            traffic = json.load(f).get("hbm_bytes_per_launch")

    result = {
        "metric": "reshard GB/s ((read+write bytes)/time) & % HBM peak, bf16 [8,4096,8192]",
        "value": round(res["value"], 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(res["ms_per_step"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",  # pure byte movement (bf16 payload never interpreted), 16-byte vector accesses
        "data": "synthetic",
        "config": {
            "workload": "configuration %d of BASELINE.json: %s" % (
                args.config, "; ".join("%s %s %s" % (a["name"], a["type"], list(a["shape"])) for a in arrays[:3])
                + (" ... (%d arrays)" % len(arrays) if len(arrays) > 3 else "")),
            "source": arrays[0]["src"], "destination": arrays[0]["dst"],
            "algorithmic_bytes": res["alg_bytes"], "buffer_sets": res["sets"],
            "plan": res["plan"], "plan_build_ms_cold": round(res["plan_build_ms"], 3),
            "plan_table_bytes": res["plan_table_bytes"], "pct_hbm_peak": round(100.0 * res["value"] / HBM_PEAK_GBS, 2),
        },
        "roofline": {
            "bound": "hbm", "achieved": round(res["achieved"], 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(res["achieved"] / HBM_PEAK_GBS, 4), "traffic": traffic,
            "kernel": res["kernel"], "kernel_ms": round(res["kernel_ms"], 5),
            "launches_per_step": res["launches"],
        },
    }
    if not args.no_cpu_baseline and args.config == 2 and args.scale == 1:
        base, cpu_out = cpu_baseline(arrays, gs)
        got = read_all(ctx, first_dsts[0])
        for dev, buf in cpu_out.items():
            if got[dev].tobytes() != buf.tobytes():
                sys.exit("bench.py: GPU result differs from the CPU restatement (device %d)" % dev)
        result["cpu_baseline"] = base
    else:
        result["cpu_baseline"] = None
    for s in first_srcs + first_dsts:
        ctx.Free(s)

    if args.all:
        others = {}
        for c in (1, 3, 4, 5):
            if c == args.config:
                continue
            r, *_rest = measure(ctx, mm, workloads, args, c)
            others["config%d" % c] = {"GB/s": round(r["achieved"], 1), "frac_hbm_peak": round(r["achieved"] / HBM_PEAK_GBS, 4),
                                       "kernel_ms": round(r["kernel_ms"], 5), "algorithmic_bytes": r["alg_bytes"],
                                       "launches_per_step": r["launches"], "kernel": r["kernel"],
                                       "plan_build_ms_cold": round(r["plan_build_ms"], 3)}
            for s in _rest[2] + _rest[3]:
                ctx.Free(s)
        result["all_configs"] = others
    ctx.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
