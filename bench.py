#!/usr/bin/env python3
"""Benchmark of the cross-submesh reshard on one MI355X.

A step is one reshard (one pass of the hot path over one batch of synthetic
input): configuration 2 of BASELINE.json, a bf16 [8, 4096, 8192] activation
resharded from hidden-sharded 8 ways (devices 0-7) to sequence-sharded 4 ways
(devices 8-11), all twelve shard buffers resident in this GPU's HBM before the
timed region starts.  Prints one JSON line.
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
    reshard_cpu.reshard(shards, so, do, out, nthreads=threads)  # warm-up, page in
    reps, t0 = 0, time.perf_counter()
    while True:
        reshard_cpu.reshard(shards, so, do, out, nthreads=threads)
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= seconds:
            break
    gbs = workloads.algorithmic_bytes(arrays) * reps / dt / 1e9
    return {"value": round(gbs, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "configuration 2 at full size, %d repetitions in %.1f s, C restatement of the reference "
                      "reshard (memcpy per contiguous run on %d pthreads)" % (reps, dt, threads)}, out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2, help="BASELINE.json configuration (1-5); 2 is the headline")
    ap.add_argument("--sets", type=int, default=3, help="independent buffer sets rotated between steps")
    ap.add_argument("--chunk-bytes", type=int, default=0)
    ap.add_argument("--order", type=int, default=0)
    ap.add_argument("--xcd-mode", type=int, default=0)
    ap.add_argument("--flags", type=int, default=0, help="debug plan flags")
    ap.add_argument("--name", type=str, default="", help="benchmark only the arrays whose name contains this")
    ap.add_argument("--scale", type=int, default=1, help="divide the large extents (probing only)")
    ap.add_argument("--only", type=int, default=-1, help="benchmark only array i of the configuration")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every logical device of both submeshes is a buffer in one "
                 "MI355X's HBM and nothing here uses a second GPU (got --gpus %d)" % args.gpus)

    import numpy as np
    import multimesh_jax_amd as mm
    from multimesh_jax_amd import workloads
    from gpu_helpers import make_stores, read_all
    from helpers import oracle_outputs

    # No torch in this process: PyTorch bundles its own HIP runtime and two HIP
    # runtimes cannot both drive the GPU.  The library owns its stream and its
    # device memory; ReshardContext raises if no GPU is present (no CPU fallback).
    arrays = workloads.config(args.config, args.scale)
    if args.only >= 0:
        arrays = [arrays[args.only]]
    if args.name:
        arrays = [a for a in arrays if args.name in a["name"]]
    gs = [workloads.generate(a) for a in arrays]
    alg_bytes = workloads.algorithmic_bytes(arrays)

    ctx = mm.ReshardContext(0)
    if args.chunk_bytes or args.order or args.xcd_mode or args.flags:
        ctx.set_plan_options(args.chunk_bytes, args.order, args.xcd_mode, args.flags)
    sets = [make_stores(ctx, arrays, gs, poison=None) for _ in range(max(1, args.sets))]

    def step(i):
        srcs, dsts = sets[i % len(sets)]
        if len(srcs) == 1:
            ctx.Reshard(srcs[0], dsts[0])
        else:
            ctx.ReshardBatch(srcs, dsts)

    # parity before timing: first set against the oracle, bit for bit
    step(0)
    ctx.Sync()
    if args.config not in (4, 9, 10, 11, 12):
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
    # HIP events on the context's own stream give the kernel time inside it
    t0 = time.perf_counter()
    ctx.StartTimer()
    for i in range(args.steps):
        step(i)
    kernel_ms = ctx.StopTimer()
    ctx.Sync()
    wall_s = time.perf_counter() - t0

    ms_per_step = wall_s * 1e3 / args.steps
    value = alg_bytes / (wall_s / args.steps) / 1e9
    launches = {1: 1, 2: 1, 3: 1, 4: 1, 5: 2}.get(args.config, 1)
    kernel_ms_per_launch = kernel_ms / args.steps
    achieved = alg_bytes / (kernel_ms_per_launch * 1e-3) / 1e9
    plan = ctx.plan_stats(sets[0][0][0], sets[0][1][0]) if len(arrays) == 1 else None

    traffic = None
    tpath = os.path.join(ROOT, "profiles", "traffic_config%d.json" % args.config)
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic = json.load(f).get("hbm_bytes_per_launch")

    result = {
        "metric": "reshard GB/s ((read+write bytes)/time) & % HBM peak, bf16 [8,4096,8192]",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u128" if args.config in (1, 2, 3, 4) else "u8",
        "data": "synthetic",
        "config": {
            "workload": "configuration %d of BASELINE.json: %s" % (
                args.config, "; ".join("%s %s %s" % (a["name"], a["type"], list(a["shape"])) for a in arrays[:3])
                + (" ... (%d arrays)" % len(arrays) if len(arrays) > 3 else "")),
            "source": arrays[0]["src"], "destination": arrays[0]["dst"],
            "algorithmic_bytes": alg_bytes, "buffer_sets": len(sets),
            "plan": plan, "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        },
        "roofline": {
            "bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
            "kernel": "mmr_copy16_kernel", "kernel_ms": round(kernel_ms_per_launch, 5),
            "launches_per_step": launches,
        },
    }
    if not args.no_cpu_baseline and args.config == 2:
        base, cpu_out = cpu_baseline(arrays, gs)
        got = read_all(ctx, sets[0][1][0])
        for dev, buf in cpu_out.items():
            if got[dev].tobytes() != buf.tobytes():
                sys.exit("bench.py: GPU result differs from the CPU restatement (device %d)" % dev)
        result["cpu_baseline"] = base
    else:
        result["cpu_baseline"] = None
    ctx.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
