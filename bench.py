#!/usr/bin/env python3
"""Benchmark of the cross-submesh reshard on one MI355X.

A step is one reshard (one pass of the hot path over one batch of synthetic
input).  The headline workload is configuration 2 of BASELINE.json, the one the
metric is quoted on: a bf16 [8, 4096, 8192] activation resharded from
hidden-sharded 8 ways (devices 0-7) to sequence-sharded 4 ways (devices 8-11),
all twelve shard buffers resident in this GPU's HBM before the timed region
starts.  The other four configurations are measured with the same protocol and
reported under `all_configs`.  Prints one JSON line.

Protocol (per configuration): every result is first compared bit for bit with
the oracle; buffer sets are rotated between launches so that the 256 MB
Infinity Cache serves none of the reads; W warm-up launches; K launches timed
as a whole (wall clock bracketed by synchronisation -> `value`; HIP events on
the library's stream around the same K launches -> `roofline.achieved`); then
at least 50 more launches with a timing mark between each two -> median and
p10 / p90 per launch.

No torch in this process: PyTorch's wheel bundles its own HIP runtime and two
HIP runtimes cannot both drive the GPU.  The library owns its stream and its
device memory, and raises if no GPU is present (there is no CPU fallback).
"""
import argparse
import glob
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak
# What the two counters report (KiB per dispatch) for a 512 MiB device-to-device copy by the HIP runtime's own kernel
# (__amd_rocclr_copyBuffer, `bench.py --calibrate-copy`): FETCH_SIZE 262,155.5 -> x 2.000, WRITE_SIZE 524,288.0 -> x 1.000
FETCH_SCALE, WRITE_SCALE = 2.000, 1.000


def kernel_sources_digest():
    """Digest of the sources the kernels and the planner are built from: a traffic profile measured on other
    sources says nothing about this build."""
    h = hashlib.sha256()
    base = os.path.join(ROOT, "multimesh-jax_amd", "csrc")
    # the kernels, the per-workgroup code and the planner (what decides which bytes a launch touches); not the host
    # code around them
    for name in ("chunk_ops.h", "geometry.cc", "group_ops.h", "kernels.h", "kernels.hip", "planner.cc", "planner.h"):
        with open(os.path.join(base, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def cpu_baseline(arrays, gs, seconds=12.0):
    """The C restatement of the reference reshard (oracle/reshard_cpu.c) timed on
    this box's host cores over the same workload; a reported baseline only."""
    import numpy as np
    from oracle import reshard_cpu, reshard_oracle as ro
    from helpers import oracle_shape, raw_global
    from multimesh_jax_amd import workloads

    visible = len(os.sched_getaffinity(0))
    # the GPU box grants one GPU's share of its host (16 threads; it exports OMP_NUM_THREADS accordingly)
    share = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
    threads = min(visible, share) if share > 0 else visible
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
            "single_thread_value": round(one, 2), "host_cores_visible": visible,
            "sample": "configuration 2 at full size: %d repetitions in %.1f s on %d pthreads (this box's share of its "
                      "host: %d hardware threads visible) and %d repetitions in %.1f s on 1 thread; C restatement of the "
                      "reference reshard, one memcpy per contiguous run"
                      % (reps, dt, threads, visible, reps1, dt1)}, out




def percentile(sorted_values, q):
    if not sorted_values:
        return None
    i = min(len(sorted_values) - 1, max(0, int(round(q * (len(sorted_values) - 1)))))
    return sorted_values[i]


def check_parity(ctx, arrays, gs, dsts, sample_only):
    """GPU result against the oracle, bit for bit; for the 10 GB pytree a sample of its arrays (every array of the
    first layer, the embedding and the output head)."""
    from gpu_helpers import read_all
    from helpers import oracle_outputs

    picked = range(len(arrays))
    if sample_only:
        picked = [i for i, a in enumerate(arrays) if a["name"].startswith("layer00.") or "." not in a["name"]]
    for i in picked:
        expect = oracle_outputs(arrays[i], gs[i])
        got = read_all(ctx, dsts[i])
        for dev in expect:
            if got[dev].tobytes() != expect[dev].tobytes():
                sys.exit("bench.py: GPU result differs from the oracle (array %s, device %d)" % (arrays[i]["name"], dev))
    return len(list(picked))


def measure(ctx, mm, workloads, args, config):
    """Creates the stores of one configuration, checks the result against the oracle, times it.
    Returns (result dict, arrays, gs, first destination stores, first source stores)."""
    from gpu_helpers import make_stores
    from helpers import lib_shape

    arrays = workloads.load_json(args.workload_json) if args.workload_json else workloads.config(config, args.scale)
    if args.name:
        arrays = [a for a in arrays if args.name in a["name"]]
    gs = [workloads.generate(a) for a in arrays]
    alg_bytes = workloads.algorithmic_bytes(arrays)
    # Buffer sets rotated between launches: at least `--sets`, and enough of them that 768 MiB of other buffers are
    # touched before a set comes round again - the 256 MB Infinity Cache must not serve a small configuration's reads
    # (an explicit --sets 1 or 2 is a probing run and is taken as given).
    n_sets = max(1, args.sets)
    if args.sets >= 3:
        n_sets = max(n_sets, -(-(768 << 20) // max(alg_bytes, 1)) + 1)
    sets = [make_stores(ctx, arrays, gs, poison=None) for _ in range(n_sets)]
    single = len(arrays) == 1

    def step(i):
        srcs, dsts = sets[i % len(sets)]
        if single:
            ctx.Reshard(srcs[0], dsts[0])
        elif args.unbatched:  # one call and one launch per array, as the reference's schedule loop issues them
            for s_, d_ in zip(srcs, dsts):
                ctx.Reshard(s_, d_)
        else:
            ctx.ReshardBatch(srcs, dsts)

    # Schedule-build time work (MpmdScheduler::AddReshardTask in the reference): plan and device tables for every
    # set.  None of it is in a timed region.
    before = ctx.stats
    step(0)
    ctx.Sync()
    launches = ctx.stats["kernel_launches"] - before["kernel_launches"]
    checked = check_parity(ctx, arrays, gs, sets[0][1], sample_only=alg_bytes > (2 << 30))

    def bind_all():
        if not args.unbatched:
            for srcs, dsts in sets:
                ctx.BindReshard(srcs, dsts)

    def timed(with_laps):
        """W warm-up steps, then exactly K steps: wall clock bracketed by synchronisation, HIP events on the
        library's own stream for the device time inside it; then five more brackets of 50 launches and, with
        `with_laps`, a timing mark between each two of at least 50 more launches."""
        for i in range(args.warmup):
            step(i)
        ctx.Sync()
        syncs_before = ctx.stats["host_blocking_syncs"]
        t0 = time.perf_counter()
        ctx.StartTimer()
        for i in range(args.steps):
            step(i)
        syncs = ctx.stats["host_blocking_syncs"] - syncs_before  # waits the K reshards themselves caused
        kernel_ms = ctx.StopTimer()  # blocks until the device gets there (a counted wait, asked for here)
        ctx.Sync()
        wall_s = time.perf_counter() - t0
        brackets = []
        for _ in range(5):
            ctx.StartTimer()
            for i in range(50):
                step(i)
            brackets.append(ctx.StopTimer() / 50)
        brackets.sort()
        laps = []
        if with_laps:
            n_laps = max(50, min(args.steps, 500))
            ctx.Lap()
            for i in range(n_laps):
                step(i)
                ctx.Lap()
            laps = sorted(ctx.Laps())
        return {"kernel_ms": kernel_ms / args.steps, "wall_s": wall_s, "syncs": syncs, "brackets": brackets, "laps": laps}

    # the planner's own launch order first ...
    bind_all()
    untuned = timed(with_laps=not (args.tune and not args.unbatched))
    run = untuned
    order_used = 0
    # ... then, on request, the order mmr_reshard_tune keeps after timing a few on the first buffer set (a caller does
    # this once, where it builds its schedule); measured again only if it kept another order than the default
    if args.tune and not args.unbatched:
        order_used = ctx.TuneReshard(sets[0][0], sets[0][1])
        if order_used != 0:
            bind_all()
            step(0)
            ctx.Sync()
            check_parity(ctx, arrays, gs, sets[0][1], sample_only=alg_bytes > (2 << 30))  # same bytes, whatever order
        run = timed(with_laps=True)  # the kept order (the default's second measurement if nothing else was kept)
    kernel_ms, wall_s, syncs_in_region = run["kernel_ms"] * args.steps, run["wall_s"], run["syncs"]
    brackets, laps = run["brackets"], run["laps"]

    batched = len(arrays) > 1 and not args.unbatched
    plan = (ctx.plan_stats(sets[0][0][0], sets[0][1][0]) if single else
            ctx.batch_plan_stats(sets[0][0], sets[0][1]) if batched else None)
    # cold plan construction (host only, outside the steady-state figure: plans are cached per descriptor pair)
    src_shapes = [lib_shape(a["type"], a["src"]) for a in arrays]
    dst_shapes = [lib_shape(a["type"], a["dst"]) for a in arrays]
    tp = time.perf_counter()
    cold = mm.Plan(src_shapes, dst_shapes, args.chunk_bytes, args.order, args.xcd_mode, args.flags)
    plan_build_ms = (time.perf_counter() - tp) * 1e3
    table_bytes = cold.stats["table_bytes"]
    del cold
    kernel = "mmr_copy16_kernel"
    if plan is not None:
        kinds = [("mmr_transpose_kernel", plan["n_transpose_chunks"] * 32768), ("mmr_span_kernel", plan["n_span_chunks"] * 8192),
                 ("mmr_copy_generic_kernel", plan["n_copy_generic_chunks"] * 5120), ("mmr_copy16_kernel", plan["n_copy16_chunks"] * 8192)]
        kernel = max(kinds, key=lambda kv: kv[1])[0]  # the class that moves most of the bytes
    med = percentile(laps, 0.5)
    res = {
        "alg_bytes": alg_bytes,
        "ms_per_step": wall_s * 1e3 / args.steps,
        "value": alg_bytes / (wall_s / args.steps) / 1e9,
        "kernel_ms": kernel_ms / args.steps,
        "achieved": alg_bytes / (kernel_ms / args.steps * 1e-3) / 1e9,
        "median_ms": med, "p10_ms": percentile(laps, 0.1), "p90_ms": percentile(laps, 0.9), "laps": len(laps),
        "bracket_median_ms": brackets[2], "bracket_min_ms": brackets[0], "bracket_max_ms": brackets[-1],
        "median_gbs": alg_bytes / (med * 1e-3) / 1e9 if med else None,
        "launches": launches, "plan": plan, "plan_build_ms": plan_build_ms, "plan_table_bytes": table_bytes,
        "kernel": kernel, "n_arrays": len(arrays), "sets": len(sets), "order_used": order_used,
        "orders_timed": plan["orders_timed"] if plan else 0, "parity_arrays": checked,
        "host_blocking_syncs_in_timed_region": syncs_in_region,
        # the same protocol with the planner's default launch order (what a caller gets who never calls mmr_reshard_tune)
        "untuned_kernel_ms": untuned["kernel_ms"], "untuned_achieved": alg_bytes / (untuned["kernel_ms"] * 1e-3) / 1e9,
        "untuned_bracket_median_ms": untuned["brackets"][2],
    }
    first_dsts = sets[0][1]
    for srcs, dsts in sets[1:]:
        for s in srcs + dsts:
            ctx.Free(s)
    return res, arrays, gs, first_dsts, sets[0][0]


def traffic_of(config, args):
    """HBM bytes per launch of the dominant kernel from the committed counter profile of this configuration
    (profiles/traffic_config<c>.json, written by --record-traffic from rocprofv3 --pmc runs), or null when that
    profile was measured on other kernel or planner sources than the ones this build comes from."""
    path = os.path.join(ROOT, "profiles", "traffic_config%d.json" % config)
    if not os.path.exists(path) or args.scale != 1 or args.name or args.workload_json:
        return None, None
    with open(path) as f:
        prof = json.load(f)
    if prof.get("kernel_sources_digest") != kernel_sources_digest():
        return None, "profiles/traffic_config%d.json is stale: measured on kernel sources %s, these are %s" % (
            config, prof.get("kernel_sources_digest"), kernel_sources_digest())
    return prof.get("hbm_bytes_per_launch"), "profiles/traffic_config%d.json (%s)" % (config, prof.get("source", ""))


def record_traffic(args):
    """Writes profiles/traffic_config<c>.json from the two counter runs of one configuration:
         rocprofv3 --pmc FETCH_SIZE --kernel-trace --output-format csv -d <dir>/FETCH_SIZE -o p -- python3 bench.py --config c ...
         rocprofv3 --pmc WRITE_SIZE ... -d <dir>/WRITE_SIZE ...
       (one counter per run).  Counter values are KiB per dispatch."""
    import csv
    from multimesh_jax_amd import workloads
    out = {}
    kernel = None
    for counter, scale in (("FETCH_SIZE", FETCH_SCALE), ("WRITE_SIZE", WRITE_SCALE)):
        files = glob.glob(os.path.join(args.record_traffic, counter, "**", "*counter_collection.csv"), recursive=True)
        if not files:
            sys.exit("no counter_collection.csv under %s/%s" % (args.record_traffic, counter))
        per_kernel = {}
        with open(files[0]) as f:
            for row in csv.DictReader(f):
                if "mmr_" in row["Kernel_Name"] and row["Counter_Name"] == counter:
                    name = row["Kernel_Name"].replace("(anonymous namespace)::", "").replace("void ", "")
                    per_kernel.setdefault(name.split("(")[0], []).append(float(row["Counter_Value"]))
        name, values = max(per_kernel.items(), key=lambda kv: sum(kv[1]))
        kernel = name
        out[counter] = {"kib_mean": sum(values) / len(values), "kib_min": min(values), "kib_max": max(values),
                        "dispatches": len(values), "scale": scale}
    arrays = workloads.config(args.config)
    alg = workloads.algorithmic_bytes(arrays)
    # a very long copy table leaves in several dispatches per launch (mmr_plan_stats.n_copy16_launches)
    per_launch = 1
    if "mmr_copy16" in kernel:
        import multimesh_jax_amd as mm
        def shape_of(type_, side):
            return mm.sharded_shape(type_, side["dims"], side["dev_start"], side["dev_count"], side.get("minor_to_major"))
        plan = mm.api.Plan([shape_of(a["type"], a["src"]) for a in arrays], [shape_of(a["type"], a["dst"]) for a in arrays])
        per_launch = plan.stats["n_copy16_launches"]
    for counter in out:
        out[counter]["dispatches_per_launch"] = per_launch
    hbm = int((out["FETCH_SIZE"]["kib_mean"] * FETCH_SCALE + out["WRITE_SIZE"]["kib_mean"] * WRITE_SCALE) * 1024 * per_launch)
    import subprocess
    try:  # the commit whose sources the counters were measured on (the digest is what bench.py checks)
        commit = subprocess.check_output(["git", "-C", ROOT, "rev-parse", "HEAD"], stderr=subprocess.DEVNULL).decode().strip()
        if subprocess.call(["git", "-C", ROOT, "diff", "--quiet", "HEAD", "--", "multimesh-jax_amd/csrc", "include"]) != 0:
            commit += " + uncommitted changes"
    except Exception:
        commit = None
    prof = {"config": args.config, "kernel": kernel, "counters": out, "hbm_bytes_per_launch": hbm,
            "algorithmic_bytes": alg, "ratio": round(hbm / alg, 4), "kernel_sources_digest": kernel_sources_digest(),
            "measured_at_commit": commit,
            "source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, one counter per run, KiB per dispatch; "
                      "FETCH_SIZE x %.3f, WRITE_SIZE x %.3f" % (FETCH_SCALE, WRITE_SCALE)}
    path = os.path.join(ROOT, "profiles", "traffic_config%d.json" % args.config)
    with open(path, "w") as f:
        json.dump(prof, f, indent=1)
        f.write("\n")
    print(json.dumps(prof))


def through_context(result, others):
    """The same reshards behind the reference-shaped interface: tests/cpp/context_bench builds configurations 2 and
    4 as a ReshardSchedule and runs ReshardSchedule::Execute over HipExecuteContext with 12 local devices (one Reshard
    call per array and local device, fresh root stores and the OpenWindow / StartTimer / ... / CloseWindow bracket
    every execution).  Each runs as a child process of its own, started after this process has closed its context."""
    import subprocess
    exe = os.path.join(ROOT, "tests", "cpp", "context_bench")
    if not os.path.exists(exe):
        return {"error": "tests/cpp/context_bench is not built (tests/cpp/build.sh)"}
    direct = {2: result if result["config"]["workload"].startswith("configuration 2") else others.get("config2"),
              4: others.get("config4")}
    out = {}
    for config, executions in ((2, 100), (4, 30)):
        try:
            p = subprocess.run([exe, str(config), str(executions)], capture_output=True, text=True, timeout=240)
        except subprocess.TimeoutExpired:
            out["config%d" % config] = {"error": "timed out"}
            continue
        if p.returncode != 0:
            out["config%d" % config] = {"error": (p.stdout + p.stderr)[-400:], "returncode": p.returncode}
            continue
        r = json.loads(p.stdout.strip().splitlines()[-1])
        d = direct.get(config)
        if d is not None:
            direct_ms = d["ms_per_step"]
            direct_kernel_ms = d["roofline"]["kernel_ms"] if "roofline" in d else d["kernel_ms"]
            r["direct_c_abi_ms_per_step"] = direct_ms
            r["direct_c_abi_kernel_ms"] = direct_kernel_ms
            r["wall_over_direct"] = round(r["wall_ms_per_execution"] / direct_ms, 4)
            r["host_ms_over_kernel_ms"] = round(r["host_ms_per_execute_median"] / direct_kernel_ms, 4)
        out["config%d" % config] = r
    return out


def summary(r):
    return {"GB/s": round(r["achieved"], 1), "frac_hbm_peak": round(r["achieved"] / HBM_PEAK_GBS, 4),
            "kernel_ms": round(r["kernel_ms"], 5), "ms_per_step": round(r["ms_per_step"], 5),
            "wall_GB/s": round(r["value"], 1), "median_ms": round(r["median_ms"], 5),
            "p10_ms": round(r["p10_ms"], 5), "p90_ms": round(r["p90_ms"], 5), "launches_timed": r["laps"],
            "bracket_median_ms": round(r["bracket_median_ms"], 5),
            "median_GB/s": round(r["median_gbs"], 1), "algorithmic_bytes": r["alg_bytes"],
            "launches_per_step": r["launches"], "kernel": r["kernel"], "buffer_sets": r["sets"],
            "plan_build_ms_cold": round(r["plan_build_ms"], 3), "plan_table_bytes": r["plan_table_bytes"],
            "order_used": r["order_used"], "orders_timed": r["orders_timed"], "parity_arrays_checked": r["parity_arrays"],
            "untuned_kernel_ms": round(r["untuned_kernel_ms"], 5), "untuned_GB/s": round(r["untuned_achieved"], 1),
            "untuned_frac_hbm_peak": round(r["untuned_achieved"] / HBM_PEAK_GBS, 4)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2, help="BASELINE.json configuration (1-5); 2 is the headline")
    ap.add_argument("--sets", type=int, default=3, help="independent buffer sets rotated between steps")
    ap.add_argument("--only", action="store_true", help="measure --config alone (no all_configs)")
    ap.add_argument("--all", action="store_true", help="accepted for compatibility: all_configs is the default")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-through-context", action="store_true",
                    help="skip the child runs that time configurations 2 and 4 through ReshardSchedule::Execute")
    ap.add_argument("--no-tune", dest="tune", action="store_false",
                    help="keep the planner's default launch order instead of timing a few on the first buffer set")
    ap.add_argument("--unbatched", action="store_true",
                    help="multi-array configurations: one Reshard call per array instead of one batched call (probing)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="instead of a reshard, copy 512 MiB device to device with the HIP runtime's own copy kernel a few "
                         "times (run under rocprofv3 --pmc FETCH_SIZE or WRITE_SIZE: the counters' factors for a kernel "
                         "that is not this library's)")
    ap.add_argument("--record-traffic", type=str, default="",
                    help="directory with FETCH_SIZE/ and WRITE_SIZE/ rocprofv3 --pmc outputs of --config: writes "
                         "profiles/traffic_config<c>.json and exits (needs no GPU)")
    # plan options (0 = library default) and probing switches
    ap.add_argument("--chunk-bytes", type=int, default=0)
    ap.add_argument("--order", type=int, default=0)
    ap.add_argument("--xcd-mode", type=int, default=0)
    ap.add_argument("--flags", type=int, default=0)
    ap.add_argument("--name", type=str, default="", help="only the arrays whose name contains this")
    ap.add_argument("--scale", type=int, default=1, help="divide the large extents (probing only)")
    ap.add_argument("--workload-json", type=str, default="",
                    help="measure the arrays described in this JSON file instead of a BASELINE.json configuration "
                         "(a list of {name, type, shape, src, dst, seed, dist} as multimesh-jax_amd/workloads.py builds them)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every logical device of both submeshes is a buffer in one "
                 "MI355X's HBM and nothing here uses a second GPU (got --gpus %d)" % args.gpus)
    if args.record_traffic:
        record_traffic(args)
        return

    import multimesh_jax_amd as mm
    from multimesh_jax_amd import workloads
    from gpu_helpers import read_all

    ctx = mm.ReshardContext(0)
    if args.calibrate_copy:
        shape = (8, 4096, 8192)
        a = mm.sharded_shape("BF16", [(n, 1, i) for i, n in enumerate(shape)], 0, 1)
        b = mm.sharded_shape("BF16", [(n, 1, i) for i, n in enumerate(shape)], 1, 1)
        src, dst = ctx.CreateStore(a), ctx.CreateStore(b)
        ptr = ctx.SliceLocalShard(0, src)
        for _ in range(5):
            ctx.AssembleShards(b, 1, ptr, existing_store=dst, size=512 << 20, where=3)
        ctx.Sync()
        print(json.dumps({"calibration": "5 x hipMemcpyAsync device to device of %d bytes" % (512 << 20)}))
        ctx.close()
        return
    if args.chunk_bytes or args.order or args.xcd_mode or args.flags:
        ctx.set_plan_options(args.chunk_bytes, args.order, args.xcd_mode, args.flags)

    res, arrays, gs, first_dsts, first_srcs = measure(ctx, mm, workloads, args, args.config)
    traffic, traffic_source = traffic_of(args.config, args)

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
            "workload": (args.workload_json or "configuration %d of BASELINE.json" % args.config) + ": " + "; ".join(
                "%s %s %s" % (a["name"], a["type"], list(a["shape"])) for a in arrays[:3])
                + (" ... (%d arrays)" % len(arrays) if len(arrays) > 3 else ""),
            "source": arrays[0]["src"], "destination": arrays[0]["dst"],
            "algorithmic_bytes": res["alg_bytes"], "buffer_sets": res["sets"],
            "plan": res["plan"], "plan_build_ms_cold": round(res["plan_build_ms"], 3),
            "plan_table_bytes": res["plan_table_bytes"], "pct_hbm_peak": round(100.0 * res["value"] / HBM_PEAK_GBS, 2),
            "order_used": res["order_used"], "orders_timed": res["orders_timed"],
            "host_blocking_syncs_in_timed_region": res["host_blocking_syncs_in_timed_region"],
        },
        "roofline": {
            "bound": "hbm", "achieved": round(res["achieved"], 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(res["achieved"] / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_source,
            "kernel": res["kernel"], "kernel_ms": round(res["kernel_ms"], 5),
            "median_ms": round(res["median_ms"], 5), "p10_ms": round(res["p10_ms"], 5), "p90_ms": round(res["p90_ms"], 5),
            "launches_timed_one_by_one": res["laps"], "median_GB/s": round(res["median_gbs"], 1),
            # median (min, max) of five brackets of 50 back-to-back launches each, events on the library's stream
            "bracket_median_ms": round(res["bracket_median_ms"], 5), "bracket_min_ms": round(res["bracket_min_ms"], 5),
            "bracket_max_ms": round(res["bracket_max_ms"], 5),
            "launches_per_step": res["launches"],
            # the planner's default launch order, measured with the same protocol before mmr_reshard_tune ran
            "untuned_kernel_ms": round(res["untuned_kernel_ms"], 5),
            "untuned_frac": round(res["untuned_achieved"] / HBM_PEAK_GBS, 4), "order_used": res["order_used"],
            # the same launch priced at the bytes the HBM counters saw instead of the algorithmic ones
            "traffic_over_algorithmic": round(traffic / res["alg_bytes"], 4) if traffic else None,
            "counter_GB/s": round(traffic / (res["kernel_ms"] * 1e-3) / 1e9, 1) if traffic else None,
        },
    }
    if not args.no_cpu_baseline and args.config == 2 and args.scale == 1 and not args.workload_json:
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
    ctx.ClearStoreCache()

    if not args.only and not args.workload_json and args.scale == 1 and not args.name:
        others = {}
        for c in (1, 2, 3, 4, 5):
            if c == args.config:
                continue
            r, _arrays, _gs, dsts_, srcs_ = measure(ctx, mm, workloads, args, c)
            others["config%d" % c] = summary(r)
            t, tsrc = traffic_of(c, args)
            others["config%d" % c]["traffic"] = t
            others["config%d" % c]["traffic_source"] = tsrc
            for s in srcs_ + dsts_:
                ctx.Free(s)
            ctx.ClearStoreCache()
        result["all_configs"] = others
    ctx.close()
    if not args.only and not args.workload_json and args.scale == 1 and not args.name and not args.no_through_context:
        result["through_context"] = through_context(result, others if "all_configs" in result else {})
    print(json.dumps(result))


if __name__ == "__main__":
    main()
