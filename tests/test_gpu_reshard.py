"""Parity of the HIP path with the oracle, through the C ABI, on a real MI355X.

Bar: bit-exact (pure data movement; integer, byte and float bit patterns alike).
"""
import random
import sys

import numpy as np
import pytest

import multimesh_jax_amd as mm
from multimesh_jax_amd import _binding as B, workloads
from oracle import reshard_cpu, reshard_oracle as ro

from helpers import lib_shape, oracle_outputs, oracle_shape, raw_global
from gpu_helpers import gpu_reshard, make_stores, read_all

pytestmark = pytest.mark.gpu


def say(msg):
    print("[gpu-test] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    c = mm.ReshardContext(0)
    yield c
    c.close()


def _compare(arrays, gs, outs):
    for a, g, out in zip(arrays, gs, outs):
        expect = oracle_outputs(a, g)
        assert sorted(out) == sorted(expect)
        for dev in expect:
            assert out[dev].tobytes() == expect[dev].tobytes(), (a["name"], dev)


@pytest.mark.parametrize("index", [1, 2, 3, 5, 6])
def test_benchmark_config_full_size(ctx, index):
    say("config %d full size" % index)
    arrays = workloads.config(index)
    gs = [workloads.generate(a) for a in arrays]
    outs = gpu_reshard(ctx, arrays, gs)
    _compare(arrays, gs, outs)


@pytest.mark.parametrize("flags", [0, B.MMR_PLAN_NO_SEGMENT_TABLES, B.MMR_PLAN_NO_SPAN, B.MMR_PLAN_ALL_GENERIC,
                                   B.MMR_PLAN_ALL_GENERIC | B.MMR_PLAN_NO_SEGMENT_TABLES])
def test_ragged_rows_through_every_gather(ctx, flags):
    """Ragged rows through the span kernel with and without its segment table, through the generic kernel, and aligned
    configurations forced through both span gathers: the same bytes every way."""
    say("ragged rows, plan flags %d" % flags)
    ctx.set_plan_options(0, 0, 0, flags)
    try:
        cases = [workloads.config(5), workloads.config(6, 4), workloads.config(2, 8), workloads.config(3, 4)]
        # long ragged rows under two row dims, 1 to 6 pieces per destination row
        for cols, s_src, s_dst in ((1031, 3, 2), (2600, 4, 5), (700, 6, 1), (130, 1, 5)):
            cases.append([{"name": "rag3", "type": "U8", "shape": (3, 50, cols),
                           "src": {"dims": [(3, 1, 0), (50, 1, 1), (cols, s_src, 2)], "dev_start": 0, "dev_count": s_src},
                           "dst": {"dims": [(3, 1, 1), (50, 1, 2), (cols, s_dst, 0)], "dev_start": 9, "dev_count": s_dst},
                           "seed": cols, "dist": "raw"}])
        for arrays in cases:
            gs = [workloads.generate(a) for a in arrays]
            _compare(arrays, gs, gpu_reshard(ctx, arrays, gs))
    finally:
        ctx.set_plan_options(0, 0)


@pytest.mark.parametrize("chunk_bytes,order", [(4096, 1), (16384, 3), (262144, 2)])
def test_plan_options_do_not_change_results(ctx, chunk_bytes, order):
    say("plan options chunk=%d order=%d" % (chunk_bytes, order))
    ctx.set_plan_options(chunk_bytes, order)
    try:
        for index, scale in ((2, 8), (3, 4), (5, 8)):
            arrays = workloads.config(index, scale)
            gs = [workloads.generate(a) for a in arrays]
            _compare(arrays, gs, gpu_reshard(ctx, arrays, gs))
    finally:
        ctx.set_plan_options(0, 0)


def test_config4_scaled_batched_bit_exact(ctx):
    say("config 4 scale 8, one batched plan")
    arrays = workloads.config(4, 8)
    gs = [workloads.generate(a) for a in arrays]
    before = ctx.stats
    outs = gpu_reshard(ctx, arrays, gs, batch=True)
    after = ctx.stats
    _compare(arrays, gs, outs)
    assert after["reshard_calls"] - before["reshard_calls"] == 1
    assert after["kernel_launches"] - before["kernel_launches"] <= 2


def test_config4_full_size_round_trip_and_samples(ctx):
    """10.7 GB of traffic: checked through size-independent properties (the
    A->B->A round trip restores every source byte; per-array XOR checksums are
    preserved) plus exact comparison with the oracle for a sample of arrays."""
    say("config 4 full size")
    arrays = workloads.config(4)
    rng = np.random.Generator(np.random.PCG64(4))
    gs = []
    pool = rng.standard_normal(size=1 << 24, dtype=np.float32) * np.float32(0.02)
    for i, a in enumerate(arrays):
        n = int(np.prod(a["shape"]))
        reps = -(-n // pool.size)
        g = np.tile(np.roll(pool, i * 977), reps)[:n].reshape(a["shape"]).view(np.uint32)
        gs.append(g)
    outs, srcs, dsts = gpu_reshard(ctx, arrays, gs, batch=True, keep=True)
    sample = [i for i, a in enumerate(arrays) if a["name"] in
              ("layer00.ln1", "layer00.wq", "layer11.w_in", "layer23.w_out", "embed", "final_ln", "lm_head")]
    _compare([arrays[i] for i in sample], [gs[i] for i in sample], [outs[i] for i in sample])
    for a, g, out in zip(arrays, gs, outs):
        x = np.bitwise_xor.reduce(g.reshape(-1))
        y = np.uint32(0)
        for buf in out.values():
            y ^= np.bitwise_xor.reduce(buf.view(np.uint32))
        assert x == y, a["name"]
    del outs
    # round trip back into fresh stores laid out like the sources
    back = [ctx.CreateStore(lib_shape(a["type"], a["src"]), name=a["name"] + ".back") for a in arrays]
    ctx.ReshardBatch(dsts, back)
    ctx.Sync()
    for a, s, b in zip(arrays, srcs, back):
        for dev in s.devices:
            assert ctx.ReadShard(s, dev).tobytes() == ctx.ReadShard(b, dev).tobytes(), (a["name"], dev)
    for st in srcs + dsts + back:
        ctx.Free(st)


def _random_array(rnd, types=("U8", "BF16", "F32", "F64", "C128"), extents=None):
    rank = rnd.randint(1, 4)
    shape = [rnd.choice(extents or [1, 2, 3, 5, 8, 17, 33, 64, 130]) for _ in range(rank)]
    while int(np.prod(shape)) > 3_000_000:
        shape[rnd.randrange(rank)] = rnd.choice([1, 2, 3, 5, 8])
    type_ = rnd.choice(types)

    def side(start):
        shard = [rnd.randint(1, 4) for _ in range(rank)]
        repl = rnd.choice([1, 1, 2, 3])
        if repl == 1 and shape[-1] == 1:
            shard[-1] = 1
        entries = shard + ([repl] if repl > 1 else [])
        perm = list(range(len(entries)))
        rnd.shuffle(perm)
        dims = [(shape[i], shard[i], perm[i]) for i in range(rank)]
        if repl > 1:
            dims.append((1, repl, perm[rank]))
        d = {"dims": dims, "dev_start": start, "dev_count": int(np.prod(entries))}
        if rnd.random() < 0.5:
            m2m = list(range(rank))
            rnd.shuffle(m2m)
            d["minor_to_major"] = m2m
        return d

    return {"name": "r", "type": type_, "shape": tuple(shape), "src": side(rnd.randint(0, 3)),
            "dst": side(rnd.randint(0, 50)), "seed": 0, "dist": "raw"}


def test_random_sharding_pairs(ctx):
    """Ragged extents, permuted device orders, replication on either side,
    permuted layouts (copy, generic and transpose kernels), every element size."""
    rnd = random.Random(1234)
    rng = np.random.Generator(np.random.PCG64(99))
    for case in range(1500):
        a = _random_array(rnd, extents=(1, 2, 3, 5, 6, 8, 17, 33, 64, 70, 129, 130, 257, 300, 1030) if case >= 60 else None)
        if case < 60 or case % 100 == 0:
            say("random case %d: %s %s src=%s dst=%s" % (case, a["type"], a["shape"], a["src"], a["dst"]))
        item = ro.ITEMSIZE[a["type"]]
        g = rng.integers(0, 256, size=int(np.prod(a["shape"])) * item, dtype=np.uint8).view(
            ro.raw_dtype(a["type"])).reshape(a["shape"])
        _compare([a], [g], gpu_reshard(ctx, [a], [g]))


def test_random_batch_mixed_kernels(ctx):
    rnd = random.Random(77)
    rng = np.random.Generator(np.random.PCG64(5))
    arrays, gs = [], []
    for _ in range(25):
        a = _random_array(rnd)
        item = ro.ITEMSIZE[a["type"]]
        arrays.append(a)
        gs.append(rng.integers(0, 256, size=int(np.prod(a["shape"])) * item, dtype=np.uint8).view(
            ro.raw_dtype(a["type"])).reshape(a["shape"]))
    say("random batch of 25 arrays")
    outs, srcs, dsts = gpu_reshard(ctx, arrays, gs, batch=True, keep=True)
    _compare(arrays, gs, outs)
    # the batch has one plan of its own; its stats count every array and every kernel class of the batch
    built = ctx.stats["plans_built"]
    st = ctx.batch_plan_stats(srcs, dsts)
    assert ctx.stats["plans_built"] == built, "the stats call found the batch's cached plan"
    assert st["n_arrays"] == 25
    # every element is written once per destination replica
    assert st["bytes_moved"] == sum(g.nbytes * (a["dst"]["dims"][-1][1] if len(a["dst"]["dims"]) > g.ndim else 1)
                                    for a, g in zip(arrays, gs))
    for s in srcs + dsts:
        ctx.Free(s)


@pytest.mark.parametrize("type_", ["U8", "BF16", "F32", "F64", "C128"])
def test_transpose_kernel_large(ctx, type_):
    """A minor-changing layout at a size that fills many 64x64 tiles (the LDS path)."""
    say("transpose " + type_)
    shape = (3, 515, 389)
    item = ro.ITEMSIZE[type_]
    a = {"name": "t", "type": type_, "shape": shape,
         "src": {"dims": [(3, 1, 0), (515, 2, 1), (389, 1, 2)], "dev_start": 0, "dev_count": 2},
         "dst": {"dims": [(3, 1, 0), (515, 1, 1), (389, 3, 2)], "dev_start": 2, "dev_count": 3,
                 "minor_to_major": [1, 2, 0]},
         "seed": 0, "dist": "raw"}
    rng = np.random.Generator(np.random.PCG64(8))
    g = rng.integers(0, 256, size=int(np.prod(shape)) * item, dtype=np.uint8).view(ro.raw_dtype(type_)).reshape(shape)
    plan = mm.Plan(lib_shape(type_, a["src"]), lib_shape(type_, a["dst"]))
    assert plan.stats["n_transpose_chunks"] > 0
    _compare([a], [g], gpu_reshard(ctx, [a], [g]))


@pytest.mark.parametrize("type_", ["U8", "BF16", "F32", "F64", "C128"])
def test_transpose_ragged_and_misaligned_tiles(ctx, type_):
    """Transposed layouts whose tiles are not 16-byte aligned or do not hold whole vectors (unaligned accesses,
    vectors slid inwards at the edges, sub-tiles thinner than a vector), and one large odd-sized array."""
    item = ro.ITEMSIZE[type_]
    rng = np.random.Generator(np.random.PCG64(41))
    for shape, st_, dt_ in (((250, 381), (2, 1), (1, 3)), ((135, 203), (1, 1), (1, 1)), ((129, 257), (1, 2), (2, 1)),
                            ((20, 300), (1, 1), (1, 1)), ((300, 20), (1, 1), (1, 1)), ((3, 500), (1, 1), (1, 1)),
                            ((2046, 1027), (2, 1), (1, 2))):
        say("ragged transpose %s %r" % (type_, shape))
        ns = st_[0] * st_[1]
        a = {"name": "t", "type": type_, "shape": shape,
             "src": {"dims": [(shape[0], st_[0], 0), (shape[1], st_[1], 1)], "dev_start": 0, "dev_count": ns},
             "dst": {"dims": [(shape[0], dt_[0], 0), (shape[1], dt_[1], 1)], "dev_start": ns,
                     "dev_count": dt_[0] * dt_[1], "minor_to_major": [0, 1]},
             "seed": 0, "dist": "raw"}
        g = rng.integers(0, 256, size=int(np.prod(shape)) * item, dtype=np.uint8).view(ro.raw_dtype(type_)).reshape(shape)
        _compare([a], [g], gpu_reshard(ctx, [a], [g]))


@pytest.mark.parametrize("type_", ["U8", "BF16", "F32", "F64"])
def test_transpose_thin_tiles(ctx, type_):
    """A dimension of a few elements moving into or out of the minor position (3 channels, 6 heads): boxes thinner
    than one 16-byte vector take the kernel's thin path, with tiles as long as the workgroup's LDS allows."""
    item = ro.ITEMSIZE[type_]
    rng = np.random.Generator(np.random.PCG64(47))
    for shape, m2m in (((40, 700, 3), [1, 0, 2]), ((50, 6, 1030), [1, 2, 0]), ((7, 1, 33000), [1, 0, 2]),
                       ((300, 2000, 3), [1, 0, 2])):
        say("thin transpose %s %r" % (type_, shape))
        a = {"name": "t", "type": type_, "shape": shape,
             "src": {"dims": [(n, 1, i) for i, n in enumerate(shape)], "dev_start": 0, "dev_count": 1},
             "dst": {"dims": [(n, 1, i) for i, n in enumerate(shape)], "dev_start": 1, "dev_count": 1,
                     "minor_to_major": m2m},
             "seed": 0, "dist": "raw"}
        g = rng.integers(0, 256, size=int(np.prod(shape)) * item, dtype=np.uint8).view(ro.raw_dtype(type_)).reshape(shape)
        _compare([a], [g], gpu_reshard(ctx, [a], [g]))


def test_python_test_toy_shapes(ctx):
    """The shapes the reference's end-to-end Python tests reshard: (4,4) and (8,4)
    f32 between two 2-device meshes and from 4 devices onto 2+2."""
    rng = np.random.Generator(np.random.PCG64(21))
    cases = [
        ((4, 4), [(4, 2, 0), (4, 1, 1)], (0, 2), [(4, 2, 0), (4, 1, 1)], (2, 2)),
        ((8, 4), [(8, 2, 0), (4, 1, 1)], (0, 2), [(8, 1, 0), (4, 2, 1)], (2, 2)),
        ((8, 4), [(8, 4, 0), (4, 1, 1)], (0, 4), [(8, 2, 0), (4, 1, 1)], (4, 2)),
        ((8, 4), [(8, 4, 0), (4, 1, 1)], (0, 4), [(8, 1, 0), (4, 1, 1), (1, 2, 2)], (6, 2)),
    ]
    for shape, sd, (ss, sc), dd, (ds, dc) in cases:
        a = {"name": "toy", "type": "F32", "shape": shape,
             "src": {"dims": sd, "dev_start": ss, "dev_count": sc},
             "dst": {"dims": dd, "dev_start": ds, "dev_count": dc}, "seed": 0, "dist": "raw"}
        g = rng.standard_normal(size=shape, dtype=np.float32).view(np.uint32)
        _compare([a], [g], gpu_reshard(ctx, [a], [g]))


def test_scalar_broadcast_to_all_devices(ctx):
    """mpmd_insert_reshard.cc:194-214: a scalar root output living on a 4-device
    submesh is blasted out to all 8 devices."""
    a = {"name": "loss", "type": "F32", "shape": (),
         "src": {"dims": [(1, 4, 0)], "dev_start": 4, "dev_count": 4},
         "dst": {"dims": [(1, 8, 0)], "dev_start": 0, "dev_count": 8}, "seed": 0, "dist": "raw"}
    g = np.array(0x40490FDB, dtype=np.uint32).reshape(())
    outs = gpu_reshard(ctx, [a], [g])
    assert all(buf.view(np.uint32)[0] == 0x40490FDB for buf in outs[0].values())
    assert len(outs[0]) == 8


def test_cpu_restatement_agrees_at_full_size(ctx):
    """Third witness at the headline size: GPU == C restatement == NumPy oracle."""
    say("config 2 full size against the C restatement")
    a = workloads.config(2)[0]
    g = workloads.generate(a)
    so, do = oracle_shape(a["type"], a["src"]), oracle_shape(a["type"], a["dst"])
    shards = ro.make_shards(raw_global(a, g), so)
    cpu = {d: np.empty(int(np.prod(ro.shard_shape(do))), dtype=np.uint16) for d in range(8, 12)}
    reshard_cpu.reshard(shards, so, do, cpu, nthreads=8)
    outs = gpu_reshard(ctx, [a], [g])
    for dev in cpu:
        assert outs[0][dev].tobytes() == cpu[dev].tobytes()


def test_store_interface(ctx):
    """CreateStore / AssembleShards / SliceLocalShard / HasLocalShard /
    GetStoreShardedShape / Free with cache, as zuku_execute_context.h:38-133 lays them out."""
    shape = mm.sharded_shape("F32", [(16, 4, 0), (8, 1, 1)], 4, 4)
    st = ctx.CreateStore(shape, name="acts")
    assert st.name == "acts" and st.unique_id >= 0
    assert ctx.HasLocalShard(st, 4) and ctx.HasLocalShard(st, 7)
    assert not ctx.HasLocalShard(st, 3) and not ctx.HasLocalShard(st, 8)
    assert mm.describe(ctx.GetStoreShardedShape(st)) == mm.describe(shape)
    assert st.shard_bytes == 4 * 8 * 4
    # fresh stores are zero-filled
    assert not ctx.ReadShard(st, 5).any()
    # host shard in, device pointer out (zero copy view through torch)
    data = np.arange(32, dtype=np.float32)
    ctx.AssembleShards(shape, 6, data, existing_store=st)
    assert ctx.ReadShard(st, 6, np.float32).tolist() == data.tolist()
    ptr = ctx.SliceLocalShard(6, st)
    assert ptr != 0 and ptr % 256 == 0
    # device shard in (the GPU branch of AssembleShardsImpl): D2D from another store's buffer
    other = ctx.CreateStore(mm.sharded_shape("F32", [(32, 1, 0)], 0, 1), name="native")
    ctx.AssembleShards(other.shape, 0, data * 2, existing_store=other)
    ctx.AssembleShards(shape, 7, ctx.SliceLocalShard(0, other, wait=False), existing_store=st, size=32 * 4)
    assert ctx.ReadShard(st, 7, np.float32).tolist() == (data * 2).tolist()
    ctx.Free(other)
    # a device outside the store's device list holds no shard
    with pytest.raises(mm.MmrError) as e:
        ctx.SliceLocalShard(3, st)
    assert e.value.status_name == "NOT_FOUND"
    with pytest.raises(mm.MmrError):
        ctx.AssembleShards(shape, 4, np.zeros(33, dtype=np.float32), existing_store=st)  # too large
    # Free(keep_in_cache) + CreateStore(allocate_from_cache) reuse the buffers
    before = ctx.stats
    ctx.Free(st, keep_in_cache=True)
    st2 = ctx.CreateStore(shape, name="acts2", allocate_from_cache=True)
    after = ctx.stats
    assert after["cache_hits"] == before["cache_hits"] + 1
    assert after["bytes_allocated"] == before["bytes_allocated"]
    assert st2.unique_id > st.unique_id
    ctx.ClearStoreCache()  # also empties the allocator's pool of freed stores: only st2 is left
    assert ctx.stats["bytes_allocated"] >= 4 * 4096
    held = ctx.stats["bytes_allocated"]
    ctx.Free(st2, keep_in_cache=True)
    assert ctx.stats["bytes_allocated"] == held  # parked, not released
    ctx.ClearStoreCache()
    assert ctx.stats["bytes_allocated"] == held - 4 * 4096
    # a store freed without keep_in_cache goes to the allocator's pool; the next store of its size takes it back
    st3 = ctx.CreateStore(shape, name="acts3")
    allocs = ctx.stats["device_allocations"]
    ctx.Free(st3)
    st4 = ctx.CreateStore(mm.sharded_shape("S32", [(32, 2, 0), (4, 2, 1)], 7, 4), name="other type, same bytes")
    assert ctx.stats["device_allocations"] == allocs and ctx.stats["pool_hits"] >= 1
    assert ctx.ReadShard(st4, 7).tobytes() == bytes(32 * 4)  # zero-filled again
    ctx.Free(st4)


def test_plan_and_binding_caches(ctx):
    """One plan per descriptor pair (keyed like ReshardKey).  The first launch on a set of buffers carries its table
    in the kernel's argument block, the second one builds the device tables for those buffers, later ones find
    them; none of it makes the calling thread wait for the device."""
    s_shape = mm.sharded_shape("BF16", [(64, 1, 0), (256, 4, 1)], 0, 4)
    d_shape = mm.sharded_shape("BF16", [(64, 2, 0), (256, 1, 1)], 4, 2)
    a, b = ctx.CreateStore(s_shape), ctx.CreateStore(d_shape)
    c, d = ctx.CreateStore(s_shape), ctx.CreateStore(d_shape)
    s0 = ctx.stats
    ctx.Reshard(a, b)   # argument block
    ctx.Reshard(a, b)   # builds the device tables
    ctx.Reshard(a, b)   # finds them
    ctx.Reshard(c, d)   # other buffers: argument block again, same plan
    s1 = ctx.stats
    ctx.Sync()
    assert ctx.stats["host_blocking_syncs"] == s1["host_blocking_syncs"] + 1  # a wait the caller asked for is counted
    assert s1["plans_built"] - s0["plans_built"] == 1
    assert s1["plan_cache_hits"] - s0["plan_cache_hits"] == 3
    assert s1["inline_launches"] - s0["inline_launches"] == 2
    assert s1["bindings_built"] - s0["bindings_built"] == 1
    assert s1["binding_cache_hits"] - s0["binding_cache_hits"] == 1
    assert s1["reshard_calls"] - s0["reshard_calls"] == 4
    assert s1["host_blocking_syncs"] == s0["host_blocking_syncs"]
    with pytest.raises(mm.MmrError):
        ctx.Reshard(a, a)
    with pytest.raises(mm.MmrError):
        ctx.Reshard(a, ctx.CreateStore(mm.sharded_shape("BF16", [(64, 2, 0), (128, 1, 1)], 4, 2)))
    for st in (a, b, c, d):
        ctx.Free(st)


def test_long_copy_tables_leave_in_pieces(ctx):
    """A table of several hundred thousand copy chunks is launched as consecutive pieces of 131,072 chunks (long
    launches lose bandwidth, a boundary restores it): the same bytes on the first launch on these buffers (device tables
    are built) and on later ones (they are found)."""
    say("long copy table in pieces")
    ctx.set_plan_options(256, 0)  # 256-byte chunks: a long table over a small array
    try:
        arrays = workloads.config(2, 2)
        gs = [workloads.generate(a) for a in arrays]
        srcs, dsts = make_stores(ctx, arrays, gs)
        chunks = ctx.plan_stats(srcs[0], dsts[0])["n_copy16_chunks"]
        assert chunks >= 3 * 131072
        pieces = -(-chunks // 131072)
        for launch in range(2):
            if launch:
                junk = np.full(dsts[0].shard_bytes, 0xA5, dtype=np.uint8)
                for dev in dsts[0].devices:
                    ctx.AssembleShards(dsts[0].shape, dev, junk, existing_store=dsts[0])
            before = ctx.stats
            ctx.Reshard(srcs[0], dsts[0])
            after = ctx.stats
            assert after["kernel_launches"] - before["kernel_launches"] == pieces
            _compare(arrays, gs, [read_all(ctx, dsts[0])])
        for st in srcs + dsts:
            ctx.Free(st)
    finally:
        ctx.set_plan_options(0, 0)


def test_plan_cache_stays_bounded_when_plans_hold_device_tables():
    """More distinct ragged descriptor pairs than the plan cache holds, each with chunk tables in device memory: the
    least recently used plans go (their tables return to the block pool, where the later plans find theirs), and a
    pair whose plan went is planned again with the same bytes."""
    say("plan cache eviction with device tables")
    with mm.ReshardContext(0) as ctx:
        ctx.set_plan_options(0, 0, 0, B.MMR_PLAN_NO_SPAN)  # ragged boxes as generic chunks: a device table per plan

        def case(rows):
            return [{"name": "evict%d" % rows, "type": "U8", "shape": (rows, 37),
                     "src": {"dims": [(rows, 1, 0), (37, 2, 1)], "dev_start": 0, "dev_count": 2},
                     "dst": {"dims": [(rows, 1, 0), (37, 3, 1)], "dev_start": 4, "dev_count": 3},
                     "seed": rows, "dist": "raw"}]

        first = case(5)
        g_first = [workloads.generate(a) for a in first]
        _compare(first, g_first, gpu_reshard(ctx, first, g_first))
        built0 = ctx.stats["plans_built"]
        pool_hits = None
        for rows in range(6, 6 + 300):
            arrays = case(rows)
            gs = [workloads.generate(a) for a in arrays]
            srcs, dsts = make_stores(ctx, arrays, gs)
            ctx.ReshardBatch(srcs, dsts)
            if rows % 50 == 0:
                _compare(arrays, gs, [read_all(ctx, d) for d in dsts])
            for st in list(srcs) + list(dsts):
                ctx.Free(st)
            if rows == 6 + 269:  # the cache has been full for a while: tables now come from the pool
                pool_hits = ctx.stats["block_pool_hits"]
        st = ctx.stats
        assert st["plans_built"] - built0 == 300
        assert st["plans_cached"] <= 256
        assert st["block_pool_hits"] - pool_hits >= 30  # one chunk table per plan at least
        _compare(first, g_first, gpu_reshard(ctx, first, g_first))  # evicted long ago: planned again
        assert ctx.stats["plans_built"] - built0 == 301


def test_first_reshard_of_a_pair_does_not_wait_for_the_device():
    """A plain Reshard on descriptors never seen before plans, binds and launches without a single blocking
    synchronisation (the reference's Reshard is asynchronous), whichever launch classes the plan has; the plan it
    builds is the same on every run (nothing is timed unless TuneReshard is called)."""
    for index, scale in ((2, 8), (5, 8), (13, 8), (4, 16)):
        arrays = workloads.config(index, scale)
        gs = [workloads.generate(a) for a in arrays]
        seen = []
        for _ in range(2):
            with mm.ReshardContext(0) as ctx:
                srcs, dsts = make_stores(ctx, arrays, gs)
                ctx.Sync()
                before = ctx.stats
                ctx.ReshardBatch(srcs, dsts)
                after = ctx.stats
                assert after["host_blocking_syncs"] == before["host_blocking_syncs"], index
                assert after["plans_built"] == before["plans_built"] + 1
                ctx.Sync()
                _compare(arrays, gs, [read_all(ctx, d) for d in dsts])
                st = ctx.batch_plan_stats(srcs, dsts)
                assert st["orders_timed"] == 0
                seen.append(st)
        assert seen[0] == seen[1]


def test_reshard_is_stream_ordered_after_assemble(ctx):
    """Read-after-reshard through SliceLocalShard observes the reshard of the
    data assembled just before it, with no explicit sync in between."""
    a = workloads.config(1, 4)[0]
    g = workloads.generate(a)
    srcs, dsts = make_stores(ctx, [a], [g])
    ctx.Reshard(srcs[0], dsts[0])
    ctx.SliceLocalShard(dsts[0].devices[0], dsts[0])  # blocks
    _compare([a], [g], [read_all(ctx, dsts[0])])
    ctx.Free(srcs[0]); ctx.Free(dsts[0])


def test_adopted_buffers_are_used_in_place(ctx):
    """Zero-copy import and export: stores living in caller-owned device buffers on either side."""
    a = workloads.config(2, 8)[0]
    g = workloads.generate(a)
    s_shape, d_shape = lib_shape(a["type"], a["src"]), lib_shape(a["type"], a["dst"])
    # "native" buffers: two ordinary stores stand in for memory another runtime owns
    srcs, dsts = make_stores(ctx, [a], [g])
    src_ptrs = [ctx.SliceLocalShard(d, srcs[0]) for d in srcs[0].devices]
    dst_ptrs = [ctx.SliceLocalShard(d, dsts[0]) for d in dsts[0].devices]
    before = ctx.stats["bytes_allocated"]
    adopted_src = ctx.AdoptShards(s_shape, src_ptrs, name="native.in")
    adopted_dst = ctx.AdoptShards(d_shape, dst_ptrs, name="native.out")
    assert ctx.stats["bytes_allocated"] == before  # nothing was allocated or copied
    assert ctx.SliceLocalShard(3, adopted_src) == src_ptrs[3]
    ctx.Reshard(adopted_src, adopted_dst)
    ctx.Sync()
    _compare([a], [g], [read_all(ctx, dsts[0])])  # the result is in the caller's buffers
    with pytest.raises(mm.MmrError):
        ctx.AdoptShards(s_shape, [p + 2 for p in src_ptrs])  # misaligned
    ctx.Free(adopted_src); ctx.Free(adopted_dst)
    # the caller's buffers outlive the adopting stores
    _compare([a], [g], [read_all(ctx, dsts[0])])
    ctx.Free(srcs[0]); ctx.Free(dsts[0])


def test_offload_to_host_and_back(ctx):
    """OffloadDtoH / OffloadHtoD: asynchronous copies between the device cache and a host cache of pinned buffers
    (zuku_execute_context_impl.cc:162-211); the mock's invariant that an offloaded store cannot take part in device
    work (mm_mock_mm_xla.cc:347-356).  Neither call makes the host wait, and the second offload of a descriptor is
    served from the host cache."""
    a = workloads.config(1, 8)[0]
    g = workloads.generate(a)
    srcs, dsts = make_stores(ctx, [a], [g])
    ctx.Sync()
    s0 = ctx.stats
    ctx.OffloadDtoH([srcs[0]])
    s1 = ctx.stats
    assert ctx.IsOffloaded(srcs[0])
    assert s1["host_blocking_syncs"] == s0["host_blocking_syncs"]
    assert s1["host_bytes_allocated"] > s0["host_bytes_allocated"]
    assert s1["bytes_allocated"] == s0["bytes_allocated"]  # the device buffer is parked in the device cache
    with pytest.raises(mm.MmrError) as e:
        ctx.Reshard(srcs[0], dsts[0])
    assert "offloaded" in str(e.value)
    with pytest.raises(mm.MmrError):
        ctx.SliceLocalShard(srcs[0].devices[0], srcs[0])
    host_view = ctx.ReadShard(srcs[0], srcs[0].devices[1])  # reading back still works
    expect = ro.make_shards(raw_global(a, g), oracle_shape(a["type"], a["src"]))
    assert host_view.tobytes() == expect[srcs[0].devices[1]].tobytes()
    s1 = ctx.stats
    ctx.OffloadHtoD([srcs[0]])
    ctx.Reshard(srcs[0], dsts[0])  # offload -> reload -> reshard, all stream-ordered, no host wait
    s2 = ctx.stats
    assert not ctx.IsOffloaded(srcs[0])
    assert s2["host_blocking_syncs"] == s1["host_blocking_syncs"]
    assert s2["cache_hits"] == s1["cache_hits"] + 1 and s2["device_allocations"] == s1["device_allocations"]
    ctx.Sync()
    _compare([a], [g], [read_all(ctx, dsts[0])])
    # a second offload of the same descriptor: the pinned buffer comes from the host cache
    ctx.OffloadDtoH([srcs[0]])
    s3 = ctx.stats
    assert s3["host_cache_hits"] == s2["host_cache_hits"] + 1
    assert s3["host_bytes_allocated"] == s2["host_bytes_allocated"]
    ctx.OffloadHtoD([srcs[0]])
    ctx.Sync()
    assert ctx.ReadShard(srcs[0], srcs[0].devices[1]).tobytes() == host_view.tobytes()
    ctx.Free(srcs[0]); ctx.Free(dsts[0])
    ctx.ClearStoreCache()
    assert ctx.stats["host_bytes_allocated"] == s0["host_bytes_allocated"]


def test_plan_prepared_before_the_first_reshard(ctx):
    s_shape = mm.sharded_shape("F32", [(96, 3, 0), (160, 1, 1)], 0, 3)
    d_shape = mm.sharded_shape("F32", [(96, 1, 0), (160, 5, 1)], 3, 5)
    s0 = ctx.stats
    ctx.PrepareReshard(s_shape, d_shape)
    s1 = ctx.stats
    assert s1["plans_built"] == s0["plans_built"] + 1
    a, b = ctx.CreateStore(s_shape), ctx.CreateStore(d_shape)
    ctx.Reshard(a, b)
    ctx.Sync()
    s2 = ctx.stats
    assert s2["plans_built"] == s1["plans_built"] and s2["plan_cache_hits"] == s1["plan_cache_hits"] + 1
    ctx.Free(a); ctx.Free(b)


def test_event_ordering_entry_points(ctx):
    """The context's stream can wait for and record a caller's HIP event."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so.7")  # the runtime the library already loaded
    ev = C.c_void_p()
    assert hip.hipEventCreate(C.byref(ev)) == 0
    lib = mm.load()
    mm._binding.check(lib.mmr_context_record_event(ctx._h, ev))
    assert hip.hipEventSynchronize(ev) == 0
    mm._binding.check(lib.mmr_context_wait_event(ctx._h, ev))
    ctx.Sync()
    assert hip.hipEventDestroy(ev) == 0


@pytest.mark.parametrize("long_table", [False, True])
def test_reshard_replays_from_a_hip_graph(long_table):
    """Once its plan and pointer table are bound, a reshard is kernel launches only.
    Captured into a HIP graph, it is replayed three times with different data in the
    stores, eager work and synchronisations of the same context in between; every
    replay must match the oracle.  An unbound reshard during capture is refused
    without breaking the capture.  `long_table`: a copy table long enough to leave
    in four launches, which the graph holds as four kernel nodes."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so.7")  # the runtime the library already loaded
    for fn in (hip.hipStreamBeginCapture, hip.hipStreamEndCapture, hip.hipGraphInstantiate, hip.hipGraphLaunch,
               hip.hipGraphExecDestroy, hip.hipGraphDestroy):
        fn.restype = C.c_int
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]

    ctx = mm.ReshardContext(0)  # a context of its own: a broken capture must not leak into other tests
    try:
        if long_table:
            ctx.set_plan_options(256, 0)  # 256-byte chunks: 524,288 of them for a 128 MiB array
            arrays = workloads.config(2, 2)
        else:
            # mixed plan: aligned chunks (configuration 2 scaled), ragged rows (configuration 5 scaled), transposed layout
            arrays = workloads.config(2, 8) + workloads.config(5, 16) + workloads.config(13, 16)
        gs = [workloads.generate(a) for a in arrays]
        srcs, dsts = make_stores(ctx, arrays, gs)
        if long_table:
            assert ctx.batch_plan_stats(srcs, dsts)["n_copy16_launches"] == 4
        other = workloads.config(1, 16)
        other_g = [workloads.generate(a) for a in other]
        other_srcs, other_dsts = make_stores(ctx, other, other_g)

        ctx.BindReshard(srcs, dsts)
        ctx.Sync()
        before = ctx.stats
        stream = ctx.stream
        say("capturing a batched reshard of %d arrays" % len(arrays))
        assert hip.hipStreamBeginCapture(stream, 0) == 0  # hipStreamCaptureModeGlobal
        with pytest.raises(mm.MmrError, match="capturing"):
            ctx.Reshard(other_srcs[0], other_dsts[0])  # not bound: would allocate
        with pytest.raises(mm.MmrError, match="capturing") as refused:
            ctx.ReshardBatchStatic(srcs, dsts)  # copies its tables from host memory on every call
        assert refused.value.status_name == "INVALID_ARGUMENT"
        for call in (lambda: ctx.StartTimer("t"), ctx.OpenWindow, ctx.CloseWindow):
            with pytest.raises(mm.MmrError, match="capturing"):
                call()  # events recorded into a graph could never be read back
        ctx.ReshardBatch(srcs, dsts)
        graph = C.c_void_p()
        assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert graph.value, "capture was invalidated"
        assert ctx.stats["plans_built"] == before["plans_built"] and ctx.stats["bindings_built"] == before["bindings_built"]
        exe = C.c_void_p()
        assert hip.hipGraphInstantiate(C.byref(exe), graph, None, None, 0) == 0

        rng = np.random.Generator(np.random.PCG64(99))
        for replay in range(3):
            if replay:  # new contents in the same source stores, junk in the destinations
                for a, s, d in zip(arrays, srcs, dsts):
                    g = rng.integers(0, 256, size=gs[arrays.index(a)].nbytes, dtype=np.uint8).view(
                        gs[arrays.index(a)].dtype).reshape(gs[arrays.index(a)].shape)
                    gs[arrays.index(a)] = g
                    so = oracle_shape(a["type"], a["src"])
                    shards = ro.make_shards(raw_global(a, g), so, a["src"].get("minor_to_major"))
                    for dev in s.devices:
                        ctx.AssembleShards(lib_shape(a["type"], a["src"]), dev, shards[dev].view(np.uint8).reshape(-1),
                                           existing_store=s)
                    junk = np.full(d.shard_bytes, 0xA5 + replay, dtype=np.uint8)
                    for dev in d.devices:
                        ctx.AssembleShards(lib_shape(a["type"], a["dst"]), dev, junk, existing_store=d)
            say("graph replay %d" % replay)
            assert hip.hipGraphLaunch(exe, stream) == 0
            ctx.Sync()
            _compare(arrays, gs, [read_all(ctx, d) for d in dsts])
            # eager work of the same context between the replays
            ctx.Reshard(other_srcs[0], other_dsts[0])
            ctx.Sync()
            _compare(other, other_g, [read_all(ctx, d) for d in other_dsts])
        assert hip.hipGraphExecDestroy(exe) == 0
        assert hip.hipGraphDestroy(graph) == 0
    finally:
        ctx.close()


def test_rotating_buffer_sets_beyond_the_binding_cache_neither_allocate_nor_wait():
    """80 sets of buffers take turns through one plan whose tables have to live in device memory: more sets than the
    cache of bound tables holds (64), so every launch recycles the least recently used block and uploads its tables
    again - through the pinned staging arena, into a pooled block.  After the warm-up rounds 200 more reshards make
    no device allocation and no host wait; a sample of the results is checked against the oracle."""
    arrays = workloads.config(1, 16)
    gs = [workloads.generate(a) for a in arrays]
    with mm.ReshardContext(0) as ctx:
        ctx.set_plan_options(0, 0, 0, B.MMR_PLAN_NO_INLINE)  # tables never travel in the argument block
        sets = [make_stores(ctx, arrays, gs) for _ in range(80)]
        ctx.Sync()
        say("rotating 80 buffer sets through one plan")
        for srcs, dsts in sets + sets[:20]:
            ctx.ReshardBatch(srcs, dsts)
        warm = ctx.stats
        assert warm["bindings_cached"] == 64
        for i in range(200):
            srcs, dsts = sets[(20 + i) % 80]
            ctx.ReshardBatch(srcs, dsts)
        after = ctx.stats
        assert after["reshard_calls"] - warm["reshard_calls"] == 200
        assert after["bindings_built"] - warm["bindings_built"] == 200  # every one of them a miss
        assert after["device_allocations"] == warm["device_allocations"]
        assert after["host_blocking_syncs"] == warm["host_blocking_syncs"]
        assert after["bindings_cached"] == 64
        ctx.Sync()
        for k in (0, 19, 20, 63, 64, 79):
            _compare(arrays, gs, [read_all(ctx, d) for d in sets[k][1]])


def test_named_timers_windows_and_marks():
    """The per-execution bracket of the reference (OpenWindow, StartTimer, MarkProfile ... StopTimer, CloseWindow,
    MarkProfile; mm_pjrt_executable.cc:362-364, 704-706) through the C ABI: named timers overlap and never make the
    host wait, windows beyond the limit do."""
    arrays = workloads.config(2, 4)
    gs = [workloads.generate(a) for a in arrays]
    with mm.ReshardContext(0) as ctx:
        srcs, dsts = make_stores(ctx, arrays, gs)
        ctx.ReshardBatch(srcs, dsts)  # plan built
        ctx.Sync()
        s0 = ctx.stats
        for step in range(12):
            ctx.OpenWindow()
            ctx.StartTimer("step")
            ctx.StartTimer("inner")
            ctx.MarkProfile("start step")
            ctx.ReshardBatch(srcs, dsts)
            ctx.StopTimer("inner")
            ctx.ReshardBatch(srcs, dsts)
            ctx.StopTimer("step")
            ctx.CloseWindow()
            ctx.MarkProfile("finish step")
        s1 = ctx.stats
        # the only host waits are the window limit's (12 windows of two 2 x 32 MiB reshards, at most 8 in flight)
        assert s1["host_blocking_syncs"] - s0["host_blocking_syncs"] == s1["window_waits"] - s0["window_waits"]
        assert s1["windows_opened"] - s0["windows_opened"] == 12
        assert s1["profile_marks"] - s0["profile_marks"] == 24
        with pytest.warns(UserWarning, match="does not exist"):
            ctx.StopTimer("never started")
        step_ms, n_step = ctx.TimerResult("step", wait=True)
        inner_ms, n_inner = ctx.TimerResult("inner", wait=True)
        assert n_step == 12 and n_inner == 12
        assert 0.0 < inner_ms < step_ms < 100.0
        assert ctx.TimerResult("never started") == (0.0, 0)
        _compare(arrays, gs, [read_all(ctx, d) for d in dsts])


def test_table_order_is_tuned_on_request_and_results_do_not_change():
    """TuneReshard times a few launch orders on the caller's buffers and keeps the fastest; whichever wins, the
    bytes are the oracle's.  Nothing is timed without it, and a fixed order leaves nothing to time."""
    arrays = workloads.config(3, 2)  # 4,096 aligned chunks
    gs = [workloads.generate(a) for a in arrays]
    for order, tuned in ((0, True), (2, False)):
        ctx = mm.ReshardContext(0)
        try:
            ctx.set_plan_options(0, order, 0, 0)
            outs, srcs, dsts = gpu_reshard(ctx, arrays, gs, keep=True)
            _compare(arrays, gs, outs)
            assert ctx.plan_stats(srcs[0], dsts[0])["orders_timed"] == 0
            syncs = ctx.stats["host_blocking_syncs"]
            used = ctx.TuneReshard(srcs[0], dsts[0])
            st = ctx.plan_stats(srcs[0], dsts[0])
            say("order %d: %d orders timed, order used %d / %d KiB" % (order, st["orders_timed"], st["order_used"],
                                                                        st["interleave_kib"]))
            assert (st["orders_timed"] >= 2) == tuned and used == st["order_used"]
            assert (ctx.stats["host_blocking_syncs"] > syncs) == tuned
            # later reshards of the same stores use the kept plan: one launch, same bytes
            before = ctx.stats["kernel_launches"]
            ctx.Reshard(srcs[0], dsts[0])
            ctx.Sync()
            assert ctx.stats["kernel_launches"] - before == 1
            _compare(arrays, gs, [read_all(ctx, d) for d in dsts])
        finally:
            ctx.close()


def test_concurrent_callers(ctx):
    """Several host threads resharding at once: four on one shared context (calls serialise on the context's
    lock, work on its one stream) and two with a context each (two streams on the GPU at the same time).
    ctypes drops the GIL during the calls, so they really overlap."""
    import threading

    def job(context, index, errors):
        try:
            arrays = workloads.config((1, 5, 13, 3)[index % 4], 8)
            gs = [workloads.generate(a) for a in arrays]
            for _ in range(3):
                outs = gpu_reshard(context, arrays, gs)
                _compare(arrays, gs, outs)
        except BaseException as e:  # noqa: BLE001 - reported by the main thread
            errors.append((index, repr(e)))

    errors = []
    own = [mm.ReshardContext(0), mm.ReshardContext(0)]
    try:
        threads = [threading.Thread(target=job, args=(ctx, i, errors)) for i in range(4)]
        threads += [threading.Thread(target=job, args=(own[i], 4 + i, errors)) for i in range(2)]
        say("six threads, three contexts")
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=100)
            assert not t.is_alive(), "a resharding thread did not finish"
        assert not errors, errors
    finally:
        for c in own:
            c.close()


def test_device_resident_shards_assemble_through_the_copy_kernel(ctx):
    """AssembleShards of a large device-resident shard (the GPU branch of AssembleShardsImpl,
    zuku_execute_context_impl.cc:405-415) runs the library's flat copy kernel; sizes that are not a multiple of 16
    finish through the runtime.  Bytes must arrive unchanged, bytes beyond `size` must stay untouched."""
    n = 48 * 1024 * 1024 + 16  # bytes per shard
    shape = mm.sharded_shape("U8", [(2 * n, 2, 0)], 0, 2)
    rng = np.random.Generator(np.random.PCG64(5))
    data = rng.integers(0, 256, size=n, dtype=np.uint8)
    src = ctx.CreateStore(shape, name="assemble.src")
    ctx.AssembleShards(shape, 0, data, existing_store=src)
    ptr = ctx.SliceLocalShard(0, src)
    dst = ctx.CreateStore(shape, name="assemble.dst")
    for size in (n, n - 5, (1 << 20) + 16, 4096):
        ctx.AssembleShards(shape, 1, np.full(n, 0x77, dtype=np.uint8), existing_store=dst)
        before = ctx.stats["kernel_launches"]
        ctx.AssembleShards(shape, 1, ptr, existing_store=dst, size=size)
        ctx.Sync()
        assert ctx.stats["kernel_launches"] - before == (1 if size >= (1 << 20) else 0)
        got = ctx.ReadShard(dst, 1)
        assert got[:size].tobytes() == data[:size].tobytes(), size
        assert (got[size:] == 0x77).all(), size
    # a caller that does not say where the pointer lives (the C++ mirror): the runtime is asked, device memory still
    # takes the kernel, host memory the runtime's copy
    before = ctx.stats["kernel_launches"]
    ctx.AssembleShards(shape, 1, ptr, existing_store=dst, size=n, where=2)
    ctx.AssembleShards(shape, 0, data.ctypes.data, existing_store=dst, size=n, where=2)
    ctx.Sync()
    assert ctx.stats["kernel_launches"] - before == 1
    assert ctx.ReadShard(dst, 1).tobytes() == data.tobytes() and ctx.ReadShard(dst, 0).tobytes() == data.tobytes()
    # rate of the device-to-device assemble
    reps = 20
    ctx.Sync()
    ctx.StartTimer()
    for _ in range(reps):
        ctx.AssembleShards(shape, 1, ptr, existing_store=dst, size=n)
    ms = ctx.StopTimer() / reps
    say("device-to-device AssembleShards of %d MiB: %.1f us, %.0f GB/s (read + write)" % (n >> 20, ms * 1e3, 2 * n / ms / 1e6))
    for s in (src, dst):
        ctx.Free(s)


def test_offsets_beyond_four_gigabytes(ctx):
    """A 5 GiB shard buffer: chunk offsets, row strides and the flat copy's vector index need 64 bits.  One device
    holding [rows, 4096] bytes -> two devices, rows split, the second stored column-major is left out on purpose
    (plain copies only); bit-exact against NumPy slices of the same buffer."""
    rows, cols = 5 * (1 << 30) // 4096 + 3, 4096
    shape_src = mm.sharded_shape("U8", [(rows, 1, 0), (cols, 1, 1)], 0, 1)
    shape_dst = mm.sharded_shape("U8", [(rows, 2, 0), (cols, 1, 1)], 1, 2)
    rng = np.random.Generator(np.random.PCG64(4))
    block = rng.integers(0, 256, size=(1 << 26), dtype=np.uint8)
    data = np.empty(rows * cols, dtype=np.uint8)
    for off in range(0, data.size, block.size):  # cheap, but different in every 64 MiB block
        n = min(block.size, data.size - off)
        np.add(block[:n], np.uint8((off >> 26) * 37 & 0xFF), out=data[off:off + n])
    say("5 GiB shard: assembling")
    src = ctx.CreateStore(shape_src, name="big.src")
    ctx.AssembleShards(shape_src, 0, data, existing_store=src)
    dst = ctx.CreateStore(shape_dst, name="big.dst")
    say("5 GiB shard: resharding")
    ctx.Reshard(src, dst)
    ctx.Sync()
    half = (rows + 1) // 2
    for k, dev in enumerate(dst.devices):
        got = ctx.ReadShard(dst, dev)
        lo, hi = k * half, min((k + 1) * half, rows)
        assert got[:(hi - lo) * cols].tobytes() == data[lo * cols:hi * cols].tobytes(), dev
        assert not got[(hi - lo) * cols:].any()  # the pad row of the short tile is zero
    # device-to-device assemble of the whole 5 GiB shard through the flat copy kernel
    copy = ctx.CreateStore(shape_src, name="big.copy")
    ctx.AssembleShards(shape_src, 0, ctx.SliceLocalShard(0, src), existing_store=copy, size=rows * cols)
    ctx.Sync()
    assert ctx.ReadShard(copy, 0).tobytes() == data.tobytes()
    for s in (src, dst, copy):
        ctx.Free(s)
