"""The planner (libmmreshard.so, host side) against the oracle, without a GPU:
its chunk tables are interpreted in NumPy and must reproduce the oracle's
destination buffers bit for bit."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

import multimesh_jax_amd as mm
from multimesh_jax_amd import workloads

from helpers import lib_shape, oracle_outputs, run_plan_on_host, test_config


def _check(arrays, globals_, **kw):
    plan, outs = run_plan_on_host(arrays, globals_, **kw)
    for a, g, out in zip(arrays, globals_, outs):
        expect = oracle_outputs(a, g)
        assert sorted(out) == sorted(expect)
        for dev in expect:
            assert out[dev].tobytes() == expect[dev].tobytes(), (a["name"], dev)
    return plan


@pytest.mark.parametrize("index,scale", [(1, 32), (2, 32), (3, 16), (5, 64), (6, 64)])
@pytest.mark.parametrize("chunk_bytes", [0, 4096])
def test_benchmark_configs_scaled(index, scale, chunk_bytes):
    arrays = workloads.config(index, scale)
    gs = [workloads.generate(a) for a in arrays]
    plan = _check(arrays, gs, chunk_bytes=chunk_bytes)
    st_ = plan.stats
    moved = sum(int(np.prod(a["shape"])) * workloads.ITEMSIZE[a["type"]] for a in arrays)
    assert st_["bytes_moved"] == moved
    assert 2 * st_["bytes_moved"] == workloads.algorithmic_bytes(arrays)


def test_config4_batched_plan_scaled():
    arrays = workloads.config(4, 64)
    assert len(arrays) == 195
    gs = [workloads.generate(a) for a in arrays]
    plan = _check(arrays, gs, chunk_bytes=8192)
    assert plan.stats["n_arrays"] == 195


def test_config4_full_size_plan_is_one_aligned_launch():
    arrays = workloads.config(4)
    plan = mm.Plan([lib_shape(a["type"], a["src"]) for a in arrays],
                   [lib_shape(a["type"], a["dst"]) for a in arrays])
    s = plan.stats
    assert s["n_arrays"] == 195
    assert s["n_transpose_chunks"] == 0 and s["n_copy_generic_chunks"] == 0 and s["n_fill_chunks"] == 0
    assert 2 * s["bytes_moved"] == 10_713_055_232 == workloads.algorithmic_bytes(arrays)
    assert s["n_slots"] == 195 * 12
    # the table is long enough to leave in pieces of 131,072 chunks
    assert s["n_copy16_chunks"] == 654_984 and s["n_copy16_launches"] == 5


def test_only_tables_of_three_pieces_and_more_leave_in_pieces():
    """Launch pieces of 131,072 chunks (measured: shorter tables lose by being cut); a contiguous tile costs two piece
    records however long it is."""
    for chunks, launches in ((65_536, 1), (262_144, 1), (393_214, 1), (393_216, 3), (400_000, 4), (655_360, 5)):
        n = chunks * 8192
        plan = mm.Plan(mm.sharded_shape("U8", [(n, 1, 0)], 0, 1), mm.sharded_shape("U8", [(n, 2, 0)], 1, 2))
        s = plan.stats
        assert s["n_copy16_chunks"] == chunks and s["n_copy16_launches"] == launches, (chunks, s)
        assert s["n_pieces"] <= 4 and s["table_bytes"] < 64 * 1024, s
    # each XCD a contiguous eighth of the table: one launch whatever the length
    plan = mm.Plan(mm.sharded_shape("U8", [(655_360 * 8192, 1, 0)], 0, 1),
                   mm.sharded_shape("U8", [(655_360 * 8192, 2, 0)], 1, 2), xcd_mode=2)
    assert plan.stats["n_copy16_launches"] == 1


def test_config2_full_size_plan_shape():
    """Full-size headline plan: 32 boxes of [8,1024,1024] bf16, 2 KiB runs, all 16-byte aligned."""
    a = workloads.config(2)[0]
    plan = mm.Plan(lib_shape(a["type"], a["src"]), lib_shape(a["type"], a["dst"]))
    s = plan.stats
    assert s["n_boxes"] == 32 and s["bytes_moved"] == 512 << 20
    assert s["n_copy_generic_chunks"] == 0 and s["n_transpose_chunks"] == 0 and s["n_fill_chunks"] == 0
    ch = plan.copy_chunks(0)
    assert (ch["w"] == 2048).all()
    assert int((ch["w"].astype(np.int64) * ch["n1"] * ch["n2"]).sum()) == 512 << 20
    # destination-address order: consecutive chunks write neighbouring 2 KiB columns of the same rows
    assert (np.diff(ch["dst_slot"].astype(np.int64)) >= 0).all()


def test_config3_keeps_the_minor_dim():
    a = workloads.config(3)[0]
    plan = mm.Plan(lib_shape(a["type"], a["src"]), lib_shape(a["type"], a["dst"]))
    s = plan.stats
    assert s["n_transpose_chunks"] == 0 and s["n_copy_generic_chunks"] == 0
    assert s["n_boxes"] == 32 and s["bytes_moved"] == 64 << 20
    assert (plan.copy_chunks(0)["w"] == 256).all()


def test_minor_changing_layout_uses_transpose_tiles():
    a = {"name": "t", "type": "F32", "shape": (70, 130),
         "src": {"dims": [(70, 2, 0), (130, 1, 1)], "dev_start": 0, "dev_count": 2},
         "dst": {"dims": [(70, 1, 0), (130, 3, 1)], "dev_start": 2, "dev_count": 3, "minor_to_major": [0, 1]},
         "seed": 3, "dist": "uniform"}
    g = workloads.generate(a)
    plan = _check([a], [g])
    assert plan.stats["n_transpose_chunks"] > 0


@pytest.mark.parametrize("type_,item", [("U8", 1), ("BF16", 2), ("F32", 4), ("F64", 8), ("C128", 16)])
def test_transpose_every_itemsize(type_, item):
    rng = np.random.Generator(np.random.PCG64(7))
    shape = (3, 67, 45)
    a = {"name": "t", "type": type_, "shape": shape,
         "src": {"dims": [(3, 1, 0), (67, 2, 1), (45, 1, 2)], "dev_start": 0, "dev_count": 2},
         "dst": {"dims": [(3, 1, 0), (67, 1, 1), (45, 2, 2)], "dev_start": 2, "dev_count": 2, "minor_to_major": [1, 2, 0]},
         "seed": 0, "dist": "raw"}
    from oracle import reshard_oracle as ro
    g = rng.integers(0, 256, size=int(np.prod(shape)) * item, dtype=np.uint8).view(ro.raw_dtype(type_)).reshape(shape)
    _check([a], [g])


def test_empty_and_degenerate_arrays():
    rng = np.random.Generator(np.random.PCG64(1))
    cases = [
        ((0, 4), [(0, 2, 0), (4, 1, 1)], 2, [(0, 1, 0), (4, 2, 1)], 2),
        ((1,), [(1, 1, 0)], 1, [(1, 1, 0), (1, 4, 1)], 4),
        ((), [(1, 4, 0)], 4, [(1, 8, 0)], 8),
        ((5,), [(5, 8, 0)], 8, [(5, 2, 0)], 2),
    ]
    for shape, sd, sc, dd, dc in cases:
        a = {"name": "e", "type": "S32", "shape": shape,
             "src": {"dims": sd, "dev_start": 0, "dev_count": sc},
             "dst": {"dims": dd, "dev_start": 10, "dev_count": dc}, "seed": 0, "dist": "raw"}
        n = int(np.prod(shape)) if shape else 1
        g = rng.integers(0, 2**32, size=n, dtype=np.uint32).reshape(shape)
        _check([a], [g])


@st.composite
def random_arrays(draw):
    rank = draw(st.integers(1, 4))
    shape = [draw(st.integers(1, 9)) for _ in range(rank)]
    type_ = draw(st.sampled_from(["U8", "BF16", "F32", "F64", "C128"]))

    def side(start):
        shard = [draw(st.integers(1, 4)) for _ in range(rank)]
        repl = draw(st.sampled_from([1, 1, 2, 3]))
        if repl == 1 and shape[-1] == 1:
            shard[-1] = 1
        entries = shard + ([repl] if repl > 1 else [])
        perm = draw(st.permutations(list(range(len(entries)))))
        dims = [(shape[i], shard[i], perm[i]) for i in range(rank)]
        if repl > 1:
            dims.append((1, repl, perm[rank]))
        d = {"dims": dims, "dev_start": start, "dev_count": int(np.prod(entries))}
        m2m = draw(st.one_of(st.none(), st.permutations(list(range(rank)))))
        if m2m is not None:
            d["minor_to_major"] = list(m2m)
        return d

    return {"name": "r", "type": type_, "shape": tuple(shape), "src": side(draw(st.integers(0, 3))),
            "dst": side(draw(st.integers(0, 50))), "seed": 0, "dist": "raw"}


@given(random_arrays(), st.sampled_from([0, 1024]), st.sampled_from([0, 1, 2, 3]))
@settings(max_examples=150, deadline=None)
def test_random_pairs(a, chunk_bytes, order):
    from oracle import reshard_oracle as ro
    item = ro.ITEMSIZE[a["type"]]
    rng = np.random.Generator(np.random.PCG64(3))
    g = rng.integers(0, 256, size=int(np.prod(a["shape"])) * item, dtype=np.uint8).view(
        ro.raw_dtype(a["type"])).reshape(a["shape"])
    _check([a], [g], chunk_bytes=chunk_bytes, order=order)


def test_plan_rejects_mismatched_pairs():
    s = mm.sharded_shape("F32", [(8, 4, 0), (8, 1, 1)], 0, 4)
    with pytest.raises(mm.MmrError) as e:
        mm.Plan(s, mm.sharded_shape("F32", [(8, 2, 0), (9, 2, 1)], 4, 4))
    assert e.value.status_name == "INVALID_ARGUMENT"
    with pytest.raises(mm.MmrError):
        mm.Plan(s, mm.sharded_shape("S32", [(8, 2, 0), (8, 2, 1)], 4, 4))
    with pytest.raises(mm.MmrError):
        mm.Plan(s, mm.sharded_shape("F32", [(8, 2, 0), (8, 2, 1)], 4, 5))  # product of shardings != devices
    with pytest.raises(mm.MmrError):
        mm.Plan(s, mm.sharded_shape("F32", [(8, 2, 0), (8, 2, 0)], 4, 4))  # permutation repeats
    with pytest.raises(mm.MmrError) as e:
        mm.sharded_shape("F32", [(8, 2, 0)], 0, 2).dtype  # fine
        bad = mm.sharded_shape("F32", [(8, 2, 0)], 0, 2)
        bad.dtype = 55
        mm.Plan(bad, bad)
    assert e.value.status_name == "UNSUPPORTED"


def test_generic_chunks_are_bounded_in_lane_work_as_well_as_in_bytes():
    """The generic kernel (ragged boxes the span kernel does not take; forced here with MMR_PLAN_NO_SPAN) spends
    one lane per (row, 16-byte slot) pair: the one-byte pad column of configuration 5's last tile must not come out
    as chunks of thousands of rows (each would keep one workgroup busy long after the rest of the launch)."""
    from multimesh_jax_amd import _binding as B
    arrays = workloads.config(5)
    plan = mm.Plan([lib_shape(a["type"], a["src"]) for a in arrays],
                   [lib_shape(a["type"], a["dst"]) for a in arrays], flags=B.MMR_PLAN_NO_SPAN)
    g = plan.copy_chunks(1)
    assert len(g) > 0 and len(plan.copy_chunks(0)) == 0 and plan.stats["n_span_chunks"] == 0
    slots = (g["w"].astype(np.int64) + 15) // 16 + 1
    pairs = g["n1"].astype(np.int64) * g["n2"] * slots
    assert pairs.max() <= 768
    fills = g[g["src_slot"] == 0xFFFFFFFF]
    assert plan.stats["n_fill_chunks"] == len(fills)
    fp8_pad = fills[fills["w"] == 1]  # 11008 rows x 1 byte after the 819 valid bytes of the last tile
    assert int(fp8_pad["n1"].sum()) == 11008 and fp8_pad["n1"].max() <= 384
    # whole rows of 820 bytes: 6 to a chunk at this plan's size (45 MB -> ~5.4 KiB chunks), 8 (7 KiB) on a plan 8 times larger
    assert int(g[g["w"] == 820]["n1"].max()) == 6
    big = test_config(10)
    plan_big = mm.Plan([lib_shape(a["type"], a["src"]) for a in big], [lib_shape(a["type"], a["dst"]) for a in big],
                       flags=B.MMR_PLAN_NO_SPAN)
    gb = plan_big.copy_chunks(1)
    assert int(gb[gb["w"] == 820]["n1"].max()) == 8


def test_ragged_rows_become_destination_spans():
    """Configuration 5 (4099-byte fp8 rows and 4097 x 4-byte rows, 3-way -> 5-way): every destination tile is one
    dense band of rows whose pieces tile the row, cut into 128-byte aligned spans; the five tiles of an array are
    interleaved in one group; the whole plan is two group records."""
    arrays = workloads.config(5)
    plan = mm.Plan([lib_shape(a["type"], a["src"]) for a in arrays],
                   [lib_shape(a["type"], a["dst"]) for a in arrays])
    s = plan.stats
    assert s["n_copy16_chunks"] == 0 and s["n_copy_generic_chunks"] == 0 and s["n_transpose_chunks"] == 0
    assert s["n_groups"] == 2  # one per array, five interleaved tiles each
    # destination shards of 8 x 3280 and 11008 x 820 bytes, five each, in spans of 4 KiB
    assert s["n_span_chunks"] == 5 * (-(-8 * 3280 // 4096)) + 5 * (-(-11008 * 820 // 4096))
    assert s["table_bytes"] < 4096
    pieces = plan.copy_chunks(2)
    fp8 = pieces[pieces["d1"] == 820]
    assert sorted(fp8["w"].tolist()) == sorted([820, 547, 273, 820, 274, 546, 819, 1])
    assert (fp8["n1"].astype(np.int64) * fp8["n2"] == 11008).all()
    assert int(fp8[fp8["src_slot"] == 0xFFFFFFFF]["w"].sum()) == 1  # the pad column of the last tile
    assert s["bytes_moved"] == 8 * 4097 * 4 + 11008 * 4099 and s["bytes_filled"] == 8 * 3 * 4 + 11008


def test_plan_tables_are_a_handful_of_records():
    """The plan of the headline configuration: 4 groups (one per destination tile) of 8 pieces each; a 195-array
    batch stays in the hundreds of KiB."""
    a = workloads.config(2)[0]
    plan = mm.Plan(lib_shape(a["type"], a["src"]), lib_shape(a["type"], a["dst"]))
    s = plan.stats
    assert s["n_groups"] == 4 and s["n_pieces"] == 32 and s["n_copy16_chunks"] == 65536
    assert s["table_bytes"] < 8192
    arrays = workloads.config(4)
    plan4 = mm.Plan([lib_shape(a["type"], a["src"]) for a in arrays], [lib_shape(a["type"], a["dst"]) for a in arrays])
    assert plan4.stats["table_bytes"] < 1 << 20
