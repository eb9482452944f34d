"""The kernels' own per-chunk code (csrc/chunk_ops.h), compiled for the host with a
bounds- and alignment-checking memory policy, against the oracle.  Catches index
errors and out-of-bounds accesses on a CPU, before a kernel runs on the GPU."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from multimesh_jax_amd import workloads

from helpers import oracle_outputs, run_plan_on_host, test_config
from test_planner_cpu import random_arrays


def _check(arrays, gs, **kw):
    plan, outs = run_plan_on_host(arrays, gs, engine="emulation", **kw)
    for a, g, out in zip(arrays, gs, outs):
        expect = oracle_outputs(a, g)
        for dev in expect:
            assert out[dev].tobytes() == expect[dev].tobytes(), (a["name"], dev)
    return plan


@pytest.mark.parametrize("index,scale", [(1, 16), (2, 16), (3, 8), (5, 32), (6, 32), (7, 32), (8, 32), (11, 64)])
@pytest.mark.parametrize("shape", [0, 1, 2, 3])
def test_configs_through_the_kernel_code(index, scale, shape):
    arrays = test_config(index, scale)
    gs = [workloads.generate(a) for a in arrays]
    _check(arrays, gs, shape=shape)


def test_span_kernel_build_options_through_the_kernel_code():
    """The span kernel's two optional variations (MMR_SPAN_ALIGNED_LOADS, MMR_SPAN_KEEP_EDGES: not in the shipped
    build, they do not pay) keep passing the same checks on the ragged configurations."""
    import helpers
    helpers.EMULATION_VARIANT = "_span_options"
    try:
        for index, scale in ((5, 32), (6, 32), (7, 32), (8, 32), (11, 64)):
            arrays = test_config(index, scale)
            gs = [workloads.generate(a) for a in arrays]
            for shape in (0, 1):
                _check(arrays, gs, shape=shape)
    finally:
        helpers.EMULATION_VARIANT = ""


@pytest.mark.parametrize("xcd_mode", [1, 2, 16, 64, 1024])
def test_every_workgroup_mapping_visits_each_chunk_once(xcd_mode):
    for index, scale in ((2, 32), (5, 64), (4, 64)):
        arrays = workloads.config(index, scale)
        gs = [workloads.generate(a) for a in arrays]
        _check(arrays, gs, xcd_mode=xcd_mode)


@pytest.mark.parametrize("chunk_bytes", [256, 1024, 8192, 65536, 1 << 20])
def test_chunk_sizes_wide_and_narrow_rows(chunk_bytes):
    # rows of 2 KiB (narrower than a 256-thread workgroup's 4 KiB pass), 8 KiB and 32 KiB (wider)
    for index, scale in ((2, 16), (1, 4), (4, 64)):
        arrays = workloads.config(index, scale)[:12]
        gs = [workloads.generate(a) for a in arrays]
        _check(arrays, gs, chunk_bytes=chunk_bytes)


@pytest.mark.parametrize("chunk_bytes", [256, 8192])
def test_long_contiguous_runs_are_folded_into_rows(chunk_bytes):
    """Tiles that are contiguous on both sides (the same dim sharded a different number of ways, whole rows regrouped)
    are copied as rows of one chunk under one piece record each - the table does not grow with the tile - plus a
    box for what is left behind the last whole row; a run under other row dims is folded the same way."""
    tile = 20 * chunk_bytes + 48  # bytes per destination tile: 20 whole rows and a tail
    cases = [
        [{"name": "flat", "type": "U8", "shape": (3 * tile,),
          "src": {"dims": [(3 * tile, 1, 0)], "dev_start": 0, "dev_count": 1},
          "dst": {"dims": [(3 * tile, 3, 0)], "dev_start": 1, "dev_count": 3}, "seed": 1, "dist": "raw"}],
        [{"name": "rows", "type": "F32", "shape": (96, tile // 16),
          "src": {"dims": [(96, 2, 0), (tile // 16, 1, 1)], "dev_start": 0, "dev_count": 2},
          "dst": {"dims": [(96, 3, 0), (tile // 16, 1, 1)], "dev_start": 2, "dev_count": 3}, "seed": 2, "dist": "raw"}],
        # long rows that stay strided on the source side: a run of 40 chunks under a row dim
        [{"name": "strided", "type": "U8", "shape": (6, 80 * chunk_bytes),
          "src": {"dims": [(6, 1, 0), (80 * chunk_bytes, 2, 1)], "dev_start": 0, "dev_count": 2},
          "dst": {"dims": [(6, 3, 0), (80 * chunk_bytes, 1, 1)], "dev_start": 2, "dev_count": 3}, "seed": 3, "dist": "raw"}],
    ]
    for arrays in cases:
        gs = [workloads.generate(a) for a in arrays]
        plan = _check(arrays, gs, chunk_bytes=chunk_bytes)
        st = plan.stats
        assert st["n_copy16_chunks"] >= 60 and st["n_pieces"] <= 12, (arrays[0]["name"], st)


def test_traffic_of_the_headline_plan_is_exactly_algorithmic():
    from helpers import emulate_plan, lib_shape
    import multimesh_jax_amd as mm
    a = workloads.config(2, 8)[0]
    plan = mm.Plan(lib_shape(a["type"], a["src"]), lib_shape(a["type"], a["dst"]))
    n = plan.stats["bytes_moved"]
    bufs = [np.zeros(n // 8, dtype=np.uint8) for _ in range(8)] + [np.zeros(n // 4, dtype=np.uint8) for _ in range(4)]
    loaded, stored = emulate_plan(plan, bufs)
    assert loaded == n and stored == n


@given(random_arrays(), st.sampled_from([0, 256, 2048]), st.sampled_from([0, 1, 2, 3]), st.sampled_from([0, 1, 16]))
@settings(max_examples=200, deadline=None)
def test_random_pairs_through_the_kernel_code(a, chunk_bytes, shape, xcd_mode):
    from oracle import reshard_oracle as ro
    item = ro.ITEMSIZE[a["type"]]
    rng = np.random.Generator(np.random.PCG64(17))
    g = rng.integers(0, 256, size=int(np.prod(a["shape"])) * item, dtype=np.uint8).view(
        ro.raw_dtype(a["type"])).reshape(a["shape"])
    _check([a], [g], chunk_bytes=chunk_bytes, shape=shape, xcd_mode=xcd_mode)


@st.composite
def ragged_2d(draw):
    """Wide ragged rows (hundreds of bytes), the shape the generic kernel is for."""
    rows = draw(st.integers(1, 40))
    cols = draw(st.integers(1, 1500))
    type_ = draw(st.sampled_from(["U8", "BF16", "S32"]))
    st_src, st_dst = draw(st.integers(1, 4)), draw(st.integers(1, 6))
    rs, rd = draw(st.integers(1, 3)), draw(st.integers(1, 3))
    return {"name": "rag", "type": type_, "shape": (rows, cols),
            "src": {"dims": [(rows, rs, 0), (cols, st_src, 1)], "dev_start": 0, "dev_count": rs * st_src},
            "dst": {"dims": [(rows, rd, 1), (cols, st_dst, 0)], "dev_start": 20, "dev_count": rd * st_dst},
            "seed": 0, "dist": "raw"}


@given(ragged_2d(), st.sampled_from([0, 1]))
@settings(max_examples=150, deadline=None)
def test_span_kernel_build_options_ragged_rows(a, shape):
    import helpers
    from oracle import reshard_oracle as ro
    item = ro.ITEMSIZE[a["type"]]
    rng = np.random.Generator(np.random.PCG64(29))
    g = rng.integers(0, 256, size=int(np.prod(a["shape"])) * item, dtype=np.uint8).view(
        ro.raw_dtype(a["type"])).reshape(a["shape"])
    if a["shape"][1] == 1 and (a["src"]["dims"][1][1] > 1 or a["dst"]["dims"][1][1] > 1):
        return  # trailing {1, R} would read as a replication entry
    helpers.EMULATION_VARIANT = "_span_options"
    try:
        _check([a], [g], shape=shape)
    finally:
        helpers.EMULATION_VARIANT = ""


@given(ragged_2d(), st.sampled_from([0, 512, 4096]), st.sampled_from([0, 1, 2, 3]))
@settings(max_examples=150, deadline=None)
def test_ragged_rows_through_the_kernel_code(a, chunk_bytes, shape):
    from oracle import reshard_oracle as ro
    item = ro.ITEMSIZE[a["type"]]
    rng = np.random.Generator(np.random.PCG64(23))
    g = rng.integers(0, 256, size=int(np.prod(a["shape"])) * item, dtype=np.uint8).view(
        ro.raw_dtype(a["type"])).reshape(a["shape"])
    if a["shape"][1] == 1 and (a["src"]["dims"][1][1] > 1 or a["dst"]["dims"][1][1] > 1):
        return  # trailing {1, R} would read as a replication entry
    _check([a], [g], chunk_bytes=chunk_bytes, shape=shape)


@st.composite
def ragged_3d(draw):
    """Long ragged rows under two row dims: the span kernel walks them piece row by piece row, across the boundary
    between the inner and the outer row dim and, with the first dim split on one side only, across tiles."""
    outer, inner = draw(st.integers(1, 5)), draw(st.integers(1, 7))
    cols = draw(st.integers(130, 2600))
    type_ = draw(st.sampled_from(["U8", "BF16"]))
    st_src, st_dst = draw(st.integers(1, 4)), draw(st.integers(1, 5))
    od = draw(st.integers(1, 2))
    return {"name": "rag3", "type": type_, "shape": (outer, inner, cols),
            "src": {"dims": [(outer, 1, 0), (inner, 1, 1), (cols, st_src, 2)], "dev_start": 0, "dev_count": st_src},
            "dst": {"dims": [(outer, od, 1), (inner, 1, 2), (cols, st_dst, 0)], "dev_start": 20,
                    "dev_count": od * st_dst},
            "seed": 0, "dist": "raw"}


@given(ragged_3d(), st.sampled_from([0, 1]))
@settings(max_examples=120, deadline=None)
def test_span_kernel_build_options_long_ragged_rows(a, shape):
    import helpers
    from oracle import reshard_oracle as ro
    item = ro.ITEMSIZE[a["type"]]
    rng = np.random.Generator(np.random.PCG64(31))
    g = rng.integers(0, 256, size=int(np.prod(a["shape"])) * item, dtype=np.uint8).view(
        ro.raw_dtype(a["type"])).reshape(a["shape"])
    helpers.EMULATION_VARIANT = "_span_options"
    try:
        _check([a], [g], shape=shape)
    finally:
        helpers.EMULATION_VARIANT = ""


@given(ragged_3d(), st.sampled_from([0, 512, 4096]), st.sampled_from([0, 1, 2, 3]))
@settings(max_examples=120, deadline=None)
def test_long_ragged_rows_under_two_row_dims(a, chunk_bytes, shape):
    from oracle import reshard_oracle as ro
    item = ro.ITEMSIZE[a["type"]]
    rng = np.random.Generator(np.random.PCG64(29))
    g = rng.integers(0, 256, size=int(np.prod(a["shape"])) * item, dtype=np.uint8).view(
        ro.raw_dtype(a["type"])).reshape(a["shape"])
    _check([a], [g], chunk_bytes=chunk_bytes, shape=shape)


@pytest.mark.parametrize("type_", ["U8", "BF16", "F32", "F64", "C128"])
@pytest.mark.parametrize("shape", [(256, 384), (192, 200), (130, 256)])
def test_transposed_layout_vector_and_element_tiles(type_, shape):
    """Aligned tiles take the 16-byte vector path, ragged edge tiles the general path."""
    from oracle import reshard_oracle as ro
    item = ro.ITEMSIZE[type_]
    a = {"name": "t", "type": type_, "shape": shape,
         "src": {"dims": [(shape[0], 2, 0), (shape[1], 1, 1)], "dev_start": 0, "dev_count": 2},
         "dst": {"dims": [(shape[0], 1, 0), (shape[1], 2, 1)], "dev_start": 2, "dev_count": 2, "minor_to_major": [0, 1]},
         "seed": 0, "dist": "raw"}
    rng = np.random.Generator(np.random.PCG64(31))
    g = rng.integers(0, 256, size=int(np.prod(shape)) * item, dtype=np.uint8).view(ro.raw_dtype(type_)).reshape(shape)
    plan = _check([a], [g])
    assert plan.stats["n_transpose_chunks"] > 0


@pytest.mark.parametrize("type_", ["U8", "BF16", "F32", "F64", "C128"])
@pytest.mark.parametrize("shape,src_tiles,dst_tiles", [
    ((250, 381), (2, 1), (1, 3)),   # odd row lengths: no stride is a multiple of 16 -> general path everywhere;
                                    # vectors cut off by the tile edge slide inwards on both sides
    ((135, 203), (1, 1), (1, 1)),   # one full sub-tile, one ragged, one thinner than a vector (element path)
    ((67, 131), (1, 1), (1, 1)),    # 3 columns past the first sub-tile
    ((129, 257), (1, 2), (2, 1)),   # a single row / column beyond full tiles
    ((20, 300), (1, 1), (1, 1)),    # short in y (packed source rows run past the edge)
    ((300, 20), (1, 1), (1, 1)),    # short in x
    ((3, 500), (1, 1), (1, 1)),     # thinner than one vector of any type but C128
])
def test_transposed_layout_ragged_and_misaligned_tiles(type_, shape, src_tiles, dst_tiles):
    """Tiles that are not 16-byte aligned or do not hold whole vectors: unaligned 16-byte accesses with vectors
    slid inwards at the edges, element by element only where a sub-tile is thinner than one vector."""
    from oracle import reshard_oracle as ro
    item = ro.ITEMSIZE[type_]
    ns = src_tiles[0] * src_tiles[1]
    a = {"name": "t", "type": type_, "shape": shape,
         "src": {"dims": [(shape[0], src_tiles[0], 0), (shape[1], src_tiles[1], 1)], "dev_start": 0, "dev_count": ns},
         "dst": {"dims": [(shape[0], dst_tiles[0], 0), (shape[1], dst_tiles[1], 1)], "dev_start": ns,
                 "dev_count": dst_tiles[0] * dst_tiles[1], "minor_to_major": [0, 1]},
         "seed": 0, "dist": "raw"}
    rng = np.random.Generator(np.random.PCG64(37))
    g = rng.integers(0, 256, size=int(np.prod(shape)) * item, dtype=np.uint8).view(ro.raw_dtype(type_)).reshape(shape)
    plan = _check([a], [g])
    assert plan.stats["n_transpose_chunks"] > 0


@pytest.mark.parametrize("type_", ["U8", "BF16", "F32", "F64"])
@pytest.mark.parametrize("shape,m2m", [
    ((40, 700, 3), [1, 0, 2]),    # 3 channels leave the minor position: x extent 3, tiles thousands of elements long in y
    ((50, 6, 1030), [1, 2, 0]),   # a dim of 6 becomes the minor one: y extent 6
    ((7, 1, 33000), [1, 0, 2]),
])
def test_transposed_layout_thin_tiles(type_, shape, m2m):
    """A box thinner than one 16-byte vector one way: the whole chunk (tiles as long as the workgroup's LDS
    allows) moves in two phases around one workgroup barrier."""
    from oracle import reshard_oracle as ro
    import multimesh_jax_amd as mm
    from helpers import lib_shape
    item = ro.ITEMSIZE[type_]
    a = {"name": "t", "type": type_, "shape": shape,
         "src": {"dims": [(n, 1, i) for i, n in enumerate(shape)], "dev_start": 0, "dev_count": 1},
         "dst": {"dims": [(n, 1, i) for i, n in enumerate(shape)], "dev_start": 1, "dev_count": 1, "minor_to_major": m2m},
         "seed": 0, "dist": "raw"}
    rng = np.random.Generator(np.random.PCG64(43))
    g = rng.integers(0, 256, size=int(np.prod(shape)) * item, dtype=np.uint8).view(ro.raw_dtype(type_)).reshape(shape)
    plan = _check([a], [g])
    t = plan.transpose_chunks()
    if shape[1] != 1:
        assert len(t) > 0
        vec = 16 // item
        thin = (t["nx"] < vec) | (t["ny"] < vec)
        if thin.any():  # (F64 has 2-element vectors: 3 channels are not thin there)
            assert (t["nb"].astype(np.int64) * t["nx"] * t["ny"] * item)[thin].max() <= 32 * 1024


def test_transposed_benchmark_workloads_scaled():
    for index in (13, 14, 15):
        arrays = workloads.config(index, 16)
        gs = [workloads.generate(a) for a in arrays]
        _check(arrays, gs)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_sanitizer_sweep_of_planner_and_kernel_code(seed):
    """tests/cpp/sanitize_sweep: planner, descriptor geometry and the kernels' per-chunk code built with the address
    and undefined-behaviour sanitizers (host only), 1,500 random sharding pairs checked element by element."""
    import os
    import subprocess
    here = os.path.dirname(os.path.abspath(__file__))
    exe = os.path.join(here, "cpp", "sanitize_sweep")
    if not os.path.exists(exe):
        subprocess.check_call(["bash", os.path.join(here, "cpp", "build.sh")])
    p = subprocess.run([exe, "1500", str(seed)], capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "cases OK" in p.stdout
