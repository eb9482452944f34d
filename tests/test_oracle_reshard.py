"""The reshard oracles (NumPy and C) against what the mathematics fixes:
single-element brute force, round trips, and each other."""
import itertools

import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from oracle import reshard_cpu, reshard_oracle as ro
from oracle.sharding_oracle import ShardedShape, ShardingDim


def SS(t, dims, start, count):
    return ShardedShape(t, tuple(ShardingDim(*d) for d in dims), start, count)


def brute_force_dst(global_array, ss, device, minor_to_major=None):
    """Destination buffer of one device, element by element: every element's
    owner tile comes from an integer division, nothing is sliced."""
    rank = ro.tensor_rank(ss)
    ext = [-(-ss.dims[i].size // ss.dims[i].sharding) for i in range(rank)]
    m2m = list(minor_to_major) if minor_to_major is not None else list(range(rank - 1, -1, -1))
    stride = [0] * rank
    acc = 1
    for d in m2m:
        stride[d] = acc
        acc *= ext[d]
    buf = np.zeros(acc, dtype=global_array.dtype)
    # device -> tile coordinate by peeling the id in significance order
    order = sorted(range(len(ss.dims)), key=lambda i: -ss.dims[i].permutation)
    rel = device - ss.dev_start
    coord = [0] * len(ss.dims)
    for i in order:
        coord[i] = rel % ss.dims[i].sharding
        rel //= ss.dims[i].sharding
    for idx in itertools.product(*[range(s) for s in global_array.shape]):
        if all(idx[i] // ext[i] == coord[i] for i in range(rank)):
            off = sum((idx[i] % ext[i]) * stride[i] for i in range(rank))
            buf[off] = global_array[idx]
    return buf


def brute_force_src_lookup(shards, ss, idx, minor_to_major=None):
    """Value of global element idx, read from the replica-0 source shard."""
    rank = ro.tensor_rank(ss)
    ext = [-(-ss.dims[i].size // ss.dims[i].sharding) for i in range(rank)]
    m2m = list(minor_to_major) if minor_to_major is not None else list(range(rank - 1, -1, -1))
    stride = [0] * rank
    acc = 1
    for d in m2m:
        stride[d] = acc
        acc *= ext[d]
    coord = [idx[i] // ext[i] for i in range(rank)] + [0] * (len(ss.dims) - rank)
    order = sorted(range(len(ss.dims)), key=lambda i: ss.dims[i].permutation)
    dev = 0
    for i in order:
        dev = dev * ss.dims[i].sharding + coord[i]
    off = sum((idx[i] % ext[i]) * stride[i] for i in range(rank))
    return shards[ss.dev_start + dev][off]


def test_device_order_follows_reference_goldens():
    # mm_sharding_test.cc:667-717: tile dims [4,2,3], permutation {2,0,1}:
    # device = (j*3 + k)*4 + i
    ss = SS("BF16", [(8, 4, 2), (4, 2, 0), (6, 3, 1)], 0, 24)
    for i, j, k in itertools.product(range(4), range(2), range(3)):
        assert ro.device_of_tile(ss, [i, j, k]) == (j * 3 + k) * 4 + i
        assert ro.tile_of_device(ss, (j * 3 + k) * 4 + i) == [i, j, k]
    # mm_sharding_test.cc:529-594: replication entry most significant
    ss = SS("BF16", [(4, 1, 1), (8, 2, 2), (12, 4, 3), (4, 2, 4), (1, 3, 0)], 0, 48)
    assert ro.device_of_tile(ss, [0, 1, 3, 1, 2]) == 2 * 16 + (1 * 4 + 3) * 2 + 1
    assert ro.has_replication_dim(ss) and ro.tensor_rank(ss) == 4
    assert ro.shard_shape(ss) == (4, 4, 3, 2)


CASES = [
    # (name, shape, dtype, src, dst, src_m2m, dst_m2m)
    ("rows4_to_2x2", (8, 8), "F32", SS("F32", [(8, 4, 0), (8, 1, 1)], 0, 4),
     SS("F32", [(8, 2, 0), (8, 2, 1)], 4, 4), None, None),
    ("hidden_to_seq", (2, 8, 16), "BF16", SS("BF16", [(2, 1, 0), (8, 1, 1), (16, 8, 2)], 0, 8),
     SS("BF16", [(2, 1, 0), (8, 4, 1), (16, 1, 2)], 8, 4), None, None),
    ("uneven_3_to_5", (4, 17), "S32", SS("S32", [(4, 1, 0), (17, 3, 1)], 0, 3),
     SS("S32", [(4, 1, 0), (17, 5, 1)], 3, 5), None, None),
    ("empty_edge_tile", (8, 3), "U8", SS("U8", [(8, 3, 0), (3, 1, 1)], 0, 3),
     SS("U8", [(8, 5, 0), (3, 1, 1)], 3, 5), None, None),
    ("replicated_src_permuted_devices", (6, 4), "F64",
     SS("F64", [(6, 3, 1), (4, 1, 2), (1, 2, 0)], 2, 6),
     SS("F64", [(6, 2, 1), (4, 2, 0)], 10, 4), None, None),
    ("replicated_dst", (4, 6), "S16", SS("S16", [(4, 2, 0), (6, 3, 1)], 0, 6),
     SS("S16", [(4, 2, 1), (6, 1, 2), (1, 3, 0)], 6, 6), None, None),
    ("heads_to_seq_transposed_layout", (2, 4, 6, 3), "BF16",
     SS("BF16", [(2, 1, 0), (4, 2, 1), (6, 1, 2), (3, 1, 3)], 0, 2),
     SS("BF16", [(2, 1, 0), (4, 1, 1), (6, 3, 2), (3, 1, 3)], 2, 3), None, [3, 1, 2, 0]),
    ("minor_changing_layout", (5, 7), "F32", SS("F32", [(5, 2, 0), (7, 1, 1)], 0, 2),
     SS("F32", [(5, 1, 0), (7, 3, 1)], 2, 3), None, [0, 1]),
    ("scalar_broadcast", (), "F32", SS("F32", [(1, 4, 0)], 0, 4), SS("F32", [(1, 8, 0)], 0, 8), None, None),
    ("c128", (3, 5), "C128", SS("C128", [(3, 3, 0), (5, 1, 1)], 0, 3),
     SS("C128", [(3, 1, 0), (5, 2, 1)], 3, 2), None, None),
]


def _global(shape, element_type, seed=0):
    dt = ro.raw_dtype(element_type)
    n = int(np.prod(shape)) if shape else 1
    rng = np.random.Generator(np.random.PCG64(seed))
    raw = rng.integers(0, 256, size=n * dt.itemsize, dtype=np.uint8)
    return raw.view(dt).reshape(shape)


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_numpy_oracle_against_element_brute_force(case):
    _, shape, et, src, dst, sm, dm = case
    g = _global(shape, et, seed=11)
    src_shards = ro.make_shards(g, src, sm)
    # source side: every global element is found where the descriptor says
    for idx in itertools.product(*[range(s) for s in shape]):
        assert brute_force_src_lookup(src_shards, src, idx, sm) == g[idx]
    out = ro.reshard(src_shards, src, dst, sm, dm)
    assert sorted(out) == list(range(dst.dev_start, dst.dev_start + dst.dev_count))
    for dev, buf in out.items():
        expect = brute_force_dst(g, dst, dev, dm)
        assert buf.tobytes() == expect.tobytes(), (dev,)


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
@pytest.mark.parametrize("threads", [1, 3])
def test_c_restatement_matches_numpy_oracle(case, threads):
    _, shape, et, src, dst, sm, dm = case
    g = _global(shape, et, seed=12)
    src_shards = ro.make_shards(g, src, sm)
    expect = ro.reshard(src_shards, src, dst, sm, dm)
    got = {d: np.full_like(v, 0xAB if v.dtype.names is None else 0) for d, v in expect.items()}
    for v in got.values():
        v.view(np.uint8)[...] = 0xAB  # poison: pad must come back zero
    reshard_cpu.reshard(src_shards, src, dst, got, threads, sm, dm)
    for d in expect:
        assert got[d].tobytes() == expect[d].tobytes(), d


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_round_trip_restores_source(case):
    _, shape, et, src, dst, sm, dm = case
    g = _global(shape, et, seed=13)
    a = ro.make_shards(g, src, sm)
    b = ro.reshard(a, src, dst, sm, dm)
    a2 = ro.reshard(b, dst, src, dm, sm)
    for d in a:
        assert a[d].tobytes() == a2[d].tobytes()


@st.composite
def sharding_pairs(draw):
    rank = draw(st.integers(1, 3))
    shape = [draw(st.integers(1, 7)) for _ in range(rank)]

    def side(start):
        shard = [draw(st.integers(1, 4)) for _ in range(rank)]
        repl = draw(st.sampled_from([1, 1, 2]))
        if repl == 1 and shape[-1] == 1:
            # a trailing {size 1, sharding R>1} entry IS the replication entry
            # (mm_sharding.cc:356-358, 646-649); keep the tensor dim unambiguous
            shard[-1] = 1
        entries = shard + ([repl] if repl > 1 else [])
        perm = draw(st.permutations(list(range(len(entries)))))
        dims = [(shape[i], shard[i], perm[i]) for i in range(rank)]
        if repl > 1:
            dims.append((1, repl, perm[rank]))
        count = int(np.prod(entries))
        m2m = draw(st.one_of(st.none(), st.permutations(list(range(rank)))))
        return SS("U16", dims, start, count), (list(m2m) if m2m is not None else None)

    src, sm = side(draw(st.integers(0, 3)))
    dst, dm = side(draw(st.integers(0, 40)))
    return shape, src, dst, sm, dm


@given(sharding_pairs())
@settings(max_examples=120, deadline=None)
def test_random_pairs_numpy_c_and_brute_force_agree(p):
    shape, src, dst, sm, dm = p
    g = _global(shape, "U16", seed=5)
    src_shards = ro.make_shards(g, src, sm)
    expect = ro.reshard(src_shards, src, dst, sm, dm)
    got = {d: np.full_like(v, 0xBEEF) for d, v in expect.items()}
    reshard_cpu.reshard(src_shards, src, dst, got, 2, sm, dm)
    for d in expect:
        assert got[d].tobytes() == expect[d].tobytes()
        assert expect[d].tobytes() == brute_force_dst(g, dst, d, dm).tobytes()


def test_fp8_workload_bits_equal_torch_cast():
    """The fp8-e4m3fn benchmark input is specified as a torch cast; the workload
    generator does it in NumPy (GPU processes stay free of torch).  Same bits on
    every representable value, every rounding midpoint and its float32
    neighbours, the overflow edge (448 / 464 / 480), specials and 3M random draws."""
    torch = pytest.importorskip("torch")
    from multimesh_jax_amd.workloads import fp8_e4m3fn_bits

    def cast(x):
        return torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()

    rng = np.random.default_rng(0)
    every = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    finite = np.sort(every[np.isfinite(every)])
    mid = ((finite[:-1].astype(np.float64) + finite[1:]) / 2).astype(np.float32)
    up, down = np.float32(np.inf), np.float32(-np.inf)
    points = np.concatenate([finite, mid, np.nextafter(mid, up), np.nextafter(mid, down), np.nextafter(finite, up),
                             np.nextafter(finite, down)]).astype(np.float32)
    special = np.array([0.0, -0.0, 1e-10, -1e-10, 2 ** -10, 2 ** -9, 3 * 2 ** -10, 2 ** -6, 447.9, 448, 463.99, 464, 464.01,
                        479.9, 480, 500, 1e9, np.inf, -np.inf, np.nan], dtype=np.float32)
    draws = [np.clip(rng.standard_normal(1_000_000, dtype=np.float32), -448, 448),
             rng.standard_normal(1_000_000, dtype=np.float32) * np.float32(0.01),
             rng.standard_normal(1_000_000, dtype=np.float32) * np.float32(200)]
    for x in [points, special] + draws:
        assert np.array_equal(fp8_e4m3fn_bits(x), cast(x))
