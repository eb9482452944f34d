"""The descriptor oracle against the reference's own known answers (tests/golden)
and against invariants the mathematics fixes."""
import itertools

import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from oracle import sharding_oracle as so


def _op(d):
    return so.OpSharding(
        type=d.get("type", "OTHER"),
        tile_assignment_dimensions=list(d.get("tile_dims", [])),
        iota_reshape_dims=list(d.get("iota_reshape_dims", [])),
        iota_transpose_perm=list(d.get("iota_transpose_perm", [])),
        tile_assignment_devices=list(d.get("tile_assignment_devices", [])),
        replicate_on_last_tile_dim=bool(d.get("replicate_on_last_tile_dim", False)),
        iota_offset=int(d.get("iota_offset", 0)),
    )


def _ss_tuple(ss):
    return {"type": ss.type, "dims": [[d.size, d.sharding, d.permutation] for d in ss.dims],
            "dev_start": ss.dev_start, "dev_count": ss.dev_count}


def test_index_set_known_answers(golden):
    for c in golden["index_set"]:
        assert so.compute_index_set(c["index"], c["dims"]) == c["expect"], c["source"]


def test_global_index_known_answers(golden):
    for c in golden["global_index"]:
        assert so.compute_global_index(c["indices"], c["dims"]) == c["expect"], c["source"]


@given(st.lists(st.integers(1, 5), min_size=0, max_size=5), st.data())
@settings(max_examples=100, deadline=None)
def test_index_round_trip(dims, data):
    n = int(np.prod(dims)) if dims else 1
    i = data.draw(st.integers(0, n - 1))
    idx = so.compute_index_set(i, dims)
    assert so.compute_global_index(idx, dims) == i
    if dims:
        assert tuple(idx) == tuple(int(v) for v in np.unravel_index(i, dims))


def test_logical_to_physical_known_answers(golden):
    for c in golden["logical_to_physical"]:
        op = so.logical_to_physical_sharding(c["axes"], tuple(c["devices"]), c["mesh"],
                                             c["list_all_devices"])
        e = c["expect"]
        assert op.type == e["type"], c["source"]
        if "tile_dims" in e:
            assert op.tile_assignment_dimensions == e["tile_dims"], c["source"]
        if "device_order" in e:
            assert so.iota_tile_assignment(op).reshape(-1).tolist() == e["device_order"], c["source"]
        if "replicate_on_last_tile_dim" in e:
            assert op.replicate_on_last_tile_dim == e["replicate_on_last_tile_dim"], c["source"]


def test_logical_to_physical_header_example():
    # worked example in the comment above the function (mm_sharding.cc:174-182):
    # mapping [(0,2), (), (1,)] on a [2,2,2] grid: tile dims [4,1,2] and logical
    # device 5 is physical device 6
    op = so.logical_to_physical_sharding([[0, 2], [], [1]], (0, 8), [2, 2, 2])
    assert op.tile_assignment_dimensions == [4, 1, 2]
    assert so.iota_tile_assignment(op).reshape(-1)[5] == 6


def test_canonicalize_known_answers(golden):
    for c in golden["canonicalize"]:
        op = _op(c["sharding"])
        if c["expect"].get("error"):
            with pytest.raises(so.ShardingError):
                so.canonicalize_sharding(op, c["shape"], c["element_type"], c["shape_is_global"])
            continue
        ss = so.canonicalize_sharding(op, c["shape"], c["element_type"], c["shape_is_global"])
        assert _ss_tuple(ss) == c["expect"], c["source"]


def test_canonicalize_local_shape_and_errors():
    # mm_sharding.cc:359-363: a local shape is scaled back to global extents
    op = _op({"tile_dims": [4, 2, 3], "iota_reshape_dims": [6, 4], "iota_transpose_perm": [1, 0]})
    ss = so.canonicalize_sharding(op, [2, 2, 2], "BF16", shape_is_global=False)
    assert [d.size for d in ss.dims] == [8, 4, 6]
    # mm_sharding.cc:422-424: FP8 and 4-bit types are rejected by the reference
    with pytest.raises(so.ShardingError):
        so.canonicalize_sharding(op, [8, 4, 6], "F8E4M3FN", True)
    # mm_sharding.cc:443-449: explicit device lists must be consecutive
    bad = _op({"tile_dims": [2, 2], "tile_assignment_devices": [0, 2, 1, 3]})
    with pytest.raises(so.ShardingError):
        so.canonicalize_sharding(bad, [4, 4], "F32", True)
    ok = _op({"tile_dims": [2, 2], "tile_assignment_devices": [4, 5, 6, 7]})
    ss = so.canonicalize_sharding(ok, [4, 4], "F32", True)
    assert _ss_tuple(ss) == {"type": "F32", "dims": [[4, 2, 0], [4, 2, 1]], "dev_start": 4, "dev_count": 4}


def test_replicated_descriptor_closed_form(golden):
    for c in golden["replicated_descriptor"]:
        ss = so.xla_shape_to_zuku_shape(c["shape"], c["element_type"], tuple(c["devices"]), _op(c["sharding"]))
        assert _ss_tuple(ss) == c["expect"], c["source"]


def test_device_list_override():
    # mm_sharding.cc:659-668: an equal-sized device list replaces the sharding's own
    op = _op({"tile_dims": [4, 1], "iota_reshape_dims": [4], "iota_transpose_perm": [0]})
    ss = so.xla_shape_to_zuku_shape([4, 4], "F32", (4, 4), op)
    assert (ss.dev_start, ss.dev_count) == (4, 4)
    with pytest.raises(so.ShardingError):
        so.xla_shape_to_zuku_shape([4, 4], "F32", (0, 8), op)


def test_needs_reshard_truth_table(golden):
    for c in golden["needs_reshard"]:
        got = so.needs_reshard(tuple(c["operand_devices"]), tuple(c["devices"]),
                               _op(c["operand_sharding"]), _op(c["sharding"]))
        assert got == c["expect"], c["source"]


def test_mesh_equivalent_sharding_cases():
    rep = _op({"type": "REPLICATED"})
    maximal = _op({"type": "MAXIMAL"})
    last = _op({"tile_dims": [1, 1, 4], "iota_reshape_dims": [4], "iota_transpose_perm": [0],
                "replicate_on_last_tile_dim": True})
    t41 = _op({"tile_dims": [4, 1], "iota_reshape_dims": [4], "iota_transpose_perm": [0]})
    t22 = _op({"tile_dims": [2, 2], "iota_reshape_dims": [4], "iota_transpose_perm": [0]})
    assert so.mesh_equivalent_sharding(rep, maximal)
    assert so.mesh_equivalent_sharding(rep, last)
    assert not so.mesh_equivalent_sharding(rep, t41)
    assert not so.mesh_equivalent_sharding(t41, rep)
    assert so.mesh_equivalent_sharding(t41, t41)
    assert not so.mesh_equivalent_sharding(t41, t22)


@given(st.lists(st.integers(1, 4), min_size=1, max_size=4), st.data())
@settings(max_examples=200, deadline=None)
def test_canonical_iota_enumerates_the_same_devices(reshape_dims, data):
    perm = data.draw(st.permutations(list(range(len(reshape_dims)))))
    n = int(np.prod(reshape_dims))
    raw = np.arange(n).reshape(reshape_dims).transpose(perm).reshape(-1)
    cd, cp = so.canonical_iota(reshape_dims, perm)
    can = np.arange(n).reshape(cd).transpose(cp).reshape(-1)
    assert raw.tolist() == can.tolist()
    assert all(d != 1 for d in cd) or cd == [1]
    # no two canonical dims stay adjacent and in order (otherwise they would merge)
    assert all(cp[i] + 1 != cp[i + 1] for i in range(len(cp) - 1))


def _device_of_tile_from_descriptor(ss, coord):
    order = sorted(range(len(ss.dims)), key=lambda i: ss.dims[i].permutation)
    dev = 0
    for i in order:
        dev = dev * ss.dims[i].sharding + coord[i]
    return ss.dev_start + dev


@given(st.data())
@settings(max_examples=150, deadline=None)
def test_canonical_descriptor_reproduces_the_tile_assignment(data):
    """For shardings whose iota transpose is an involution (all the reference's
    goldens are), `permutation` must reproduce XLA's device of every tile."""
    mesh = data.draw(st.lists(st.integers(1, 3), min_size=1, max_size=3))
    nlog = data.draw(st.integers(1, 3))
    axes_pool = list(range(len(mesh)))
    assign = [[] for _ in range(nlog)]
    for ax in axes_pool:
        where = data.draw(st.integers(-1, nlog - 1))
        if where >= 0:
            assign[where].append(ax)
    start = data.draw(st.integers(0, 5))
    op = so.logical_to_physical_sharding(assign, (start, int(np.prod(mesh))), mesh, list_all_devices=True)
    if op.type != "OTHER":
        return
    _, cperm = so.canonical_iota(op.iota_reshape_dims, op.iota_transpose_perm)
    if [cperm[p] for p in cperm] != list(range(len(cperm))):
        return  # the reference's group walk is only exercised on involutions
    shape = [t * 2 for t in op.tile_assignment_dimensions[:nlog]]
    try:
        ss = so.canonicalize_sharding(op, shape, "F32", True)
    except so.ShardingError:
        return
    ta = so.iota_tile_assignment(op)
    for coord in itertools.product(*[range(t) for t in op.tile_assignment_dimensions]):
        assert _device_of_tile_from_descriptor(ss, coord) == int(ta[coord])
