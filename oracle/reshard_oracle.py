"""NumPy oracle of the cross-submesh reshard.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library imports this file;
only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may.

What it restates.  The reference's reshard entry point forwards two sharded
arrays to a third-party runtime (src/pjrt_client/zuku_execute_context_impl.cc:
437-452 -> zuku::Reshard, zuku 24.9.0 @ dd24496e, not vendored; its Realm copy
engine is legion 24.9.0 @ 228238b0).  No reference test pins the bytes that call
produces (every C++ test uses a mock, mm_mock_mm_xla.cc:255-269), so the result
is fixed by what the call means, with the descriptors exactly as the reference
fills them (mm_sharding.cc:345-372, 427-431, 638-654):

  * dims[i] = {size = GLOBAL extent, sharding = number of tiles,
    permutation = rank of this dim in device-id significance, 0 = most
    significant}; an optional trailing {size 1, sharding R} entry replicates
    the array R times (mm_sharding.cc:356-358, 646-649).
  * devices = contiguous ids [start, start + num_devices).
  * a tile holds ceil(size / sharding) elements per dim, the XLA convention
    the plugin's shard shapes come from (spmd::MakePartitionedShape, call
    sites mm_sharding.cc:69, mm_pjrt_executable.cc:537); the last tiles of a
    non-divisible dim are short or empty.
  * every destination tile := the slice of the global array it covers, the
    global array being the concatenation of the source tiles by tile
    coordinate.

Pinned by: brute force over single elements on tiny inputs
(tests/test_oracle_reshard.py computes each element's owner tile by integer division,
independently of the slicing below), the round trip A->B->A, and the three
device-order goldens of mm_sharding_test.cc:529-717 for the device <-> tile
coordinate map.

Two things are NOT reference behaviour and therefore "parity unpinned":
  * pad content of short tiles (the reference rejects non-divisible shardings,
    mpmd_logical_to_gspmd_sharding.cc:101-113): defined here as zero;
  * a physical layout per shard (`minor_to_major`) and 1-byte FP8 types: the
    reference descriptor carries neither (mm_sharding.cc:376-425 rejects FP8).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from .sharding_oracle import ShardedShape, ShardingDim  # noqa: F401

ITEMSIZE = {
    "PRED": 1, "S8": 1, "U8": 1, "F8E4M3FN": 1, "F8E5M2": 1,
    "F16": 2, "BF16": 2, "S16": 2, "U16": 2,
    "F32": 4, "S32": 4, "U32": 4,
    "F64": 8, "S64": 8, "U64": 8, "C64": 8,
    "C128": 16,
}


def raw_dtype(element_type: str) -> np.dtype:
    """Bit-moving dtype of one element (nothing is ever typed as float)."""
    n = ITEMSIZE[element_type]
    if n == 16:
        return np.dtype([("lo", "<u8"), ("hi", "<u8")])
    return np.dtype("<u%d" % n)


def has_replication_dim(ss: ShardedShape) -> bool:
    return len(ss.dims) > 0 and ss.dims[-1].size == 1 and ss.dims[-1].sharding > 1


def tensor_rank(ss: ShardedShape) -> int:
    return len(ss.dims) - (1 if has_replication_dim(ss) else 0)


def global_shape(ss: ShardedShape) -> Tuple[int, ...]:
    return tuple(d.size for d in ss.dims[:tensor_rank(ss)])


def tile_extent(size: int, sharding: int) -> int:
    return -(-size // sharding)


def shard_shape(ss: ShardedShape) -> Tuple[int, ...]:
    """Logical (row-major) shape of every shard buffer, padding included."""
    return tuple(tile_extent(d.size, d.sharding) for d in ss.dims[:tensor_rank(ss)])


def device_strides(ss: ShardedShape) -> List[int]:
    """Stride of every descriptor dim in the device id: the dim whose
    `permutation` is largest varies fastest."""
    n = len(ss.dims)
    perms = sorted(d.permutation for d in ss.dims)
    if perms != list(range(n)):
        raise ValueError("permutation fields are not a permutation of 0..n-1")
    strides = [0] * n
    acc = 1
    for rank in range(n - 1, -1, -1):
        i = next(k for k in range(n) if ss.dims[k].permutation == rank)
        strides[i] = acc
        acc *= ss.dims[i].sharding
    if acc != ss.dev_count:
        raise ValueError("product of shardings %d != device count %d" % (acc, ss.dev_count))
    return strides


def device_of_tile(ss: ShardedShape, coord: Sequence[int]) -> int:
    st = device_strides(ss)
    return ss.dev_start + sum(c * s for c, s in zip(coord, st))


def tile_of_device(ss: ShardedShape, device: int) -> List[int]:
    st = device_strides(ss)
    rel = device - ss.dev_start
    if not 0 <= rel < ss.dev_count:
        raise ValueError("device %d outside the store's device list" % device)
    return [(rel // st[i]) % ss.dims[i].sharding for i in range(len(ss.dims))]


def tile_bounds(ss: ShardedShape, coord: Sequence[int]) -> List[Tuple[int, int]]:
    """[lo, hi) of the valid region of a tile per tensor dim (may be empty)."""
    out = []
    for i in range(tensor_rank(ss)):
        d = ss.dims[i]
        e = tile_extent(d.size, d.sharding)
        lo = min(coord[i] * e, d.size)
        hi = min(lo + e, d.size)
        out.append((lo, hi))
    return out


def _default_m2m(rank: int) -> List[int]:
    return list(range(rank - 1, -1, -1))


def _to_physical(tile: np.ndarray, minor_to_major: Optional[Sequence[int]]) -> np.ndarray:
    if minor_to_major is None or list(minor_to_major) == _default_m2m(tile.ndim):
        return np.ascontiguousarray(tile)
    major_to_minor = list(minor_to_major)[::-1]
    return np.ascontiguousarray(tile.transpose(major_to_minor))


def _to_logical(buf: np.ndarray, shape: Sequence[int],
                minor_to_major: Optional[Sequence[int]]) -> np.ndarray:
    rank = len(shape)
    if minor_to_major is None or list(minor_to_major) == _default_m2m(rank):
        return buf.reshape(shape)
    major_to_minor = list(minor_to_major)[::-1]
    phys_shape = [shape[d] for d in major_to_minor]
    inv = np.argsort(major_to_minor)
    return buf.reshape(phys_shape).transpose(inv)


def make_shards(global_array: np.ndarray, ss: ShardedShape,
                minor_to_major: Optional[Sequence[int]] = None) -> Dict[int, np.ndarray]:
    """Lay a global array (already in its raw_dtype) out under `ss`:
    device id -> flat physical shard buffer, pad zero-filled."""
    assert tuple(global_array.shape) == global_shape(ss)
    sshape = shard_shape(ss)
    out = {}
    for dev in range(ss.dev_start, ss.dev_start + ss.dev_count):
        coord = tile_of_device(ss, dev)
        b = tile_bounds(ss, coord)
        tile = np.zeros(sshape, dtype=global_array.dtype)
        sl_g = tuple(slice(lo, hi) for lo, hi in b)
        sl_t = tuple(slice(0, hi - lo) for lo, hi in b)
        tile[sl_t] = global_array[sl_g]
        out[dev] = _to_physical(tile, minor_to_major).reshape(-1)
    return out


def assemble_global(shards: Dict[int, np.ndarray], ss: ShardedShape,
                    minor_to_major: Optional[Sequence[int]] = None) -> np.ndarray:
    """Concatenate source tiles by tile coordinate; of R replicas the one with
    the lowest device id is read (replicas are identical, so which one is
    unobservable)."""
    rank = tensor_rank(ss)
    sshape = shard_shape(ss)
    any_buf = next(iter(shards.values()))
    g = np.zeros(global_shape(ss), dtype=any_buf.dtype)
    for dev in range(ss.dev_start, ss.dev_start + ss.dev_count):
        coord = tile_of_device(ss, dev)
        if has_replication_dim(ss) and coord[-1] != 0:
            continue
        b = tile_bounds(ss, coord)
        tile = _to_logical(shards[dev], sshape, minor_to_major)
        sl_g = tuple(slice(lo, hi) for lo, hi in b)
        sl_t = tuple(slice(0, hi - lo) for lo, hi in b)
        g[sl_g] = tile[sl_t]
    assert g.ndim == rank
    return g


def reshard(src_shards: Dict[int, np.ndarray], src: ShardedShape, dst: ShardedShape,
            src_minor_to_major: Optional[Sequence[int]] = None,
            dst_minor_to_major: Optional[Sequence[int]] = None) -> Dict[int, np.ndarray]:
    """Every destination shard buffer (device id -> flat physical buffer)."""
    if global_shape(src) != global_shape(dst):
        raise ValueError("source and destination describe different global shapes")
    if ITEMSIZE[src.type] != ITEMSIZE[dst.type]:
        raise ValueError("source and destination element sizes differ")
    g = assemble_global(src_shards, src, src_minor_to_major)
    return make_shards(g, dst, dst_minor_to_major)
