"""mmreshard: MI355X-native cross-submesh resharding.

The compute path is libmmreshard.so (C ABI in include/mmreshard.h: host-side
planner + gfx950 HIP kernels).  This package is the ctypes view of that ABI with
the reference's names for the path.
"""
from . import _binding
from ._binding import LIB_PATH, MmrError, load  # noqa: F401
from .api import (  # noqa: F401
    CanonicalizeSharding, ComputeGlobalIndex, ComputeIndexSet, DeviceListOfSharding, LogicalShardingToOpSharding, LogicalToPhysicalSharding,
    MeshEquivalentSharding, NeedsReshard, Plan, ReplicateDims, ReshardContext, ResizeSharding, StoreHandle, TileAssignmentDevices,
    ToMpmdSharding,
    XlaShapeToZukuShape, describe, device_of_tile, itemsize, op_sharding, partition_spec_to_sharded_shape, shard_bytes,
    shard_extents,
    sharded_shape, tile_of_device,
)
