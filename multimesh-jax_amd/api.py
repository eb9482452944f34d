"""Host-side mirror of the reference's reshard interface over the C ABI.

Names and argument meaning follow the reference's C++ surface for this path:
the descriptor functions of src/pjrt_client/mm_sharding.{h,cc} and the store
subset of xla::ZukuExecuteContext (src/pjrt_client/zuku_execute_context.h:38-133).
Everything here is a thin ctypes call into libmmreshard.so; no arithmetic of the
path is done in Python and there is no fallback when the library or the GPU is
missing.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import numpy as np

from . import _binding as B
from ._binding import MmrError  # noqa: F401  (re-export)

ITEMSIZE = {name: None for name in B.DTYPES}


def itemsize(element_type: str) -> int:
    return B.load().mmr_itemsize(B.DTYPES[element_type])


# --------------------------------------------------------------------------
# descriptors
# --------------------------------------------------------------------------
def sharded_shape(type: str, dims: Sequence[Tuple[int, int, int]], dev_start: int, dev_count: int,
                  minor_to_major: Optional[Sequence[int]] = None) -> B.ShardedShape:
    """zuku::ShardedShape{type, sharding{dims{size, sharding, permutation}, devices{start, num_devices}}}."""
    if len(dims) > B.MMR_MAX_DIMS:
        raise ValueError("at most %d descriptor entries" % B.MMR_MAX_DIMS)
    s = B.ShardedShape()
    s.dtype = B.DTYPES[type]
    s.ndims = len(dims)
    for i, (size, sharding, permutation) in enumerate(dims):
        s.dims[i] = B.ShardingDim(size, sharding, permutation)
    s.dev_start, s.dev_count = dev_start, dev_count
    if minor_to_major is not None:
        s.has_layout = 1
        for i, m in enumerate(minor_to_major):
            s.minor_to_major[i] = m
    return s


def describe(s: B.ShardedShape) -> dict:
    d = {"type": B.DTYPE_NAMES.get(s.dtype, s.dtype),
         "dims": [[s.dims[i].size, s.dims[i].sharding, s.dims[i].permutation] for i in range(s.ndims)],
         "dev_start": s.dev_start, "dev_count": s.dev_count}
    if s.has_layout:
        d["minor_to_major"] = [s.minor_to_major[i] for i in range(s.ndims)]
    return d


def op_sharding(type: str = "OTHER", tile_dims: Sequence[int] = (), iota_reshape_dims: Sequence[int] = (),
                iota_transpose_perm: Sequence[int] = (), tile_assignment_devices: Sequence[int] = (),
                replicate_on_last_tile_dim: bool = False, iota_offset: int = 0) -> B.OpSharding:
    o = B.OpSharding()
    o.type = B.SHARDING_TYPES[type]
    o.n_tile_dims = len(tile_dims)
    for i, t in enumerate(tile_dims):
        o.tile_dims[i] = t
    o.n_iota_dims = len(iota_reshape_dims)
    for i, t in enumerate(iota_reshape_dims):
        o.iota_reshape_dims[i] = t
    perm = list(iota_transpose_perm) or list(range(len(iota_reshape_dims)))
    for i, t in enumerate(perm):
        o.iota_transpose_perm[i] = t
    o.replicate_on_last_tile_dim = int(replicate_on_last_tile_dim)
    o.iota_offset = iota_offset
    if tile_assignment_devices:
        arr = (C.c_int64 * len(tile_assignment_devices))(*tile_assignment_devices)
        o._keepalive = arr
        o.tile_assignment_devices = C.cast(arr, C.POINTER(C.c_int64))
        o.n_devices = len(tile_assignment_devices)
    return o


def _i64(values: Sequence[int]):
    return (C.c_int64 * max(len(values), 1))(*values)


def ComputeIndexSet(global_index: int, dims: Sequence[int]) -> List[int]:
    out = _i64([0] * len(dims))
    B.check(B.load().mmr_compute_index_set(global_index, _i64(dims), len(dims), out))
    return list(out)[:len(dims)]


def ComputeGlobalIndex(indices: Sequence[int], dims: Sequence[int]) -> int:
    out = C.c_int64()
    B.check(B.load().mmr_compute_global_index(_i64(indices), _i64(dims), len(dims), C.byref(out)))
    return out.value


def LogicalToPhysicalSharding(logical_to_device_axes: Sequence[Sequence[int]], devices: Tuple[int, int],
                              dims: Sequence[int], list_all_devices: bool = False) -> B.OpSharding:
    flat: List[int] = []
    begin = [0]
    for axes in logical_to_device_axes:
        flat.extend(axes)
        begin.append(len(flat))
    out = B.OpSharding()
    B.check(B.load().mmr_logical_to_physical_sharding(
        (C.c_int32 * max(len(flat), 1))(*flat), (C.c_int32 * len(begin))(*begin), len(logical_to_device_axes),
        devices[0], devices[1], _i64(dims), len(dims), int(list_all_devices), C.byref(out)))
    return out


def _strs(values: Sequence[str]):
    return (C.c_char_p * max(len(values), 1))(*[v.encode() for v in values])


def LogicalShardingToOpSharding(mesh_dims: Sequence[int], mesh_axes: Sequence[str],
                                logical_axes: Sequence[Tuple[str, str]], logical_axis_names: Sequence[Sequence[str]],
                                shape: Sequence[int], devices: Tuple[int, int], total_devices: int) -> B.OpSharding:
    """PartitionSpec-style names of one array -> OpSharding (mpmd_logical_to_gspmd_sharding.cc:21-124)."""
    flat: List[str] = []
    begin = [0]
    for names in logical_axis_names:
        flat.extend(names)
        begin.append(len(flat))
    out = B.OpSharding()
    B.check(B.load().mmr_logical_sharding_to_op_sharding(
        _i64(mesh_dims), _strs(mesh_axes), len(mesh_dims), _strs([a for a, _ in logical_axes]),
        _strs([b for _, b in logical_axes]), len(logical_axes), _strs(flat), (C.c_int32 * len(begin))(*begin),
        len(logical_axis_names), _i64(shape), devices[0], devices[1], total_devices, C.byref(out)))
    return out


def partition_spec_to_sharded_shape(mesh: Sequence[Tuple[str, int]], spec: Sequence[Optional[str]],
                                    shape: Sequence[int], element_type: str, devices: Tuple[int, int],
                                    total_devices: Optional[int] = None) -> B.ShardedShape:
    """A jax-style PartitionSpec on a named mesh -> the descriptor the reshard consumes:
    LogicalShardingToOpSharding with every mesh axis as its own logical axis, then XlaShapeToZukuShape."""
    axes = [n for n, _ in mesh]
    op = LogicalShardingToOpSharding([s for _, s in mesh], axes, [(n, n) for n in axes],
                                     [[p] if p else [] for p in spec], shape, devices,
                                     total_devices if total_devices is not None else devices[1])
    return XlaShapeToZukuShape(shape, element_type, devices, op, True)


def TileAssignmentDevices(op: B.OpSharding) -> List[int]:
    n = 1
    for i in range(op.n_tile_dims):
        n *= op.tile_dims[i]
    out = _i64([0] * n)
    got = C.c_int64()
    B.check(B.load().mmr_tile_assignment_devices(C.byref(op), out, n, C.byref(got)))
    return list(out)[:got.value]


def CanonicalizeSharding(op: B.OpSharding, shape: Sequence[int], element_type: str,
                         shape_is_global: bool = True) -> B.ShardedShape:
    out = B.ShardedShape()
    B.check(B.load().mmr_canonicalize_sharding(C.byref(op), _i64(shape), len(shape), B.DTYPES[element_type],
                                               int(shape_is_global), C.byref(out)))
    return out


def XlaShapeToZukuShape(shape: Sequence[int], element_type: str, devices: Tuple[int, int], op: B.OpSharding,
                        shape_is_global: bool = True) -> B.ShardedShape:
    out = B.ShardedShape()
    B.check(B.load().mmr_xla_shape_to_sharded_shape(_i64(shape), len(shape), B.DTYPES[element_type], devices[0],
                                                    devices[1], C.byref(op), int(shape_is_global), C.byref(out)))
    return out


def MeshEquivalentSharding(lhs: B.OpSharding, rhs: B.OpSharding) -> bool:
    out = C.c_int32()
    B.check(B.load().mmr_mesh_equivalent_sharding(C.byref(lhs), C.byref(rhs), C.byref(out)))
    return bool(out.value)


def NeedsReshard(operand_devices: Tuple[int, int], devices: Tuple[int, int], operand_sharding: B.OpSharding,
                 sharding: B.OpSharding) -> bool:
    out = C.c_int32()
    B.check(B.load().mmr_needs_reshard(operand_devices[0], operand_devices[1], devices[0], devices[1],
                                       C.byref(operand_sharding), C.byref(sharding), C.byref(out)))
    return bool(out.value)


def DeviceListOfSharding(sharding: B.OpSharding) -> Tuple[int, int]:
    """(start, count) of the contiguous device range a sharding covers (mpmd_utils.cc:151-175)."""
    start, count = C.c_int64(), C.c_int64()
    B.check(B.load().mmr_device_list_of_sharding(C.byref(sharding), C.byref(start), C.byref(count)))
    return start.value, count.value


def ToMpmdSharding(rank: int, sharding: B.OpSharding, task_devices: Tuple[int, int],
                   global_devices: Tuple[int, int]) -> B.OpSharding:
    """A sharding written relative to a task's devices -> the sharding over global device ids
    (mpmd_partition.cc:128-166).  Device ranges are (start, count)."""
    out = B.OpSharding()
    n = max(int(sharding.n_devices), 1)
    devices = _i64([0] * n)
    B.check(B.load().mmr_to_mpmd_sharding(rank, C.byref(sharding), task_devices[0], task_devices[1], global_devices[0],
                                          global_devices[1], C.byref(out), devices, n))
    out._keepalive = devices
    return out


def ReplicateDims(replicated_dims: Sequence[int], sharding: B.OpSharding) -> B.OpSharding:
    """The tiling of the given tile-assignment dims moves into the trailing replication dim
    (mm_sharding.cc:458-582)."""
    out = B.OpSharding()
    B.check(B.load().mmr_replicate_dims(C.byref(sharding), _i64(list(replicated_dims) or [0]), len(replicated_dims),
                                        C.byref(out)))
    return out


def ResizeSharding(shape: Sequence[int], sharding: B.OpSharding, num_elements: int,
                   devices: Optional[Tuple[int, int]] = None) -> Optional[B.OpSharding]:
    """A sharding with `num_elements` tiles grown or shrunk from `sharding`, or None where the reference finds
    none (mm_sharding.cc:98-161).  `devices` = (start, count)."""
    out = B.OpSharding()
    found = C.c_int32()
    start, count = devices if devices is not None else (0, 0)
    backing = _i64([0] * max(count, 1))
    B.check(B.load().mmr_resize_sharding(_i64(list(shape) or [0]), len(shape), C.byref(sharding), num_elements, start, count,
                                         C.byref(out), backing, max(count, 1), C.byref(found)))
    if not found.value:
        return None
    out._keepalive = backing
    return out


def shard_extents(s: B.ShardedShape) -> Tuple[int, ...]:
    ext = _i64([0] * B.MMR_MAX_DIMS)
    rank = C.c_int32()
    B.check(B.load().mmr_shard_extents(C.byref(s), ext, C.byref(rank)))
    return tuple(ext[i] for i in range(rank.value))


def shard_bytes(s: B.ShardedShape) -> int:
    out = C.c_int64()
    B.check(B.load().mmr_shard_bytes(C.byref(s), C.byref(out)))
    return out.value


def device_of_tile(s: B.ShardedShape, coord: Sequence[int]) -> int:
    out = C.c_int64()
    B.check(B.load().mmr_device_of_tile(C.byref(s), _i64(coord), C.byref(out)))
    return out.value


def tile_of_device(s: B.ShardedShape, device: int) -> List[int]:
    out = _i64([0] * B.MMR_MAX_DIMS)
    B.check(B.load().mmr_tile_of_device(C.byref(s), device, out))
    return [out[i] for i in range(s.ndims)]


# --------------------------------------------------------------------------
# plans (host only)
# --------------------------------------------------------------------------
def _shape_array(shapes: Sequence[B.ShardedShape]):
    arr = (B.ShardedShape * max(len(shapes), 1))()
    for i, s in enumerate(shapes):
        arr[i] = s
    return arr


class Plan:
    """Copy plan of one or more (source, destination) descriptor pairs."""

    def __init__(self, srcs: Sequence[B.ShardedShape], dsts: Sequence[B.ShardedShape],
                 chunk_bytes: int = 0, order: int = 0, xcd_mode: int = 0, flags: int = 0):
        if isinstance(srcs, B.ShardedShape):
            srcs, dsts = [srcs], [dsts]
        self._lib = B.load()
        self._h = C.c_void_p()
        opt = B.PlanOptions(chunk_bytes, order, xcd_mode, flags)
        B.check(self._lib.mmr_plan_create(_shape_array(srcs), _shape_array(dsts), len(srcs), C.byref(opt),
                                          C.byref(self._h)))

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.mmr_plan_destroy(self._h)
            self._h = None

    @property
    def stats(self) -> dict:
        st = B.PlanStats()
        B.check(self._lib.mmr_plan_get_stats(self._h, C.byref(st)))
        return st.as_dict()

    def copy_chunks(self, kind: int) -> np.ndarray:
        """kind 0: the chunks of the copy-group launch, decoded in launch order; kind 1: generic chunks;
        kind 2: the row pieces of the span groups, one record each (structured array)."""
        n = self._lib.mmr_plan_get_copy_chunks(self._h, kind, None, 0)
        buf = (B.CopyChunk * max(n, 1))()
        self._lib.mmr_plan_get_copy_chunks(self._h, kind, buf, n)
        return np.frombuffer(buf, dtype=np.dtype(B.CopyChunk), count=n).copy()

    def transpose_chunks(self) -> np.ndarray:
        n = self._lib.mmr_plan_get_transpose_chunks(self._h, None, 0)
        buf = (B.TransposeChunk * max(n, 1))()
        self._lib.mmr_plan_get_transpose_chunks(self._h, buf, n)
        return np.frombuffer(buf, dtype=np.dtype(B.TransposeChunk), count=n).copy()

    def slot_bases(self) -> List[int]:
        n = self._lib.mmr_plan_get_slot_bases(self._h, None, 0)
        buf = _i64([0] * n)
        self._lib.mmr_plan_get_slot_bases(self._h, buf, n)
        return list(buf)[:n]


# --------------------------------------------------------------------------
# execution
# --------------------------------------------------------------------------
class StoreHandle:
    """One sharded array: a buffer per device of its device list (store_handle_fwd.h:15-19)."""

    def __init__(self, ctx: "ReshardContext", handle: C.c_void_p, shape: B.ShardedShape, name: str):
        self._ctx = ctx
        self._h = handle
        self.shape = shape
        self.name = name
        self.unique_id = B.load().mmr_store_id(handle)

    @property
    def devices(self) -> range:
        return range(self.shape.dev_start, self.shape.dev_start + self.shape.dev_count)

    @property
    def shard_bytes(self) -> int:
        return shard_bytes(self.shape)


class ReshardContext:
    """Store subset of xla::ZukuExecuteContext on one MI355X.

    Every logical device is a separate buffer in this GPU's HBM, so the
    per-device arguments of the reference (local_device_id, global_device_id)
    become an explicit `device` where one shard is meant and disappear where the
    reference call is control-replicated over the devices.
    """

    def __init__(self, hip_device: int = 0, hip_stream: Optional[int] = None):
        self._lib = B.load()
        self._h = C.c_void_p()
        B.check(self._lib.mmr_context_create(hip_device, C.c_void_p(hip_stream) if hip_stream else None,
                                             C.byref(self._h)))

    def close(self) -> None:
        if self._h:
            self._lib.mmr_context_destroy(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- stores -----------------------------------------------------------
    def CreateStore(self, shape: B.ShardedShape, name: Optional[str] = None,
                    allocate_from_cache: bool = False, min_cache_size: int = 1,
                    uninitialized: bool = False) -> StoreHandle:
        h = C.c_void_p()
        flags = (B.MMR_STORE_FROM_CACHE if allocate_from_cache else 0) | (B.MMR_STORE_UNINITIALIZED if uninitialized else 0)
        B.check(self._lib.mmr_store_create_ex(self._h, C.byref(shape), name.encode() if name else None, flags,
                                              min_cache_size, C.byref(h)))
        return StoreHandle(self, h, shape, name or "anonymous")

    def AssembleShards(self, shape: B.ShardedShape, device: int, data, existing_store: Optional[StoreHandle] = None,
                       size: Optional[int] = None, where: int = 1) -> StoreHandle:
        """Shard{data, local_device_id, size}: `data` is a NumPy array (host) or an int pointer; `where` says what an
        int pointer points at: 1 device memory, 0 host memory, 2 let the runtime find out, 3 device memory copied by
        the runtime's own kernel."""
        store = existing_store if existing_store is not None else self.CreateStore(shape)
        if isinstance(data, np.ndarray):
            arr = np.ascontiguousarray(data)
            B.check(self._lib.mmr_store_assemble(self._h, store._h, device, arr.ctypes.data, arr.nbytes, 0))
        else:
            if size is None:
                raise ValueError("size is required for a device pointer")
            B.check(self._lib.mmr_store_assemble(self._h, store._h, device, C.c_void_p(int(data)), size, where))
        return store

    def AdoptShards(self, shape: B.ShardedShape, device_ptrs: Sequence[int], name: Optional[str] = None) -> StoreHandle:
        """Zero-copy import: device_ptrs[k] becomes the buffer of device dev_start + k."""
        h = C.c_void_p()
        arr = (C.c_void_p * max(len(device_ptrs), 1))(*[C.c_void_p(int(p)) for p in device_ptrs])
        if len(device_ptrs) != shape.dev_count:
            raise ValueError("one pointer per device of the descriptor")
        B.check(self._lib.mmr_store_adopt(self._h, C.byref(shape), name.encode() if name else None, arr, C.byref(h)))
        return StoreHandle(self, h, shape, name or "anonymous")

    def OffloadDtoH(self, to_offload: Sequence[StoreHandle]) -> None:
        for s in to_offload:
            B.check(self._lib.mmr_store_offload(self._h, s._h))

    def OffloadHtoD(self, to_offload: Sequence[StoreHandle]) -> None:
        for s in to_offload:
            B.check(self._lib.mmr_store_reload(self._h, s._h))

    def IsOffloaded(self, store: StoreHandle) -> bool:
        out = C.c_int32()
        B.check(self._lib.mmr_store_is_offloaded(store._h, C.byref(out)))
        return bool(out.value)

    def PrepareReshard(self, srcs, dsts) -> None:
        """Build and upload the plan of descriptor pair(s) before any store exists."""
        if isinstance(srcs, B.ShardedShape):
            srcs, dsts = [srcs], [dsts]
        B.check(self._lib.mmr_context_prepare(self._h, _shape_array(srcs), _shape_array(dsts), len(srcs)))

    def BindReshard(self, srcs, dsts) -> None:
        """Plan and pointer table of these stores, built and uploaded without launching: the next
        Reshard / ReshardBatch of the same stores only launches kernels (and may be captured into a HIP graph)."""
        if isinstance(srcs, StoreHandle):
            srcs, dsts = [srcs], [dsts]
        n = len(srcs)
        sa = (C.c_void_p * max(n, 1))(*[s._h for s in srcs])
        da = (C.c_void_p * max(n, 1))(*[d._h for d in dsts])
        B.check(self._lib.mmr_reshard_bind(self._h, sa, da, n))

    def TuneReshard(self, srcs, dsts) -> int:
        """Times a few launch orders of the plan of these stores on the stores themselves and keeps the fastest
        (blocking; never done implicitly).  Returns the order now in use (0 = the default)."""
        if isinstance(srcs, StoreHandle):
            srcs, dsts = [srcs], [dsts]
        n = len(srcs)
        sa = (C.c_void_p * max(n, 1))(*[s._h for s in srcs])
        da = (C.c_void_p * max(n, 1))(*[d._h for d in dsts])
        used = C.c_int64()
        B.check(self._lib.mmr_reshard_tune(self._h, sa, da, n, C.byref(used)))
        return used.value

    def ClearPlans(self) -> None:
        B.check(self._lib.mmr_context_clear_plans(self._h))

    def set_flags(self, flags: int) -> None:
        B.check(self._lib.mmr_context_set_flags(self._h, flags))

    def SliceLocalShard(self, device: int, store: StoreHandle, wait: bool = True) -> int:
        p = C.c_void_p()
        fn = self._lib.mmr_store_shard_ptr if wait else self._lib.mmr_store_shard_ptr_async
        B.check(fn(self._h, store._h, device, C.byref(p)))
        return p.value or 0

    def ReadShard(self, store: StoreHandle, device: int, dtype=np.uint8) -> np.ndarray:
        """Host copy of one shard's bytes (what ToLiteral reads through SliceLocalShard)."""
        out = np.empty(store.shard_bytes, dtype=np.uint8)
        B.check(self._lib.mmr_store_read_shard(self._h, store._h, device, out.ctypes.data, out.nbytes))
        return out.view(dtype)

    def HasLocalShard(self, store: StoreHandle, device: int) -> bool:
        out = C.c_int32()
        B.check(self._lib.mmr_store_has_shard(store._h, device, C.byref(out)))
        return bool(out.value)

    def GetStoreShardedShape(self, store: StoreHandle) -> B.ShardedShape:
        out = B.ShardedShape()
        B.check(self._lib.mmr_store_get_shape(store._h, C.byref(out)))
        return out

    def Free(self, store: StoreHandle, keep_in_cache: bool = False) -> None:
        B.check(self._lib.mmr_store_free(self._h, store._h, int(keep_in_cache)))
        store._h = None

    def Destroy(self, store: StoreHandle) -> None:
        self.Free(store, keep_in_cache=False)

    def ClearStoreCache(self) -> None:
        B.check(self._lib.mmr_clear_store_cache(self._h))

    # -- the hot path -----------------------------------------------------
    def Reshard(self, src: StoreHandle, dst: StoreHandle) -> None:
        B.check(self._lib.mmr_reshard(self._h, src._h, dst._h))

    def ReshardBatch(self, srcs: Sequence[StoreHandle], dsts: Sequence[StoreHandle]) -> None:
        n = len(srcs)
        if n != len(dsts):
            raise ValueError("as many destinations as sources")
        key = (tuple(s.unique_id for s in srcs), tuple(d.unique_id for d in dsts))
        cached = getattr(self, "_batch_args", None)
        if cached is None or cached[0] != key:
            sa = (C.c_void_p * max(n, 1))(*[s._h for s in srcs])
            da = (C.c_void_p * max(n, 1))(*[d._h for d in dsts])
            self._batch_args = cached = (key, sa, da)
        B.check(self._lib.mmr_reshard_batch(self._h, cached[1], cached[2], n))

    def ReshardBatchStatic(self, srcs: Sequence[StoreHandle], dsts: Sequence[StoreHandle]) -> None:
        """ReshardBatch without any device allocation: the launch's tables live in the GPU's static scratch array
        (B.MMR_STATIC_SCRATCH_BYTES); a plan that does not fit raises INVALID_ARGUMENT."""
        n = len(srcs)
        if n != len(dsts):
            raise ValueError("as many destinations as sources")
        sa = (C.c_void_p * max(n, 1))(*[s._h for s in srcs])
        da = (C.c_void_p * max(n, 1))(*[d._h for d in dsts])
        B.check(self._lib.mmr_reshard_batch_static(self._h, sa, da, n))

    def Sync(self) -> None:
        B.check(self._lib.mmr_sync(self._h))

    # -- measurement and inspection ----------------------------------------
    def set_plan_options(self, chunk_bytes: int = 0, order: int = 0, xcd_mode: int = 0, flags: int = 0) -> None:
        opt = B.PlanOptions(chunk_bytes, order, xcd_mode, flags)
        B.check(self._lib.mmr_context_set_plan_options(self._h, C.byref(opt)))

    def StartTimer(self, name: Optional[str] = None) -> None:
        """StartTimer(name) of the reference (zuku_execute_context_impl.cc:462-467): named, any number pending, does
        not wait.  Without a name: the unnamed benchmark stopwatch (one interval at a time)."""
        if name is None:
            B.check(self._lib.mmr_timer_start(self._h))
        else:
            B.check(self._lib.mmr_timer_begin(self._h, name.encode()))

    def StopTimer(self, name: Optional[str] = None) -> Optional[float]:
        """StopTimer(name) (:469-486): does not wait; an unknown name is a warning as in the reference.  Without a
        name: stops the benchmark stopwatch, BLOCKS until the device gets there and returns milliseconds."""
        if name is None:
            ms = C.c_float()
            B.check(self._lib.mmr_timer_stop_wait(self._h, C.byref(ms)))
            return ms.value
        rc = self._lib.mmr_timer_end(self._h, name.encode())
        if rc == 5:  # MMR_NOT_FOUND
            import warnings
            warnings.warn(self._lib.mmr_last_error().decode("utf-8", "replace"))
            return None
        B.check(rc)
        return None

    def TimerResult(self, name: str, wait: bool = False):
        """(milliseconds of the most recent completed interval of `name`, intervals completed).  Never waits unless
        `wait` is set."""
        ms, n = C.c_float(), C.c_int64()
        fn = self._lib.mmr_timer_wait if wait else self._lib.mmr_timer_poll
        B.check(fn(self._h, name.encode(), C.byref(ms), C.byref(n)))
        return ms.value, n.value

    def MarkProfile(self, name: str) -> None:
        B.check(self._lib.mmr_profile_mark(self._h, name.encode()))

    def OpenWindow(self) -> None:
        B.check(self._lib.mmr_window_open(self._h))

    def CloseWindow(self) -> None:
        B.check(self._lib.mmr_window_close(self._h))

    def set_max_open_windows(self, n: int) -> None:
        B.check(self._lib.mmr_context_set_max_open_windows(self._h, n))

    def Lap(self) -> None:
        """A timing mark on the stream (see Laps)."""
        B.check(self._lib.mmr_timer_lap(self._h))

    def Laps(self, capacity: int = 4096) -> List[float]:
        """Device milliseconds between consecutive marks set with Lap() (blocks until the last one is reached)."""
        buf = (C.c_float * capacity)()
        n = C.c_int32()
        B.check(self._lib.mmr_timer_laps(self._h, buf, capacity, C.byref(n)))
        return [buf[i] for i in range(n.value)]

    @property
    def stream(self) -> int:
        p = C.c_void_p()
        B.check(self._lib.mmr_context_stream(self._h, C.byref(p)))
        return p.value or 0

    @property
    def stats(self) -> dict:
        st = B.ContextStats()
        B.check(self._lib.mmr_context_get_stats(self._h, C.byref(st)))
        return st.as_dict()

    def plan_stats(self, src: StoreHandle, dst: StoreHandle) -> dict:
        st = B.PlanStats()
        B.check(self._lib.mmr_reshard_plan_stats(self._h, src._h, dst._h, C.byref(st)))
        return st.as_dict()

    def batch_plan_stats(self, srcs: Sequence[StoreHandle], dsts: Sequence[StoreHandle]) -> dict:
        """Stats of the plan a ReshardBatch of these stores uses (table order chosen on first use included)."""
        n = len(srcs)
        if n == 0 or n != len(dsts):
            raise ValueError("as many destinations as sources, at least one")
        sa = (C.c_void_p * n)(*[s._h for s in srcs])
        da = (C.c_void_p * n)(*[d._h for d in dsts])
        st = B.PlanStats()
        B.check(self._lib.mmr_reshard_batch_plan_stats(self._h, sa, da, n, C.byref(st)))
        return st.as_dict()
