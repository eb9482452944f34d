"""CPU restatement of the reference's sharding-descriptor arithmetic.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library imports this file;
only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may.

Every function follows one function of the reference plugin (paths relative to
the reference checkout) and is pinned by the reference's own known-answer
tests, re-expressed as numbers in tests/golden/sharding_golden.json:

  compute_index_set / compute_global_index
      src/pjrt_client/mm_sharding.h:63-91
      pinned by mm_sharding_test.cc:57-99 (8 known answers)
  iota_tile_assignment
      XLA's IotaTileAssignment (iota(N).reshape(reshape_dims)
      .transpose(perm).reshape(tile_dims)), plus the plugin-specific
      `iota_offset` the reference adds (mm_sharding.cc:270)
      pinned by the device orders mm_sharding_test.cc:101-228 expects
  logical_to_physical_sharding
      src/pjrt_client/mm_sharding.cc:183-273
      pinned by mm_sharding_test.cc:101-228 (8 cases)
  logical_sharding_to_op_sharding
      src/pjrt_client/mpmd_logical_to_gspmd_sharding.cc:21-124
      pinned by the OpShardings mpmd_logical_to_gspmd_sharding_test.cc:48-64,
      190-205 expects (3 active cases, exact fields) and :116-187 (2 cases the
      reference skips; given in XLA's canonical form, compared as tile dims
      plus device order)
  to_mpmd_sharding
      src/pjrt_client/mpmd_partition.cc:128-166
      pinned by the store shardings mpmd_partition_test.cc:1381-1418 and
      :1455-1484 expect (rebased iota offsets; replication on a submesh)
  replicate_dims / resize_sharding (same file, off the reshard path: they
  serve sharding propagation at compile time)
      src/pjrt_client/mm_sharding.cc:458-582, 98-161
      pinned by mm_sharding_test.cc:247-527 (9 ReplicateDims cases, compared
      as tile dims + device order + the replication flag, which is what
      HloSharding equality compares) and :230-245 (3 ResizeSharding answers)
  canonicalize_sharding
      src/pjrt_client/mm_sharding.cc:275-456
      pinned by mm_sharding_test.cc:529-737 (3 golden descriptors, 1 error)
  xla_shape_to_zuku_shape
      src/pjrt_client/mm_sharding.cc:583-671
      replicated branch (:638-654) is a closed form; tiled branch is
      canonicalize_sharding + the device-list override (:659-668)
  is_replicated_* / mesh_equivalent_sharding / needs_reshard
      src/pjrt_client/mm_sharding.cc:19-51, mpmd_insert_reshard.cc:33-43
      pinned by the scenarios of mpmd_insert_reshard_test.cc:78-377
      re-expressed as truth-table rows

Descriptors are plain Python data:
  OpSharding  - the subset of XLA's OpSharding proto the reference reads
  ShardedShape - mirror of zuku::ShardedShape as the reference fills it
                 (mm_sharding.cc:345-372, 427-431, 638-654)
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

import numpy as np

# Element types the reference accepts (mm_sharding.cc:376-425); anything else is
# "Unsupported type".
SUPPORTED_TYPES = (
    "PRED", "F16", "BF16", "F32", "F64", "S8", "S16", "S32", "S64",
    "U8", "U16", "U32", "U64", "C64", "C128",
)


class ShardingError(ValueError):
    """The reference returns a non-OK absl::Status at this point."""


@dataclass
class OpSharding:
    type: str = "OTHER"  # "REPLICATED" | "MAXIMAL" | "OTHER"
    tile_assignment_dimensions: List[int] = field(default_factory=list)
    iota_reshape_dims: List[int] = field(default_factory=list)
    iota_transpose_perm: List[int] = field(default_factory=list)
    tile_assignment_devices: List[int] = field(default_factory=list)
    replicate_on_last_tile_dim: bool = False
    iota_offset: int = 0

    @property
    def is_replicated(self) -> bool:
        return self.type == "REPLICATED"

    @property
    def is_tile_maximal(self) -> bool:
        return self.type == "MAXIMAL"

    @property
    def has_iota(self) -> bool:
        return len(self.iota_reshape_dims) > 0

    def num_elements(self) -> int:
        n = 1
        for d in self.tile_assignment_dimensions:
            n *= d
        return n


@dataclass(frozen=True)
class ShardingDim:
    size: int
    sharding: int
    permutation: int


@dataclass(frozen=True)
class ShardedShape:
    type: str
    dims: Tuple[ShardingDim, ...]
    dev_start: int
    dev_count: int


# --------------------------------------------------------------------------
# mm_sharding.h:63-91
# --------------------------------------------------------------------------
def compute_index_set(global_index: int, dims: Sequence[int]) -> List[int]:
    indices = [0] * len(dims)
    remainder = global_index
    dim_stride = 1
    for d in dims:
        dim_stride *= d
    for i, d in enumerate(dims):
        dim_stride //= d
        indices[i] = remainder // dim_stride
        remainder -= indices[i] * dim_stride
    return indices


def compute_global_index(indices: Sequence[int], dims: Sequence[int]) -> int:
    stride = 1
    index = 0
    for dim in range(len(indices) - 1, -1, -1):
        index += stride * indices[dim]
        stride *= dims[dim]
    return index


# --------------------------------------------------------------------------
# XLA IotaTileAssignment (+ the reference's iota_offset)
# --------------------------------------------------------------------------
def iota_tile_assignment(op: OpSharding) -> np.ndarray:
    """Device id of every tile, shaped like tile_assignment_dimensions."""
    dims = list(op.tile_assignment_dimensions)
    if op.has_iota:
        n = int(np.prod(op.iota_reshape_dims))
        a = np.arange(n, dtype=np.int64).reshape(op.iota_reshape_dims)
        perm = list(op.iota_transpose_perm) or list(range(a.ndim))
        a = a.transpose(perm).reshape(dims)
        return a + op.iota_offset
    return np.asarray(op.tile_assignment_devices, dtype=np.int64).reshape(dims)


def canonical_iota(reshape_dims: Sequence[int], transpose_perm: Sequence[int]
                   ) -> Tuple[List[int], List[int]]:
    """Canonical (reshape_dims, transpose_perm) of an iota tile assignment.

    The reference never sees a raw proto: HloSharding::FromProto builds the
    assignment through XLA's IotaTileAssignment::Create (third-party, pinned in
    cmake/versions.json), which drops size-1 iota dims and merges iota dims
    that stay adjacent and in order after the transpose.  CanonicalizeSharding
    (mm_sharding.cc:275-339) walks that canonical form.  The form is pinned by
    an invariant: it must enumerate exactly the same devices as the raw one.
    """
    dims = list(reshape_dims)
    perm = list(transpose_perm) if transpose_perm else list(range(len(dims)))
    # drop size-1 dims, renumber the survivors
    keep = [i for i, d in enumerate(dims) if d != 1]
    renum = {old: new for new, old in enumerate(keep)}
    perm = [renum[p] for p in perm if p in renum]
    dims = [dims[i] for i in keep]
    if not dims:
        return [1], [0]
    # merge dims that are consecutive both before and after the transpose
    merged_perm_groups: List[List[int]] = []
    for p in perm:
        if merged_perm_groups and merged_perm_groups[-1][-1] + 1 == p:
            merged_perm_groups[-1].append(p)
        else:
            merged_perm_groups.append([p])
    # new iota dims in original order
    order = sorted(range(len(merged_perm_groups)), key=lambda g: merged_perm_groups[g][0])
    new_index = {g: i for i, g in enumerate(order)}
    new_dims = []
    for g in order:
        n = 1
        for p in merged_perm_groups[g]:
            n *= dims[p]
        new_dims.append(n)
    new_perm = [new_index[g] for g in range(len(merged_perm_groups))]
    return new_dims, new_perm


# --------------------------------------------------------------------------
# mm_sharding.cc:183-273
# --------------------------------------------------------------------------
def logical_to_physical_sharding(
    logical_to_device_axes: Sequence[Sequence[int]],
    devices: Tuple[int, int],
    dims: Sequence[int],
    list_all_devices: bool = False,
) -> OpSharding:
    """devices = (start, num_devices); dims = device-mesh axis sizes."""
    num_logical_dims = len(logical_to_device_axes)
    device_axes_used = [0] * len(dims)
    fully_replicated = True
    for axes in logical_to_device_axes:
        for d in axes:
            device_axes_used[d] = 1
            if dims[d] > 1:
                fully_replicated = False

    if num_logical_dims == 0 or (fully_replicated and not list_all_devices):
        return OpSharding(type="REPLICATED")

    replicated_device_axes = []
    replication_size = 1
    total_mesh_size = 1
    for d, sz in enumerate(dims):
        if device_axes_used[d] == 0:
            replicated_device_axes.append(d)
            replication_size *= sz
        total_mesh_size *= sz

    tile_dims = [1] * num_logical_dims
    dim_permutation: List[int] = []
    for ld in range(num_logical_dims):
        assigned = sorted(logical_to_device_axes[ld])
        t = 1
        for ax in assigned:
            t *= dims[ax]
            dim_permutation.append(ax)
        tile_dims[ld] = t
    for d in range(len(dims)):
        if not device_axes_used[d]:
            dim_permutation.append(d)
    if replicated_device_axes:
        tile_dims.append(replication_size)

    need_permutation = any(i != p for i, p in enumerate(dim_permutation))
    op = OpSharding(type="OTHER", tile_assignment_dimensions=tile_dims)
    if need_permutation:
        op.iota_transpose_perm = list(dim_permutation)
        op.iota_reshape_dims = list(dims)
    else:
        op.iota_reshape_dims = [total_mesh_size]
        op.iota_transpose_perm = [0]
    op.replicate_on_last_tile_dim = bool(replicated_device_axes)
    op.iota_offset = devices[0]
    return op


# --------------------------------------------------------------------------
# mpmd_logical_to_gspmd_sharding.cc:21-124
# --------------------------------------------------------------------------
def logical_sharding_to_op_sharding(mesh_dims: Sequence[int], mesh_axes: Sequence[str],
                                    logical_axes: Sequence[Tuple[str, str]],
                                    logical_axis_names: Sequence[Sequence[str]], shape: Sequence[int],
                                    devices: Tuple[int, int], total_devices: int) -> OpSharding:
    """PartitionSpec-style logical axis names of one array -> OpSharding, the way a
    task's options (mesh dims, mesh axis names, ordered logical->device axis
    pairs) resolve them.  Pinned by the closed form it reduces to: the result is
    logical_to_physical_sharding of the resolved device axes, and non-divisible
    shardings are rejected (:101-113)."""
    n = len(logical_axis_names)
    to_device: List[List[int]] = [[] for _ in range(n)]
    used = set()
    sharding_on_axis = [1] * n
    for logical_ax, device_ax in logical_axes:
        for idx, names in enumerate(logical_axis_names):
            for name in names:
                if name == logical_ax:
                    if device_ax not in mesh_axes:
                        raise ShardingError("unknown device axis '%s' in autosharding" % device_ax)
                    di = list(mesh_axes).index(device_ax)
                    total = sharding_on_axis[idx] * mesh_dims[di]
                    if total <= shape[idx] and di not in used:
                        to_device[idx].append(di)
                        used.add(di)
                        sharding_on_axis[idx] = total
                    break
    list_all = devices[1] < total_devices
    op = logical_to_physical_sharding(to_device, devices, mesh_dims, list_all)
    if op.type == "OTHER":
        for d in range(len(shape)):
            if shape[d] % op.tile_assignment_dimensions[d]:
                raise ShardingError("sharding does not evenly divide shape")
    return op


# --------------------------------------------------------------------------
# mm_sharding.cc:275-456
# --------------------------------------------------------------------------
def _canonicalize_iota(
    op: OpSharding,
    ta_dims: Sequence[int],
    reshape_dims: Sequence[int],
    transpose_perm: Sequence[int],
    offset: int,
    shape_dims: Sequence[int],
    element_type: str,
    shape_is_global: bool,
) -> ShardedShape:
    # :284-295
    if not transpose_perm:
        permuted_reshape_dims = list(reshape_dims)
    else:
        permuted_reshape_dims = [reshape_dims[p] for p in transpose_perm]

    # :297-325  un-group tile dims that one iota dim spans
    dimension_groups: List[List[int]] = [[]]
    iota_dim = 0
    spanned = 1
    ta_dim = 0
    while ta_dim < len(ta_dims) and iota_dim < len(permuted_reshape_dims):
        spanned *= ta_dims[ta_dim]
        iota_group_span = permuted_reshape_dims[iota_dim]
        if iota_group_span < ta_dims[ta_dim]:
            raise ShardingError(
                "CanonicalizeSharding: multiple iota dims within a single "
                "tensor dimension, which is not yet supported")
        dimension_groups[-1].append(ta_dim)
        if spanned >= iota_group_span:
            iota_dim += 1
            if iota_dim < len(permuted_reshape_dims):
                dimension_groups.append([])
            spanned = 1
        ta_dim += 1
    while ta_dim < len(ta_dims):
        dimension_groups[-1].append(ta_dim)
        ta_dim += 1

    # :327-339  the reference indexes the groups with transpose_perm itself
    permuted_groups: List[List[int]] = [[] for _ in dimension_groups]
    for k, src_dim in enumerate(transpose_perm):
        permuted_groups[k] = dimension_groups[src_dim]
    full_permutation = [d for g in permuted_groups for d in g]

    # :341-369
    num_shape_dims = len(ta_dims) - 1 if op.replicate_on_last_tile_dim else len(ta_dims)
    dims: List[Optional[ShardingDim]] = [None] * len(ta_dims)
    perm_dim = 0
    for k in range(len(full_permutation)):
        tdim = full_permutation[k]
        extent = ta_dims[tdim]
        if tdim == num_shape_dims:
            size, shard = 1, extent
        else:
            size = shape_dims[tdim]
            if not shape_is_global:
                size *= extent
            shard = extent
        dims[tdim] = ShardingDim(size=size, sharding=shard, permutation=perm_dim)
        perm_dim += 1
    if any(d is None for d in dims):
        raise ShardingError("CanonicalizeSharding: tile dimension left without a descriptor")

    n = 1
    for r in reshape_dims:
        n *= r
    if element_type not in SUPPORTED_TYPES:  # :376-425
        raise ShardingError("Unsupported type: %s" % element_type)
    return ShardedShape(type=element_type, dims=tuple(dims), dev_start=offset, dev_count=n)


def canonicalize_sharding(op: OpSharding, shape_dims: Sequence[int],
                          element_type: str, shape_is_global: bool = True) -> ShardedShape:
    ta_dims = list(op.tile_assignment_dimensions)
    if op.has_iota:  # :438-441
        reshape_dims, perm = canonical_iota(op.iota_reshape_dims, op.iota_transpose_perm)
        return _canonicalize_iota(op, ta_dims, reshape_dims, perm, op.iota_offset,
                                  shape_dims, element_type, shape_is_global)
    # :443-455  an explicit list is accepted only if it is consecutive
    devs = list(op.tile_assignment_devices)
    prev = devs[0] - 1
    for d in devs:
        if d != prev + 1:
            raise ShardingError("CanonicalizeSharding: only supported for iota tile assignment")
        prev = d
    return _canonicalize_iota(op, ta_dims, [len(devs)], [0], devs[0],
                              shape_dims, element_type, shape_is_global)


# --------------------------------------------------------------------------
# mm_sharding.cc:583-671
# --------------------------------------------------------------------------
def xla_shape_to_zuku_shape(shape_dims: Sequence[int], element_type: str,
                            devices: Tuple[int, int], op: OpSharding,
                            shape_is_global: bool = True) -> ShardedShape:
    if element_type not in SUPPORTED_TYPES:  # :586-636
        raise ShardingError("Unsupported type: %s" % element_type)
    if op.is_replicated or op.is_tile_maximal:  # :638-654
        dims = [ShardingDim(size=s, sharding=1, permutation=i)
                for i, s in enumerate(shape_dims)]
        if devices[1] > 1:
            dims.append(ShardingDim(size=1, sharding=devices[1], permutation=len(shape_dims)))
        return ShardedShape(type=element_type, dims=tuple(dims),
                            dev_start=devices[0], dev_count=devices[1])
    ss = canonicalize_sharding(op, shape_dims, element_type, shape_is_global)
    if (ss.dev_start, ss.dev_count) != tuple(devices):  # :659-668
        if ss.dev_count != devices[1]:
            raise ShardingError("devices given to XlaShapeToZukuShape differ from sharding")
        ss = ShardedShape(type=ss.type, dims=ss.dims, dev_start=devices[0], dev_count=devices[1])
    return ss


# --------------------------------------------------------------------------
# mm_sharding.cc:19-51 and mpmd_insert_reshard.cc:33-43
# --------------------------------------------------------------------------
def is_replicated_on_assigned_submesh(op: OpSharding) -> bool:
    if op.is_replicated:
        return True
    if op.replicate_on_last_tile_dim:
        return all(d == 1 for d in op.tile_assignment_dimensions[:-1])
    return False


def is_replicated_or_submesh_replicate(op: OpSharding) -> bool:
    return op.is_replicated or is_replicated_on_assigned_submesh(op) or op.is_tile_maximal


def mesh_equivalent_sharding(lhs: OpSharding, rhs: OpSharding) -> bool:
    if is_replicated_or_submesh_replicate(lhs):
        return is_replicated_or_submesh_replicate(rhs)
    if is_replicated_or_submesh_replicate(rhs):
        return False
    return list(lhs.tile_assignment_dimensions) == list(rhs.tile_assignment_dimensions)


def device_list_contains(outer: Tuple[int, int], inner: Tuple[int, int]) -> bool:
    """zuku::DeviceList::Contains(list): the contiguous range holds the other range."""
    return outer[0] <= inner[0] and inner[0] + inner[1] <= outer[0] + outer[1]


def needs_reshard(operand_devices: Tuple[int, int], devices: Tuple[int, int],
                  operand_sharding: OpSharding, sharding: OpSharding) -> bool:
    if (operand_sharding.is_replicated and sharding.is_replicated
            and device_list_contains(operand_devices, devices)):
        return False
    return tuple(operand_devices) != tuple(devices) or not mesh_equivalent_sharding(
        operand_sharding, sharding)


def to_mpmd_sharding(rank: int, sharding: OpSharding, task_devices: Tuple[int, int],
                     global_devices: Tuple[int, int]) -> OpSharding:
    """mpmd_partition.cc:128-166.  `sharding` is written relative to the task's devices (ids 0..n-1); the result
    names global device ids.  Device ranges are (start, count)."""
    t_start, t_count = task_devices
    if sharding.type == "REPLICATED" and tuple(task_devices) == tuple(global_devices):   # :132-134
        return OpSharding(type="REPLICATED")
    if t_count == 1 and sharding.type in ("MAXIMAL", "REPLICATED"):                       # :136-139
        return OpSharding(type="MAXIMAL", tile_assignment_devices=[t_start])
    if sharding.type == "REPLICATED" and rank > 0:                                         # :152-163
        return OpSharding(type="OTHER", tile_assignment_dimensions=[1] * rank + [t_count], iota_reshape_dims=[t_count],
                          iota_transpose_perm=[0], replicate_on_last_tile_dim=True, iota_offset=t_start)
    out = OpSharding(type=sharding.type, tile_assignment_dimensions=list(sharding.tile_assignment_dimensions),
                     iota_reshape_dims=list(sharding.iota_reshape_dims),
                     iota_transpose_perm=list(sharding.iota_transpose_perm),
                     replicate_on_last_tile_dim=sharding.replicate_on_last_tile_dim, iota_offset=sharding.iota_offset)
    if sharding.has_iota:
        out.iota_offset = t_start                                                          # :143-144
    else:
        for rel in sharding.tile_assignment_devices:                                        # :145-150
            if not 0 <= rel < t_count:
                raise ShardingError("relative device id %d outside the task's %d devices" % (rel, t_count))
        out.tile_assignment_devices = [t_start + rel for rel in sharding.tile_assignment_devices]
    return out


def replicate_dims(replicated_dims: Sequence[int], sharding: OpSharding) -> OpSharding:
    """mm_sharding.cc:458-582.  Moves the tiling of `replicated_dims` (tile-assignment dims) into the trailing
    replication dim.  The reference walks the HloSharding's iota, i.e. XLA's canonical form of it."""
    if not sharding.has_iota:                                                               # :465-468
        raise ShardingError("ReplicateDims only supported for iota tile assignment")
    ta = list(sharding.tile_assignment_dimensions)
    reshape, perm = canonical_iota(sharding.iota_reshape_dims, sharding.iota_transpose_perm)
    # :476-514  un-group the iota dims into tile-assignment dims, then order the groups as the transpose does
    groups: List[List[int]] = [[]]
    iota_dim, spanned, ta_dim = 0, 1, 0
    while ta_dim < len(ta) and iota_dim < len(perm):
        spanned *= ta[ta_dim]
        span = reshape[perm[iota_dim]]
        groups[-1].append(ta_dim)
        if spanned >= span:
            iota_dim += 1
            if iota_dim < len(perm):
                groups.append([])
            spanned = 1
        ta_dim += 1
    groups[-1].extend(range(ta_dim, len(ta)))
    if len(groups) != len(perm):
        raise ShardingError("iota dims do not group into tile assignment dims")
    current = [d for src in perm for d in groups[src]]
    # :516-540
    new_reshape = [ta[d] for d in current] + [1] * len(replicated_dims)
    num_shape_dims = len(ta) - 1 if sharding.replicate_on_last_tile_dim else len(ta)
    new_perm = list(current)
    extra = len(new_perm)
    for dim in replicated_dims:
        new_perm.append(current[dim])
        new_perm[dim] = extra
        extra += 1
    total = ta[num_shape_dims] if sharding.replicate_on_last_tile_dim else 1               # :542-552
    for dim in replicated_dims:
        total *= ta[dim]
    n = 1
    for d in ta:
        n *= d
    if total == n:                                                                          # :554-557
        return OpSharding(type="REPLICATED")
    ta_dims = list(ta)                                                                      # :559-571
    if sharding.replicate_on_last_tile_dim:
        ta_dims[num_shape_dims] = total
    else:
        ta_dims.append(total)
    for dim in replicated_dims:
        ta_dims[dim] = 1
    return OpSharding(type="OTHER", tile_assignment_dimensions=ta_dims, iota_reshape_dims=new_reshape,
                      iota_transpose_perm=new_perm, replicate_on_last_tile_dim=True,
                      iota_offset=sharding.iota_offset)


def resize_sharding(shape_dims: Sequence[int], sharding: OpSharding, num_elements: int,
                    devices: Optional[Tuple[int, int]] = None) -> Optional[OpSharding]:
    """mm_sharding.cc:98-161.  Grows or shrinks the first tiled dim that can take it so that the tile assignment
    has `num_elements` tiles; None where the reference returns nullopt.  `devices` = (start, count) or None."""
    if sharding.has_iota:                                                                   # :101-109
        _, perm = canonical_iota(sharding.iota_reshape_dims, sharding.iota_transpose_perm)
        if any(i != p for i, p in enumerate(perm)):
            return None
    ta = list(sharding.tile_assignment_dimensions)
    src_size = 1
    for d in ta:
        src_size *= d
    dst_size = num_elements
    dims: List[int] = []
    replicate_last = False
    matched = False
    for dim, old in enumerate(ta):                                                          # :120-142
        new = old * dst_size // src_size
        if not matched and old > 1 and new > 0 and new <= shape_dims[dim]:
            if (src_size > dst_size and src_size % dst_size) or (src_size < dst_size and dst_size % src_size):
                continue
            dims.append(new)
            matched = True
        else:
            dims.append(old)
        # (the reference indexes the dims written so far by `dim`; after a skipped dim no match can follow, since the
        # divisibility test that skips does not depend on the dim, and the result is nullopt either way)
        if dim == len(ta) - 1 and sharding.replicate_on_last_tile_dim and len(dims) == dim + 1 and dims[dim] > 1:
            replicate_last = True
    if not matched:
        return None
    out = OpSharding(type="OTHER", tile_assignment_dimensions=dims, replicate_on_last_tile_dim=replicate_last)
    if sharding.has_iota or devices is None:                                                # :144-150
        out.iota_reshape_dims = [num_elements]
        out.iota_transpose_perm = [0]
        if devices is not None:
            out.iota_offset = devices[0]
    else:                                                                                   # :151-154
        out.tile_assignment_devices = list(range(devices[0], devices[0] + devices[1]))
    # HloSharding::FromProto (XLA) refuses a tile assignment whose tile count differs from its device count
    n = 1
    for d in dims:
        n *= d
    count = num_elements if out.has_iota else len(out.tile_assignment_devices)
    if n != count:
        return None
    return out
