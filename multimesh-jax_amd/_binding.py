"""ctypes view of include/mmreshard.h (the C ABI of libmmreshard.so).

There is no Python or CPU fallback behind these calls: if the library is
missing, loading fails; if no GPU is present, mmr_context_create fails.
"""
from __future__ import annotations

import ctypes as C
import os

MMR_MAX_DIMS = 9
MMR_SLOT_FILL = 0xFFFFFFFF
MMR_STORE_FROM_CACHE = 1
MMR_STORE_UNINITIALIZED = 2
MMR_PLAN_ALL_GENERIC, MMR_PLAN_NO_AUTOTUNE, MMR_PLAN_NO_SPAN = 1, 2, 4
MMR_PLAN_NO_INLINE, MMR_PLAN_NO_SEGMENT_TABLES = 8, 16
MMR_CHECK_INVARIANTS = 1
MMR_STATIC_SCRATCH_BYTES = 1 << 20

STATUS_NAMES = {0: "OK", 1: "INVALID_ARGUMENT", 2: "UNSUPPORTED", 3: "OUT_OF_MEMORY",
                4: "HIP_ERROR", 5: "NOT_FOUND", 6: "INTERNAL"}

DTYPES = {
    "PRED": 0, "F16": 1, "BF16": 2, "F32": 3, "F64": 4, "S8": 5, "S16": 6, "S32": 7, "S64": 8,
    "U8": 9, "U16": 10, "U32": 11, "U64": 12, "C64": 13, "C128": 14,
    "F8E4M3FN": 100, "F8E5M2": 101,
}
DTYPE_NAMES = {v: k for k, v in DTYPES.items()}

SHARDING_TYPES = {"REPLICATED": 0, "MAXIMAL": 1, "OTHER": 3}
SHARDING_TYPE_NAMES = {v: k for k, v in SHARDING_TYPES.items()}


class ShardingDim(C.Structure):
    _fields_ = [("size", C.c_int64), ("sharding", C.c_int64), ("permutation", C.c_int64)]


class ShardedShape(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32), ("ndims", C.c_int32),
        ("dims", ShardingDim * MMR_MAX_DIMS),
        ("dev_start", C.c_int64), ("dev_count", C.c_int64),
        ("has_layout", C.c_int32), ("minor_to_major", C.c_int32 * MMR_MAX_DIMS),
    ]


class OpSharding(C.Structure):
    _fields_ = [
        ("type", C.c_int32), ("n_tile_dims", C.c_int32),
        ("tile_dims", C.c_int64 * MMR_MAX_DIMS),
        ("n_iota_dims", C.c_int32),
        ("iota_reshape_dims", C.c_int64 * MMR_MAX_DIMS),
        ("iota_transpose_perm", C.c_int32 * MMR_MAX_DIMS),
        ("replicate_on_last_tile_dim", C.c_int32),
        ("iota_offset", C.c_int64),
        ("tile_assignment_devices", C.POINTER(C.c_int64)),
        ("n_devices", C.c_int64),
    ]


class CopyChunk(C.Structure):
    _fields_ = [
        ("src_slot", C.c_uint32), ("dst_slot", C.c_uint32),
        ("src_off", C.c_uint64), ("dst_off", C.c_uint64),
        ("w", C.c_uint32), ("n1", C.c_uint32), ("n2", C.c_uint32), ("align", C.c_uint32),
        ("s1", C.c_int64), ("d1", C.c_int64), ("s2", C.c_int64), ("d2", C.c_int64),
    ]


class TransposeChunk(C.Structure):
    _fields_ = [
        ("src_slot", C.c_uint32), ("dst_slot", C.c_uint32),
        ("src_off", C.c_uint64), ("dst_off", C.c_uint64),
        ("nx", C.c_uint32), ("ny", C.c_uint32), ("nb", C.c_uint32), ("itemsize", C.c_uint32),
        ("src_ystride", C.c_int64), ("dst_xstride", C.c_int64),
        ("src_bstride", C.c_int64), ("dst_bstride", C.c_int64),
    ]


class PlanOptions(C.Structure):
    _fields_ = [("chunk_bytes", C.c_uint32), ("order", C.c_uint32), ("xcd_mode", C.c_uint32),
                ("flags", C.c_uint32)]


class PlanStats(C.Structure):
    _fields_ = [(n, C.c_int64) for n in (
        "n_arrays", "n_boxes", "n_copy16_chunks", "n_span_chunks", "n_groups", "n_pieces", "n_copy_generic_chunks",
        "n_transpose_chunks",
        "n_fill_chunks", "bytes_moved", "bytes_filled", "table_bytes", "n_slots", "order_used", "interleave_kib",
        "orders_timed", "n_copy16_launches")]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


class ContextStats(C.Structure):
    _fields_ = [(n, C.c_int64) for n in (
        "plans_built", "plan_cache_hits", "bindings_built", "binding_cache_hits", "kernel_launches",
        "reshard_calls", "bytes_allocated", "bytes_high_watermark", "stores_live", "cache_hits",
        "host_bytes_allocated", "host_bytes_high_watermark", "host_blocking_syncs", "inline_launches",
        "device_allocations", "host_cache_hits", "pool_hits", "plans_cached", "bindings_cached", "invariant_checks",
        "operation_hash", "block_pool_hits", "timers_resolved", "windows_opened", "window_waits", "profile_marks", "events_recorded")]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


# Every symbol include/mmreshard.h declares: name -> (restype, argtypes)
P = C.POINTER
VP = C.c_void_p
I32, I64 = C.c_int32, C.c_int64
PROTOTYPES = {
    "mmr_last_error": (C.c_char_p, []),
    "mmr_version": (C.c_char_p, []),
    "mmr_itemsize": (C.c_int, [I32]),
    "mmr_compute_index_set": (C.c_int, [I64, P(I64), I32, P(I64)]),
    "mmr_compute_global_index": (C.c_int, [P(I64), P(I64), I32, P(I64)]),
    "mmr_logical_to_physical_sharding": (C.c_int, [P(I32), P(I32), I32, I64, I64, P(I64), I32, I32, P(OpSharding)]),
    "mmr_logical_sharding_to_op_sharding": (C.c_int, [P(I64), P(C.c_char_p), I32, P(C.c_char_p), P(C.c_char_p), I32,
                                                      P(C.c_char_p), P(I32), I32, P(I64), I64, I64, I64, P(OpSharding)]),
    "mmr_tile_assignment_devices": (C.c_int, [P(OpSharding), P(I64), I64, P(I64)]),
    "mmr_canonicalize_sharding": (C.c_int, [P(OpSharding), P(I64), I32, I32, I32, P(ShardedShape)]),
    "mmr_xla_shape_to_sharded_shape": (C.c_int, [P(I64), I32, I32, I64, I64, P(OpSharding), I32, P(ShardedShape)]),
    "mmr_mesh_equivalent_sharding": (C.c_int, [P(OpSharding), P(OpSharding), P(I32)]),
    "mmr_needs_reshard": (C.c_int, [I64, I64, I64, I64, P(OpSharding), P(OpSharding), P(I32)]),
    "mmr_device_list_of_sharding": (C.c_int, [P(OpSharding), P(I64), P(I64)]),
    "mmr_to_mpmd_sharding": (C.c_int, [I32, P(OpSharding), I64, I64, I64, I64, P(OpSharding), P(I64), I64]),
    "mmr_replicate_dims": (C.c_int, [P(OpSharding), P(I64), I32, P(OpSharding)]),
    "mmr_resize_sharding": (C.c_int, [P(I64), I32, P(OpSharding), I64, I64, I64, P(OpSharding), P(I64), I64, P(I32)]),
    "mmr_validate_sharded_shape": (C.c_int, [P(ShardedShape)]),
    "mmr_shard_extents": (C.c_int, [P(ShardedShape), P(I64), P(I32)]),
    "mmr_shard_bytes": (C.c_int, [P(ShardedShape), P(I64)]),
    "mmr_device_of_tile": (C.c_int, [P(ShardedShape), P(I64), P(I64)]),
    "mmr_tile_of_device": (C.c_int, [P(ShardedShape), I64, P(I64)]),
    "mmr_plan_create": (C.c_int, [P(ShardedShape), P(ShardedShape), I32, P(PlanOptions), P(VP)]),
    "mmr_plan_destroy": (None, [VP]),
    "mmr_plan_get_stats": (C.c_int, [VP, P(PlanStats)]),
    "mmr_plan_get_copy_chunks": (I64, [VP, I32, P(CopyChunk), I64]),
    "mmr_plan_get_transpose_chunks": (I64, [VP, P(TransposeChunk), I64]),
    "mmr_plan_get_slot_bases": (I64, [VP, P(I64), I64]),
    "mmr_context_create": (C.c_int, [I32, VP, P(VP)]),
    "mmr_context_destroy": (None, [VP]),
    "mmr_context_stream": (C.c_int, [VP, P(VP)]),
    "mmr_context_set_plan_options": (C.c_int, [VP, P(PlanOptions)]),
    "mmr_store_create": (C.c_int, [VP, P(ShardedShape), C.c_char_p, C.c_uint32, P(VP)]),
    "mmr_store_create_ex": (C.c_int, [VP, P(ShardedShape), C.c_char_p, C.c_uint32, I64, P(VP)]),
    "mmr_context_set_flags": (C.c_int, [VP, C.c_uint32]),
    "mmr_context_clear_plans": (C.c_int, [VP]),
    "mmr_reshard_tune": (C.c_int, [VP, P(VP), P(VP), I32, P(I64)]),
    "mmr_store_adopt": (C.c_int, [VP, P(ShardedShape), C.c_char_p, P(VP), P(VP)]),
    "mmr_store_offload": (C.c_int, [VP, VP]),
    "mmr_store_reload": (C.c_int, [VP, VP]),
    "mmr_store_is_offloaded": (C.c_int, [VP, P(I32)]),
    "mmr_context_prepare": (C.c_int, [VP, P(ShardedShape), P(ShardedShape), I32]),
    "mmr_context_wait_event": (C.c_int, [VP, VP]),
    "mmr_context_record_event": (C.c_int, [VP, VP]),
    "mmr_store_free": (C.c_int, [VP, VP, I32]),
    "mmr_clear_store_cache": (C.c_int, [VP]),
    "mmr_store_assemble": (C.c_int, [VP, VP, I64, VP, C.c_size_t, I32]),
    "mmr_store_shard_ptr": (C.c_int, [VP, VP, I64, P(VP)]),
    "mmr_store_shard_ptr_async": (C.c_int, [VP, VP, I64, P(VP)]),
    "mmr_store_read_shard": (C.c_int, [VP, VP, I64, VP, C.c_size_t]),
    "mmr_store_has_shard": (C.c_int, [VP, I64, P(I32)]),
    "mmr_store_get_shape": (C.c_int, [VP, P(ShardedShape)]),
    "mmr_store_id": (I64, [VP]),
    "mmr_reshard": (C.c_int, [VP, VP, VP]),
    "mmr_reshard_batch": (C.c_int, [VP, P(VP), P(VP), I32]),
    "mmr_reshard_batch_static": (C.c_int, [VP, P(VP), P(VP), I32]),
    "mmr_reshard_bind": (C.c_int, [VP, P(VP), P(VP), I32]),
    "mmr_reshard_validate": (C.c_int, [VP, VP, VP]),
    "mmr_context_run_after": (C.c_int, [VP, C.CFUNCTYPE(None, VP), VP]),
    "mmr_sync": (C.c_int, [VP]),
    "mmr_timer_start": (C.c_int, [VP]),
    "mmr_timer_stop_wait": (C.c_int, [VP, P(C.c_float)]),
    "mmr_timer_begin": (C.c_int, [VP, C.c_char_p]),
    "mmr_timer_end": (C.c_int, [VP, C.c_char_p]),
    "mmr_timer_poll": (C.c_int, [VP, C.c_char_p, P(C.c_float), P(I64)]),
    "mmr_timer_wait": (C.c_int, [VP, C.c_char_p, P(C.c_float), P(I64)]),
    "mmr_profile_mark": (C.c_int, [VP, C.c_char_p]),
    "mmr_profile_range_push": (C.c_int, [VP, C.c_char_p]),
    "mmr_profile_range_pop": (C.c_int, [VP]),
    "mmr_profile_available": (C.c_int, []),
    "mmr_window_open": (C.c_int, [VP]),
    "mmr_window_close": (C.c_int, [VP]),
    "mmr_context_set_max_open_windows": (C.c_int, [VP, I32]),
    "mmr_timer_lap": (C.c_int, [VP]),
    "mmr_timer_laps": (C.c_int, [VP, P(C.c_float), I32, P(I32)]),
    "mmr_context_get_stats": (C.c_int, [VP, P(ContextStats)]),
    "mmr_reshard_plan_stats": (C.c_int, [VP, VP, VP, P(PlanStats)]),
    "mmr_reshard_batch_plan_stats": (C.c_int, [VP, P(VP), P(VP), I32, P(PlanStats)]),
}

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libmmreshard.so")


class MmrError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__("%s: %s" % (STATUS_NAMES.get(status, status), message))
        self.status = status
        self.status_name = STATUS_NAMES.get(status, str(status))


_lib = None


def source_digest():
    """Digest of the sources next to this file, computed as csrc/build.sh does; None where they are not there."""
    import hashlib
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    names = sorted([os.path.join("include", n) for n in os.listdir(os.path.join(root, "include")) if n.endswith(".h")]
                   + [os.path.join("multimesh-jax_amd", "csrc", n)
                      for n in os.listdir(os.path.join(root, "multimesh-jax_amd", "csrc"))]) \
        if os.path.isdir(os.path.join(root, "include")) and os.path.isdir(os.path.join(root, "multimesh-jax_amd", "csrc")) else None
    if not names:
        return None
    h = hashlib.sha256()
    for n in names:
        h.update(n.encode() + b"\n")
        with open(os.path.join(root, n), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def load():
    """Loads libmmreshard.so and types every entry point. Raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with multimesh-jax_amd/csrc/build.sh (hipcc, gfx950); "
                "there is no fallback implementation" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        built_from = lib.mmr_version().decode().rsplit(" ", 1)[-1]
        here = source_digest()
        if here is not None and built_from != here:
            raise ImportError(
                "%s was built from other sources (digest %s) than the ones next to it (%s): rebuild it with "
                "multimesh-jax_amd/csrc/build.sh" % (LIB_PATH, built_from, here))
        _lib = lib
    return _lib


def check(status: int) -> None:
    if status != 0:
        raise MmrError(status, load().mmr_last_error().decode("utf-8", "replace"))
