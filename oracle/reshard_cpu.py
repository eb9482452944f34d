"""ctypes loader of the C restatement (oracle/reshard_cpu.c).

TEST INFRASTRUCTURE ONLY: used by tests/, smoke() and bench.py's cpu_baseline leg.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Dict, Optional, Sequence

import numpy as np

from .reshard_oracle import ITEMSIZE
from .sharding_oracle import ShardedShape

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libreshard_oracle.so")
ORC_MAX_DIMS = 9


class OrcDesc(ctypes.Structure):
    _fields_ = [
        ("itemsize", ctypes.c_int32),
        ("ndims", ctypes.c_int32),
        ("size", ctypes.c_int64 * ORC_MAX_DIMS),
        ("sharding", ctypes.c_int64 * ORC_MAX_DIMS),
        ("permutation", ctypes.c_int64 * ORC_MAX_DIMS),
        ("dev_start", ctypes.c_int64),
        ("dev_count", ctypes.c_int64),
        ("has_layout", ctypes.c_int32),
        ("minor_to_major", ctypes.c_int32 * ORC_MAX_DIMS),
    ]


def build() -> str:
    """Compile the C restatement (gcc); returns the library path."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "-B", "libreshard_oracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_reshard.restype = ctypes.c_int
        _lib.orc_reshard.argtypes = [
            ctypes.POINTER(OrcDesc), ctypes.POINTER(ctypes.c_void_p),
            ctypes.POINTER(OrcDesc), ctypes.POINTER(ctypes.c_void_p), ctypes.c_int]
    return _lib


def to_desc(ss: ShardedShape, minor_to_major: Optional[Sequence[int]] = None) -> OrcDesc:
    d = OrcDesc()
    d.itemsize = ITEMSIZE[ss.type]
    d.ndims = len(ss.dims)
    for i, dim in enumerate(ss.dims):
        d.size[i] = dim.size
        d.sharding[i] = dim.sharding
        d.permutation[i] = dim.permutation
    d.dev_start = ss.dev_start
    d.dev_count = ss.dev_count
    if minor_to_major is not None:
        d.has_layout = 1
        for i, m in enumerate(minor_to_major):
            d.minor_to_major[i] = m
    return d


def reshard(src_shards: Dict[int, np.ndarray], src: ShardedShape, dst: ShardedShape,
            dst_shards: Dict[int, np.ndarray], nthreads: int = 1,
            src_minor_to_major: Optional[Sequence[int]] = None,
            dst_minor_to_major: Optional[Sequence[int]] = None) -> None:
    """Fill the preallocated flat `dst_shards` buffers (device id -> array) in place."""
    sd, dd = to_desc(src, src_minor_to_major), to_desc(dst, dst_minor_to_major)
    sp = (ctypes.c_void_p * src.dev_count)(
        *[src_shards[src.dev_start + k].ctypes.data for k in range(src.dev_count)])
    dp = (ctypes.c_void_p * dst.dev_count)(
        *[dst_shards[dst.dev_start + k].ctypes.data for k in range(dst.dev_count)])
    rc = lib().orc_reshard(ctypes.byref(sd), sp, ctypes.byref(dd), dp, int(nthreads))
    if rc != 0:
        raise ValueError("orc_reshard rejected the descriptor pair (code %d)" % rc)
