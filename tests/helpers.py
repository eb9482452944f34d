"""Shared test helpers: conversions between the neutral workload dicts, the
oracle's descriptors and the library's, and a NumPy interpreter of plan tables
(so the planner can be checked against the oracle without a GPU)."""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import numpy as np

import multimesh_jax_amd as mm
from oracle import reshard_oracle as ro
from oracle.sharding_oracle import ShardedShape, ShardingDim


def test_config(index: int, scale: int = 1):
    """The benchmark configurations of the package plus ragged shapes only the tests use."""
    from multimesh_jax_amd import workloads as w

    def one(name, type_, shape, src_tiles, dst_tiles, seed):
        return [{"name": name, "type": type_, "shape": shape, "src": w.side(shape, src_tiles, 0),
                 "dst": w.side(shape, dst_tiles, 3), "seed": seed, "dist": "raw"}]
    if index == 7:  # 4-byte elements, uneven 3-way -> 5-way (dword-aligned, not 16-byte-aligned runs)
        return one("ragged_s32", "S32", (11008 // scale, 1025), (1, 3), (1, 5), 7)
    if index == 8:  # 2-byte elements, uneven 3-way -> 5-way
        return one("ragged_u16", "U16", (11008 // scale, 2051), (1, 3), (1, 5), 8)
    if index == 10:  # configuration 5's fp8 array with 8 times the rows
        return one("ragged_fp8_big", "F8E4M3FN", (88064 // scale, 4099), (1, 3), (1, 5), 6)
    if index == 11:  # ragged rows, every destination row from one source tile
        return one("ragged_fp8_1to5", "F8E4M3FN", (44032 // scale, 4099), (1, 1), (1, 5), 6)
    return w.config(index, scale)


test_config.__test__ = False  # a helper, not a test


def oracle_shape(type: str, side: dict) -> ShardedShape:
    return ShardedShape(type, tuple(ShardingDim(*d) for d in side["dims"]), side["dev_start"], side["dev_count"])


def lib_shape(type: str, side: dict):
    return mm.sharded_shape(type, side["dims"], side["dev_start"], side["dev_count"], side.get("minor_to_major"))


def raw_global(a: dict, g: np.ndarray) -> np.ndarray:
    return g.view(ro.raw_dtype(a["type"]))


def apply_plan(plan: "mm.Plan", buffers: Sequence[np.ndarray]) -> None:
    """Executes a plan's tables on host buffers (one flat uint8 array per slot)
    exactly as the kernels define a chunk; pure NumPy, for CPU-side checks."""
    for kind in (0, 1, 2):  # copy-group chunks as decoded, generic chunks, the row pieces of the span groups
        for c in plan.copy_chunks(kind):
            dst = buffers[int(c["dst_slot"])]
            fill = int(c["src_slot"]) == 0xFFFFFFFF
            src = None if fill else buffers[int(c["src_slot"])]
            w = int(c["w"])
            if kind == 0:
                assert int(c["align"]) == 16
            for r2 in range(int(c["n2"])):
                for r1 in range(int(c["n1"])):
                    do = int(c["dst_off"]) + r2 * int(c["d2"]) + r1 * int(c["d1"])
                    assert do + w <= dst.size
                    if fill:
                        dst[do:do + w] = 0
                    else:
                        so = int(c["src_off"]) + r2 * int(c["s2"]) + r1 * int(c["s1"])
                        assert so + w <= src.size
                        dst[do:do + w] = src[so:so + w]
            a = int(c["align"])
            for v in ("dst_off", "w", "d1", "d2") + (() if fill else ("src_off", "s1", "s2")):
                assert int(c[v]) % a == 0, (v, c)
    for c in plan.transpose_chunks():
        src = buffers[int(c["src_slot"])]
        dst = buffers[int(c["dst_slot"])]
        it = int(c["itemsize"])
        edge = {1: 128, 16: 32}.get(it, 64)
        assert int(c["nx"]) <= edge and int(c["ny"]) <= edge
        for b in range(int(c["nb"])):
            for y in range(int(c["ny"])):
                for x in range(int(c["nx"])):
                    so = int(c["src_off"]) + b * int(c["src_bstride"]) + y * int(c["src_ystride"]) + x * it
                    do = int(c["dst_off"]) + b * int(c["dst_bstride"]) + x * int(c["dst_xstride"]) + y * it
                    dst[do:do + it] = src[so:so + it]


_emu = {}
EMULATION_VARIANT = ""  # "_span_options": the build with the span kernel's two optional variations switched on


def emulation_lib():
    """tests/cpp/libmmr_emulation.so: the kernels' own per-chunk code compiled for the host with bounds checks."""
    if EMULATION_VARIANT not in _emu:
        import ctypes as C
        import os
        import subprocess
        here = os.path.dirname(os.path.abspath(__file__))
        path = os.path.join(here, "cpp", "libmmr_emulation%s.so" % EMULATION_VARIANT)
        if not os.path.exists(path):
            subprocess.check_call(["bash", os.path.join(here, "cpp", "build.sh")])
        lib = C.CDLL(path)
        lib.mmr_emulate_plan.restype = C.c_int
        lib.mmr_emulate_plan.argtypes = [C.c_void_p, C.POINTER(C.c_void_p), C.POINTER(C.c_size_t), C.c_int64,
                                         C.c_uint32, C.c_int, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64),
                                         C.c_char_p, C.c_size_t]
        _emu[EMULATION_VARIANT] = lib
    return _emu[EMULATION_VARIANT]


def _aligned_copy(buf: np.ndarray) -> np.ndarray:
    """A 64-byte aligned uint8 copy of buf (device buffers are at least that aligned)."""
    raw = np.empty(buf.size + 64, dtype=np.uint8)
    off = (-raw.ctypes.data) % 64
    out = raw[off:off + buf.size]
    out[...] = buf
    return out


def emulate_plan(plan: "mm.Plan", buffers: Sequence[np.ndarray], xcd_mode: int = 0, shape: int = 0):
    """Runs the plan through the kernels' per-chunk routines on the host, in
    place on aligned copies of `buffers`, and copies the results back.
    Raises on any out-of-bounds or misaligned access.  Returns (loaded, stored) bytes."""
    import ctypes as C
    lib = emulation_lib()
    work = [_aligned_copy(b) for b in buffers]
    ptrs = (C.c_void_p * len(work))(*[w.ctypes.data for w in work])
    sizes = (C.c_size_t * len(work))(*[w.size for w in work])
    err = C.create_string_buffer(512)
    loaded, stored = C.c_uint64(), C.c_uint64()
    rc = lib.mmr_emulate_plan(plan._h, ptrs, sizes, len(work), xcd_mode, shape, C.byref(loaded), C.byref(stored),
                              err, 512)
    if rc != 0:
        raise AssertionError("kernel emulation: " + err.value.decode())
    for b, w in zip(buffers, work):
        b[...] = w
    return loaded.value, stored.value


def run_plan_on_host(arrays: Sequence[dict], globals_: Sequence[np.ndarray], chunk_bytes: int = 0,
                     order: int = 0, poison: int = 0xA5, engine: str = "numpy", xcd_mode: int = 0, shape: int = 0):
    """Returns (plan, per-array dict device -> uint8 dst buffer) after interpreting
    the batch plan on host copies of the shards."""
    srcs = [lib_shape(a["type"], a["src"]) for a in arrays]
    dsts = [lib_shape(a["type"], a["dst"]) for a in arrays]
    plan = mm.Plan(srcs, dsts, chunk_bytes=chunk_bytes, order=order)
    bases = plan.slot_bases()
    buffers = [None] * plan.stats["n_slots"]
    outs = []
    for a, g, base in zip(arrays, globals_, bases):
        so = oracle_shape(a["type"], a["src"])
        do = oracle_shape(a["type"], a["dst"])
        shards = ro.make_shards(raw_global(a, g), so, a["src"].get("minor_to_major"))
        for k in range(so.dev_count):
            buffers[base + k] = shards[so.dev_start + k].view(np.uint8).reshape(-1)
        nbytes = int(np.prod(ro.shard_shape(do))) * ro.ITEMSIZE[a["type"]] if ro.shard_shape(do) else ro.ITEMSIZE[a["type"]]
        out = {}
        for k in range(do.dev_count):
            buf = np.full(nbytes, poison, dtype=np.uint8)
            buffers[base + so.dev_count + k] = buf
            out[do.dev_start + k] = buf
        outs.append(out)
    if engine == "numpy":
        apply_plan(plan, buffers)
    else:
        emulate_plan(plan, buffers, xcd_mode, shape)
    return plan, outs


def oracle_outputs(a: dict, g: np.ndarray) -> Dict[int, np.ndarray]:
    so = oracle_shape(a["type"], a["src"])
    do = oracle_shape(a["type"], a["dst"])
    shards = ro.make_shards(raw_global(a, g), so, a["src"].get("minor_to_major"))
    out = ro.reshard(shards, so, do, a["src"].get("minor_to_major"), a["dst"].get("minor_to_major"))
    return {d: v.view(np.uint8).reshape(-1) for d, v in out.items()}
