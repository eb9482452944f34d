"""GPU-side test helpers: run a list of workload arrays through the C ABI on the
GPU and hand back every destination shard."""
from __future__ import annotations

from typing import Dict, List, Sequence

import numpy as np

import multimesh_jax_amd as mm
from oracle import reshard_oracle as ro

from helpers import lib_shape, oracle_shape, raw_global


def make_stores(ctx, arrays: Sequence[dict], globals_: Sequence[np.ndarray], poison: int = 0x5A):
    """Creates and fills the source stores; creates destination stores whose
    buffers are pre-filled with `poison` so untouched bytes show."""
    srcs, dsts = [], []
    for a, g in zip(arrays, globals_):
        so = oracle_shape(a["type"], a["src"])
        shards = ro.make_shards(raw_global(a, g), so, a["src"].get("minor_to_major"))
        s_shape = lib_shape(a["type"], a["src"])
        store = ctx.CreateStore(s_shape, name=a["name"] + ".src")
        for dev in store.devices:
            ctx.AssembleShards(s_shape, dev, shards[dev].view(np.uint8).reshape(-1), existing_store=store)
        srcs.append(store)
        d_shape = lib_shape(a["type"], a["dst"])
        dstore = ctx.CreateStore(d_shape, name=a["name"] + ".dst")
        if poison is not None and dstore.shard_bytes:
            junk = np.full(dstore.shard_bytes, poison, dtype=np.uint8)
            for dev in dstore.devices:
                ctx.AssembleShards(d_shape, dev, junk, existing_store=dstore)
        dsts.append(dstore)
    return srcs, dsts


def read_all(ctx, store) -> Dict[int, np.ndarray]:
    return {dev: ctx.ReadShard(store, dev) for dev in store.devices}


def gpu_reshard(ctx, arrays: Sequence[dict], globals_: Sequence[np.ndarray], batch: bool = True,
                keep: bool = False):
    srcs, dsts = make_stores(ctx, arrays, globals_)
    if batch and len(arrays) > 1:
        ctx.ReshardBatch(srcs, dsts)
    else:
        for s, d in zip(srcs, dsts):
            ctx.Reshard(s, d)
    ctx.Sync()
    outs = [read_all(ctx, d) for d in dsts]
    if keep:
        return outs, srcs, dsts
    for s in srcs + dsts:
        ctx.Free(s)
    return outs
