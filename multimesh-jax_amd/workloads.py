"""The five benchmark configurations of the reshard path as descriptor pairs plus
seeded synthetic inputs (host NumPy, raw bits).  Shared by the tests, the smoke
check and the benchmark; nothing here computes a reshard.

Every array is a dict:
  name, type, shape,
  src / dst: {"dims": [(size, sharding, permutation)...], "dev_start", "dev_count",
              "minor_to_major" (optional)},
  seed, dist ("uniform" | "normal" | "normal_002" | "int32000" | "fp8")
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np

ITEMSIZE = {"F32": 4, "BF16": 2, "S32": 4, "F8E4M3FN": 1, "U8": 1, "U16": 2, "U32": 4, "F64": 8, "C128": 16}


def _side(shape: Sequence[int], sharding: Sequence[int], dev_start: int, replication: int = 1,
          minor_to_major: Optional[Sequence[int]] = None) -> dict:
    """Row-major device order (the dim listed first is the most significant digit
    of the device id), replication entry last, as the reference's canonical
    descriptors come out for plain PartitionSpecs."""
    dims = [(int(s), int(t), i) for i, (s, t) in enumerate(zip(shape, sharding))]
    count = int(np.prod(sharding)) if len(sharding) else 1
    if replication > 1:
        dims.append((1, replication, len(shape)))
        count *= replication
    d = {"dims": dims, "dev_start": dev_start, "dev_count": count}
    if minor_to_major is not None:
        d["minor_to_major"] = list(minor_to_major)
    return d


def _array(name, type, shape, src, dst, seed, dist):
    return {"name": name, "type": type, "shape": tuple(int(s) for s in shape), "src": src, "dst": dst,
            "seed": seed, "dist": dist}


def config(index: int, scale: int = 1) -> List[dict]:
    """Arrays of benchmark configuration `index` (1..5).  scale > 1 divides the
    large extents so the same sharding structure runs in seconds on a CPU."""
    s = scale
    if index == 0:  # calibration: one device to one device, i.e. a plain copy of known size (512 MiB)
        shape = (8, 4096 // s, 8192 // s)
        return [_array("copy", "BF16", shape, _side(shape, (1, 1, 1), 0), _side(shape, (1, 1, 1), 1), 2, "normal")]
    if index == 1:  # fp32 [4096,4096]: rows 4-way on devices 0-3 -> 2x2 blocks on devices 4-7
        shape = (4096 // s, 4096 // s)
        return [_array("c1", "F32", shape, _side(shape, (4, 1), 0), _side(shape, (2, 2), 4), 1, "uniform")]
    if index == 2:  # bf16 [8,4096,8192]: hidden 8-way on 0-7 -> seq 4-way on 8-11
        shape = (8, 4096 // s, 8192 // s)
        return [_array("c2", "BF16", shape, _side(shape, (1, 1, 8), 0), _side(shape, (1, 4, 1), 8), 2, "normal")]
    if index == 3:  # bf16 [4,32,2048,128]: heads 4-way x 2 replicas on 0-7 -> seq 8-way stored [b,s,h,d] on 8-15
        shape = (4, 32, 2048 // s, 128)
        return [_array("c3", "BF16", shape, _side(shape, (1, 4, 1, 1), 0, replication=2),
                       _side(shape, (1, 1, 8, 1), 8, minor_to_major=(3, 1, 2, 0)), 3, "normal")]
    if index == 4:  # 24-layer decoder pytree: last dim 4-way on 0-3 -> first dim 8-way on 4-11
        d_model, ffn, vocab, layers = 2048 // s, 8192 // s, 32000 // s, 24
        arrays = []

        def add(name, shape):
            if len(shape) == 1:
                src, dst = _side(shape, (4,), 0), _side(shape, (8,), 4)
            else:
                src, dst = _side(shape, (1, 4), 0), _side(shape, (8, 1), 4)
            arrays.append(_array(name, "F32", shape, src, dst, 4, "normal_002"))

        for layer in range(layers):
            p = "layer%02d." % layer
            add(p + "ln1", (d_model,))
            for w in ("wq", "wk", "wv", "wo"):
                add(p + w, (d_model, d_model))
            add(p + "ln2", (d_model,))
            add(p + "w_in", (d_model, ffn))
            add(p + "w_out", (ffn, d_model))
        add("embed", (vocab, d_model))
        add("final_ln", (d_model,))
        add("lm_head", (d_model, vocab))
        return arrays
    if index == 5:  # uneven 3-way -> 5-way on the last dim: int32 [8,4097] and fp8-e4m3 [11008,4099]
        a = (8, 4097)
        b = (11008 // s, 4099)
        return [
            _array("c5_tokens", "S32", a, _side(a, (1, 3), 0), _side(a, (1, 5), 3), 5, "int32000"),
            _array("c5_fp8", "F8E4M3FN", b, _side(b, (1, 3), 0), _side(b, (1, 5), 3), 6, "fp8"),
        ]
    if index == 6:  # variant of 5 sharding dim 0 (8 rows 3-way -> 5-way leaves an empty edge tile)
        a = (8, 4097)
        b = (11008 // s, 4099)
        return [
            _array("c5b_tokens", "S32", a, _side(a, (3, 1), 0), _side(a, (5, 1), 3), 5, "int32000"),
            _array("c5b_fp8", "F8E4M3FN", b, _side(b, (3, 1), 0), _side(b, (5, 1), 3), 6, "fp8"),
        ]
    if index in (13, 14, 15):  # transposed destination layout: rows 4-way, row-major -> columns 4-way, column-major
        type_ = {13: "BF16", 14: "F32", 15: "U8"}[index]
        shape = (8192 // s, 8192 // s)
        return [_array("transposed", type_, shape, _side(shape, (4, 1), 0),
                       _side(shape, (1, 4), 4, minor_to_major=(0, 1)), 13, "raw")]
    raise ValueError("configuration %r" % (index,))


def load_json(path: str) -> List[dict]:
    """Arrays of a user-defined workload: a JSON list of dicts with the keys described at the top of this file."""
    import json
    with open(path) as f:
        arrays = json.load(f)
    for a in arrays:
        a["shape"] = tuple(int(s) for s in a["shape"])
        for side in ("src", "dst"):
            a[side]["dims"] = [tuple(int(v) for v in d) for d in a[side]["dims"]]
        a.setdefault("seed", 0)
        a.setdefault("dist", "raw")
    return arrays


def side(shape: Sequence[int], sharding: Sequence[int], dev_start: int, replication: int = 1,
         minor_to_major: Optional[Sequence[int]] = None) -> dict:
    """One side of a workload array: row-major device order over `sharding` tiles per dim."""
    return _side(shape, sharding, dev_start, replication, minor_to_major)


def algorithmic_bytes(arrays: Sequence[dict]) -> int:
    """2 x valid elements x itemsize per array: each element read once from one
    source replica and written once per destination shard that owns it."""
    total = 0
    for a in arrays:
        n = int(np.prod(a["shape"])) if a["shape"] else 1
        repl = 1
        dims = a["dst"]["dims"]
        if len(dims) > len(a["shape"]):
            repl = dims[-1][1]
        total += n * ITEMSIZE[a["type"]] * (1 + repl)
    return total


def fp8_e4m3fn_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> float8 e4m3fn bit patterns (1 sign, 4 exponent bits of bias 7, 3 mantissa bits, no infinity,
    0x7f = NaN, largest finite 448), round to nearest even.  Same bits as torch's `.to(torch.float8_e4m3fn)`;
    kept in NumPy so that processes driving the GPU never import torch."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    sign = ((bits >> np.uint32(24)) & np.uint32(0x80)).astype(np.uint8)
    mag = bits & np.uint32(0x7FFFFFFF)
    a = mag.view(np.float32)
    # normal range (>= 2^-6): round the mantissa to 3 bits, ties to even; a carry runs into the exponent by itself
    lsb = (mag >> np.uint32(20)) & np.uint32(1)
    rounded = (mag + np.uint32(0x7FFFF) + lsb) >> np.uint32(20)          # exponent (8 bits) | mantissa (3 bits)
    normal = rounded.astype(np.int64) - ((127 - 7) << 3)
    # subnormal range (< 2^-6): multiples of 2^-9; rint rounds ties to even, 8 lands on the smallest normal
    sub = np.rint(np.where(a < np.float32(1.0), a, np.float32(0.0)).astype(np.float64) * 512.0).astype(np.int64)
    code = np.where(a < np.float32(2.0 ** -6), sub, normal)
    code = np.where((code > 0x7E) | np.isnan(a), 0x7F, code)              # beyond 448 after rounding, or NaN
    return (code.astype(np.uint8) | sign).reshape(x.shape)


def _bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns, round to nearest even."""
    u = x.astype(np.float32).view(np.uint32)
    rounded = u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    return (rounded >> np.uint32(16)).astype(np.uint16)


def generate(a: dict) -> np.ndarray:
    """Global array of `a` as raw bits (unsigned dtype of the element size)."""
    rng = np.random.Generator(np.random.PCG64(a["seed"]))
    shape, dist = a["shape"], a["dist"]
    if dist == "uniform":
        x = rng.uniform(-1.0, 1.0, size=shape).astype(np.float32)
    elif dist == "normal":
        x = rng.standard_normal(size=shape, dtype=np.float32)
    elif dist == "normal_002":
        x = rng.standard_normal(size=shape, dtype=np.float32) * np.float32(0.02)
    elif dist == "raw":
        n = int(np.prod(shape)) * ITEMSIZE[a["type"]]
        return rng.integers(0, 256, size=n, dtype=np.uint8).view("<u%d" % ITEMSIZE[a["type"]]).reshape(shape)
    elif dist == "int32000":
        return rng.integers(0, 32000, size=shape, dtype=np.int32).view(np.uint32)
    elif dist == "fp8":
        return fp8_e4m3fn_bits(np.clip(rng.standard_normal(size=shape, dtype=np.float32), -448.0, 448.0))
    else:
        raise ValueError(dist)
    if a["type"] == "BF16":
        return _bf16_bits(x)
    if a["type"] == "F32":
        return x.view(np.uint32)
    raise ValueError(a["type"])
