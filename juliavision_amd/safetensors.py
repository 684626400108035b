"""Minimal safetensors reader: a u64 little-endian header length, a JSON header mapping each
name to dtype / shape / byte range, then the raw data (readsafetensors, safetensors.jl:1-37).

The reference hands tensors back with their extents reversed because Julia is column-major;
torch is row-major like the file, so shapes come back as stored.  The file is memory-mapped:
``read`` returns views into the mapping (no copy until a tensor is moved to the device),
``load_to`` uploads every tensor once, which is what ``graph.Executor`` takes as its weights.
"""
from __future__ import annotations

import json
import mmap
import struct
from typing import Dict, Iterable, List, Optional

import numpy as np
import torch

# safetensors.jl:39-52; bf16 has no numpy dtype and is reinterpreted by torch
_NP = {"F64": np.float64, "F32": np.float32, "F16": np.float16, "BF16": np.uint16, "I64": np.int64, "I32": np.int32,
       "I16": np.int16, "I8": np.int8, "U8": np.uint8, "BOOL": np.bool_, "U64": np.uint64, "U32": np.uint32, "U16": np.uint16,
       "C64": np.complex64, "C128": np.complex128}


class SafetensorsError(ValueError):
    pass


def _header(buf) -> (dict, int):
    if len(buf) < 8:
        raise SafetensorsError("file shorter than its header length field")
    (hlen,) = struct.unpack_from("<Q", buf, 0)
    if hlen > len(buf) - 8:
        raise SafetensorsError(f"header length {hlen} exceeds the file ({len(buf)} bytes)")
    try:
        header = json.loads(bytes(buf[8:8 + hlen]).decode("utf-8"))
    except (UnicodeDecodeError, json.JSONDecodeError) as e:
        raise SafetensorsError(f"header is not JSON: {e}") from None
    if not isinstance(header, dict):
        raise SafetensorsError("header is not a JSON object")
    return header, 8 + hlen


def names(path: str) -> List[str]:
    """Header only, without touching tensor data (safetensorsnames, safetensors.jl:54-65)."""
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) < 8:
            raise SafetensorsError("file shorter than its header length field")
        (hlen,) = struct.unpack("<Q", head)
        header = json.loads(f.read(hlen).decode("utf-8"))
    return [k for k in header if k != "__metadata__"]


def read(path: str, only: Optional[Iterable[str]] = None) -> Dict[str, torch.Tensor]:
    """name -> CPU tensor backed by a read-only mapping of the file (copy-on-write: writing to a tensor
    does not change the file)."""
    with open(path, "rb") as f:
        mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_COPY)
    header, base = _header(mm)
    want = None if only is None else set(only)
    out: Dict[str, torch.Tensor] = {}
    for name, spec in header.items():
        if name == "__metadata__" or (want is not None and name not in want):
            continue
        try:
            dt = _NP[spec["dtype"]]
        except KeyError:
            raise SafetensorsError(f"{name}: dtype {spec.get('dtype')!r} is not one this reader knows") from None
        shape = [int(d) for d in spec["shape"]]
        lo, hi = (int(v) for v in spec["data_offsets"])
        count = int(np.prod(shape, dtype=np.int64)) if shape else 1
        if lo < 0 or hi < lo or base + hi > len(mm) or (hi - lo) != count * np.dtype(dt).itemsize:
            raise SafetensorsError(f"{name}: byte range [{lo}, {hi}) does not hold {shape} of {spec['dtype']}")
        a = np.frombuffer(mm, dtype=dt, count=count, offset=base + lo).reshape(shape)
        t = torch.from_numpy(a)
        out[name] = t.view(torch.bfloat16) if spec["dtype"] == "BF16" else t
    if want is not None and want - set(out):
        raise KeyError(f"not in {path}: {sorted(want - set(out))}")
    return out


def load_to(path: str, device="cuda", dtype: Optional[torch.dtype] = None, only: Optional[Iterable[str]] = None) -> Dict[str, torch.Tensor]:
    """Every tensor uploaded once; floating tensors converted to ``dtype`` when given (weights stored in fp32
    for an fp16 graph)."""
    out = {}
    for name, t in read(path, only).items():
        t = t.to(device)
        if dtype is not None and t.is_floating_point():
            t = t.to(dtype)
        out[name] = t
    return out
