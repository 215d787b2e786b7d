"""safetensors files at the edge of the device path: zyx's `Module::save` / `load_safetensors`
(zyx/src/module.rs:37-64, 436-530; dtype names zyx/src/dtype.rs:227-263) read and written as plain data.

Format: u64 little-endian header length, a JSON header {name: {"dtype", "shape", "data_offsets": [begin, end]}}
(offsets relative to the end of the header, an optional "__metadata__" entry is skipped), then the raw
little-endian tensor bytes. Nothing in a file is executed. `load` maps the file and yields numpy views (bf16 as
its uint16 bit patterns, which is how the device path stores it); `load_to_pool` uploads every tensor into a
HIPMemoryPool buffer sized like zyx's Allocate node (one extra element)."""
from __future__ import annotations

import json
import mmap
import struct

import numpy as np

from .backend import DType, HIPMemoryPool

_NP = {"BF16": np.uint16, "F16": np.float16, "F32": np.float32, "F64": np.float64, "U8": np.uint8, "U16": np.uint16,
       "U32": np.uint32, "U64": np.uint64, "I8": np.int8, "I16": np.int16, "I32": np.int32, "I64": np.int64, "BOOL": np.bool_}
_DT = {"BF16": DType.BF16, "F16": DType.F16, "F32": DType.F32, "F64": DType.F64, "U8": DType.U8, "U16": DType.U16,
       "U32": DType.U32, "U64": DType.U64, "I8": DType.I8, "I16": DType.I16, "I32": DType.I32, "I64": DType.I64, "BOOL": DType.Bool}
_NAME = {v: k for k, v in _DT.items()}


def load(path: str) -> dict:
    """-> {name: (DType, numpy array)}; arrays are read-only views of the mapped file."""
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) != 8:
            raise ValueError("Failed to parse header len in safetensors file.")
        (n,) = struct.unpack("<Q", head)
        size = f.seek(0, 2)
        if 8 + n > size:
            raise ValueError("safetensors header is longer than the file")
        mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
    header = json.loads(bytes(mm[8:8 + n]).decode("utf-8"))
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        if meta["dtype"] not in _NP:
            raise ValueError(f"Cannot parse safetensors dtype: {meta['dtype']}")
        begin, end = meta["data_offsets"]
        shape = tuple(int(d) for d in meta["shape"])
        np_dt = np.dtype(_NP[meta["dtype"]])
        count = int(np.prod(shape, dtype=np.int64))
        if end - begin != count * np_dt.itemsize or 8 + n + end > size or begin < 0:
            raise ValueError(f"safetensors tensor {name}: offsets do not match shape and dtype")
        out[name] = (_DT[meta["dtype"]], np.frombuffer(mm, np_dt, count, 8 + n + begin).reshape(shape))
    return out


def save(path: str, tensors: dict) -> None:
    """tensors: {name: (DType, array)} or {name: array} (dtype from the array; uint16 arrays need the explicit form
    to be written as BF16). Layout as Module::save writes it: header entries and data in iteration order."""
    header, blobs, begin = {}, [], 0
    for name, val in tensors.items():
        dt, arr = val if isinstance(val, tuple) else (None, val)
        arr = np.ascontiguousarray(arr)
        if dt is None:
            dt = {np.dtype(v): k for k, v in _NP.items() if k != "BF16"}[arr.dtype]
        else:
            dt = _NAME[DType(dt)]
            if np.dtype(_NP[dt]).itemsize != arr.dtype.itemsize:
                raise ValueError(f"tensor {name}: array dtype {arr.dtype} cannot hold {dt}")
        raw = arr.astype(arr.dtype.newbyteorder("<"), copy=False).tobytes()
        header[name] = {"dtype": dt, "shape": list(arr.shape), "data_offsets": [begin, begin + len(raw)]}
        begin += len(raw)
        blobs.append(raw)
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for raw in blobs:
            f.write(raw)


def load_to_pool(path: str, pool: HIPMemoryPool) -> dict:
    """-> {name: (buffer id, DType, shape)}: every tensor uploaded (allocation + host_to_pool), all copies synced."""
    out, events, keep = {}, [], []
    for name, (dt, arr) in load(path).items():
        arr = np.ascontiguousarray(arr)
        keep.append(arr)  # the source must outlive the copy's event
        buf, ev = pool.allocate(arr.nbytes + arr.itemsize)
        events.append(pool.host_to_pool(arr, buf, [ev]))
        out[name] = (buf, dt, arr.shape)
    pool.sync_events(events)
    return out
