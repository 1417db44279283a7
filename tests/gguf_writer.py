"""A minimal GGUF v3 writer for the loader tests, written from the published file format (not from the reference):
header, typed metadata pairs, tensor records, alignment padding, tensor data."""
from __future__ import annotations

import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}


def _s(text: str) -> bytes:
    raw = text.encode()
    return struct.pack("<Q", len(raw)) + raw


def _value(vtype: int, value) -> bytes:
    if vtype == STRING:
        return _s(value)
    if vtype == ARRAY:
        etype, items = value
        return struct.pack("<IQ", etype, len(items)) + b"".join(_value(etype, v) for v in items)
    return struct.pack(_FMT[vtype], value)


def write_gguf(path: str, metadata: list[tuple[str, int, object]], tensors: list[tuple[str, list[int], int, bytes]], alignment: int = 32, version: int = 3,
               magic: bytes = b"GGUF") -> dict[str, int]:
    """tensors: (name, dims in ggml order, ggml type, raw bytes).  Returns name -> absolute file offset of the data."""
    head = magic + struct.pack("<IQQ", version, len(tensors), len(metadata))
    for key, vtype, value in metadata:
        head += _s(key) + struct.pack("<I", vtype) + _value(vtype, value)
    offsets, pos = [], 0
    for _, _, _, raw in tensors:
        offsets.append(pos)
        pos = (pos + len(raw) + alignment - 1) // alignment * alignment
    for (name, dims, ttype, _), off in zip(tensors, offsets):
        head += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", ttype, off)
    data_start = (len(head) + alignment - 1) // alignment * alignment
    body = bytearray(head) + bytes(data_start - len(head))
    where = {}
    for (name, _, _, raw), off in zip(tensors, offsets):
        body += bytes(data_start + off - len(body))
        where[name] = len(body)
        body += raw
    with open(path, "wb") as f:
        f.write(body)
    return where


def f32_bytes(values) -> bytes:
    return np.asarray(values, dtype=np.float32).tobytes()
