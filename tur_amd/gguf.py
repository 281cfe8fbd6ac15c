"""Minimal GGUF writer (v3) used to build test and benchmark files from raw block bytes.

Reading is done by ``libturq.so`` (``turq_gguf_*``); this module only writes, so that the reader can
be exercised on files that hold the synthetic tensors of ``tur_amd.synth``.
"""
from __future__ import annotations

import struct
from typing import Dict, Iterable, Tuple

import numpy as np

from . import synth

GGUF_MAGIC = 0x46554747
VT_U32, VT_I32, VT_F32, VT_BOOL, VT_STRING, VT_ARRAY, VT_U64, VT_I64, VT_F64 = 4, 5, 6, 7, 8, 9, 10, 11, 12


def _s(v: str) -> bytes:
    b = v.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _value(v) -> bytes:
    if isinstance(v, bool):
        return struct.pack("<IB", VT_BOOL, int(v))
    if isinstance(v, int):
        return struct.pack("<II", VT_U32, v) if 0 <= v < 2**32 else struct.pack("<Iq", VT_I64, v)
    if isinstance(v, float):
        return struct.pack("<If", VT_F32, v)
    if isinstance(v, str):
        return struct.pack("<I", VT_STRING) + _s(v)
    if isinstance(v, (list, tuple)):
        if all(isinstance(e, str) for e in v):
            return struct.pack("<IIQ", VT_ARRAY, VT_STRING, len(v)) + b"".join(_s(e) for e in v)
        if all(isinstance(e, int) for e in v):
            return struct.pack("<IIQ", VT_ARRAY, VT_I32, len(v)) + b"".join(struct.pack("<i", e) for e in v)
        if all(isinstance(e, float) for e in v):
            return struct.pack("<IIQ", VT_ARRAY, VT_F32, len(v)) + b"".join(struct.pack("<f", e) for e in v)
    raise TypeError(f"unsupported metadata value {v!r}")


def write_gguf(path: str, tensors: Iterable[Tuple[str, int, Tuple[int, ...], np.ndarray]], metadata: Dict[str, object] | None = None,
               alignment: int = 32) -> None:
    """tensors: (name, ggml_dtype, shape outermost-first e.g. (n, k), raw bytes as uint8 array)."""
    tensors = list(tensors)
    metadata = dict(metadata or {})
    if alignment != 32:
        metadata["general.alignment"] = alignment
    head = struct.pack("<IIQQ", GGUF_MAGIC, 3, len(tensors), len(metadata))
    for k, v in metadata.items():
        head += _s(k) + _value(v)
    offset = 0
    blobs = []
    for name, dt, shape, raw in tensors:
        raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        nelem = int(np.prod(shape))
        expect = nelem // synth.BLOCK_ELEMS[dt] * synth.BLOCK_BYTES[dt]
        if raw.size != expect:
            raise ValueError(f"{name}: {raw.size} bytes, shape {shape} of dtype {dt} needs {expect}")
        head += _s(name) + struct.pack("<I", len(shape))
        for d in reversed(shape):       # GGUF stores the innermost dimension first
            head += struct.pack("<Q", d)
        head += struct.pack("<IQ", dt, offset)
        blobs.append((offset, raw))
        offset += (raw.size + alignment - 1) // alignment * alignment
    pad = (-len(head)) % alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        base = f.tell()
        for off, raw in blobs:
            f.seek(base + off)
            f.write(raw.tobytes())
        end = base + offset
        f.seek(0, 2)
        if f.tell() < end:
            f.write(b"\0" * (end - f.tell()))
