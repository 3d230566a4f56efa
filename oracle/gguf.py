"""GGUF v3 writer: a restatement of hf2q's own writer, used to make the files the reader tests open.

TEST INFRASTRUCTURE ONLY (like the rest of this package).  Follows
src/backends/gguf/types.rs:20-32 (magic, version 3, 32-byte alignment), :41-53 (value type codes),
:96-188 (string and key/value encoding) and src/backends/gguf/writer.rs:171-258, 260-330 (header, tensor
directory entry, padding before the data section and after every tensor; offsets relative to the start
of the data section).
"""
from __future__ import annotations

import struct

MAGIC = b"GGUF"
VERSION = 3
ALIGNMENT = 32

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_SCALAR = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q",
           I64: "<q", F64: "<d"}


def _string(s: str) -> bytes:                      # types.rs:96-101
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _value(t: int, v) -> bytes:
    return _string(v) if t == STRING else struct.pack(_SCALAR[t], v)


def metadata_kv(key: str, t: int, v, elem_type: int | None = None) -> bytes:   # types.rs:103-188
    out = _string(key) + struct.pack("<I", t)
    if t == ARRAY:
        out += struct.pack("<IQ", elem_type, len(v)) + b"".join(_value(elem_type, e) for e in v)
    else:
        out += _value(t, v)
    return out


def align_up(n: int, a: int = ALIGNMENT) -> int:
    return (n + a - 1) // a * a


def build(metadata, tensors, alignment: int = ALIGNMENT) -> tuple[bytes, list]:
    """metadata: [(key, type, value[, elem_type])]; tensors: [(name, dims (GGUF order), ggml_type, payload)].
    Returns (file bytes, data-section-relative offsets)."""
    out = bytearray(MAGIC + struct.pack("<IQQ", VERSION, len(tensors), len(metadata)))   # writer.rs:171-183
    for m in metadata:
        out += metadata_kv(*m)
    offsets, rel = [], 0
    for name, dims, ggml_type, payload in tensors:                                       # writer.rs:186-222
        offsets.append(rel)
        out += _string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", ggml_type, rel)
        rel = align_up(rel + len(payload), alignment)                                    # writer.rs:309-316
    out += b"\0" * (align_up(len(out), alignment) - len(out))                            # writer.rs:260-275
    for (_, _, _, payload) in tensors:
        out += payload
        out += b"\0" * (align_up(len(payload), alignment) - len(payload))
    return bytes(out), offsets


def write(path: str, metadata, tensors, alignment: int = ALIGNMENT) -> list:
    data, offsets = build(metadata, tensors, alignment)
    with open(path, "wb") as f:
        f.write(data)
    return offsets
