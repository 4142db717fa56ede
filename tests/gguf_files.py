"""Writes small GGUF files for the reader tests: the same byte layout the
reference's test fixture builds (src/loader/gguf.rs:709-748), generalised to
arbitrary metadata, per-tensor types and payloads."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B",
        U64: "<Q", I64: "<q", F64: "<d"}


def string(s):
    raw = s if isinstance(s, bytes) else s.encode("utf-8")
    return struct.pack("<Q", len(raw)) + raw


def value(type_id, v, element=None):
    if type_id == STRING:
        return string(v)
    if type_id == ARRAY:
        return struct.pack("<IQ", element, len(v)) + b"".join(value(element, item) for item in v)
    return struct.pack(_FMT[type_id], v)


def header(tensors, metadata, version=3):
    """tensors: [(name, dims, type_id, offset)], metadata: [(key, type_id, value[, element])]."""
    out = bytearray(b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(metadata)))
    for key, type_id, v, *element in metadata:
        out += string(key) + struct.pack("<I", type_id) + value(type_id, v, *element)
    for name, dims, type_id, offset in tensors:
        out += string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", type_id, offset)
    return out


STANDARD = [("general.architecture", STRING, "qwen2"), ("general.quantization_version", U32, 2)]


def build(tensors, metadata=STANDARD, alignment=32, version=3):
    """tensors: [(name, dims, type_id, payload bytes)] laid out back to back at
    aligned offsets.  Returns the file's bytes."""
    placed, payloads, cursor = [], [], 0
    for name, dims, type_id, payload in tensors:
        payload = np.ascontiguousarray(payload, dtype=np.uint8).tobytes()
        placed.append((name, dims, type_id, cursor))
        payloads.append((cursor, payload))
        cursor = -(-(cursor + len(payload)) // alignment) * alignment
    out = header(placed, metadata, version)
    out += bytes(-len(out) % alignment)
    base = len(out)
    out += bytes(cursor)
    for offset, payload in payloads:
        out[base + offset:base + offset + len(payload)] = payload
    return bytes(out)


def reference_fixture(type_id, dims, offsets, names, block=(32, 34)):
    """The reference's own fixture: tensor i is filled with byte i+1 at offsets[i]."""
    out = header([(n, dims, type_id, o) for n, o in zip(names, offsets)], STANDARD)
    out += bytes(-len(out) % 32)
    payload = block[1] * int(np.prod(dims)) // block[0]
    base = len(out)
    out += bytes(max(offsets, default=0) + payload)
    for i, o in enumerate(offsets):
        out[base + o:base + o + payload] = bytes([i + 1]) * payload
    return bytes(out)
