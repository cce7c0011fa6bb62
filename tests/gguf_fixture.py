"""Builds GGUF v3 bytes for the host-layer tests: a header, metadata of all thirteen value
types, a tensor table and aligned payloads.  Written with struct only, independent of the
C++ writer it is also used to check.  Layout: the reference's own fixture builder places
tensors the same way (crates/neura-gguf/tests/support/mod.rs:21-64)."""
import struct

KINDS = {"u8": (0, "<B"), "i8": (1, "<b"), "u16": (2, "<H"), "i16": (3, "<h"), "u32": (4, "<I"), "i32": (5, "<i"), "f32": (6, "<f"),
         "bool": (7, "<B"), "u64": (10, "<Q"), "i64": (11, "<q"), "f64": (12, "<d")}


def _text(held):
    raw = held.encode()
    return struct.pack("<Q", len(raw)) + raw


def _body(kind, value):
    if kind == "string":
        return _text(value)
    if kind == "array":
        inner, items = value
        code = 8 if inner == "string" else 9 if inner == "array" else KINDS[inner][0]
        return struct.pack("<IQ", code, len(items)) + b"".join(_body(inner, item) for item in items)
    return struct.pack(KINDS[kind][1], value)


def _value(kind, value):
    code = 8 if kind == "string" else 9 if kind == "array" else KINDS[kind][0]
    return struct.pack("<I", code) + _body(kind, value)


def build(alignment, metadata, tensors, version=3):
    """metadata: [(key, kind, value)]; tensors: [(name, ggml_type, shape, payload)].
    Returns (bytes, data_start, {name: offset in the tensor data})."""
    out = b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(metadata))
    for key, kind, value in metadata:
        out += _text(key) + _value(kind, value)
    at, cursor = {}, 0
    for name, kind, shape, payload in tensors:
        at[name] = cursor
        out += _text(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape) + struct.pack("<IQ", kind, cursor)
        cursor = (cursor + len(payload) + alignment - 1) // alignment * alignment
    out += b"\0" * (-len(out) % alignment)
    data = len(out)
    for name, kind, shape, payload in tensors:
        out += bytes(payload)
        out += b"\0" * (-len(out) % alignment)
    return out, data, at
