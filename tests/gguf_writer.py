"""A minimal GGUF v3 writer for the loader tests (container layout as in the public GGUF
specification: header, typed key/value pairs, tensor directory, aligned tensor data)."""
import struct

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_SCALAR = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B",
           U64: "<Q", I64: "<q", F64: "<d"}


def _string(text):
    data = text if isinstance(text, bytes) else text.encode()
    return struct.pack("<Q", len(data)) + data


def _value(kind, value):
    if kind == STRING:
        return _string(value)
    if kind == ARRAY:
        element, items = value
        return struct.pack("<IQ", element, len(items)) + b"".join(_value(element, v) for v in items)
    return struct.pack(_SCALAR[kind], value)


def build(metadata, tensors, alignment=32, version=3, magic=0x46554747, offsets=None, pad_tail=0):
    """metadata: [(key, kind, value)]; tensors: [(name, dims, qtype, bytes)]. Returns (file bytes,
    relative offsets). offsets overrides the computed relative offsets (for refusal cases)."""
    out = struct.pack("<IIQQ", magic, version, len(tensors), len(metadata))
    for key, kind, value in metadata:
        out += _string(key) + struct.pack("<I", kind) + _value(kind, value)
    relative, cursor = [], 0
    for _, _, _, data in tensors:
        relative.append(cursor)
        cursor += (len(data) + alignment - 1) // alignment * alignment
    if offsets is not None:
        relative = list(offsets)
    for (name, dims, qtype, _), offset in zip(tensors, relative):
        out += _string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", qtype, offset)
    out += b"\0" * (-len(out) % alignment)
    start = len(out)
    body = bytearray(max([o + len(t[3]) for o, t in zip(relative, tensors)] + [0]) + pad_tail)
    for (_, _, _, data), offset in zip(tensors, relative):
        body[offset:offset + len(data)] = data
    return out + bytes(body), relative, start
