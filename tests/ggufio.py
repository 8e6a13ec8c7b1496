"""A GGUF writer for the tests, straight from the public container layout (ggml's gguf.md):
magic, version, counts, metadata key/value pairs, tensor infos, padding, tensor data.

It exists so that the library's reader is checked against files produced by independent code.
"""
import struct

(U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64) = range(13)
_SCALAR = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q",
           F64: "<d"}

# ggml type id -> (block elements, block bytes)
GGML = {0: (1, 4), 1: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 36),
        10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292), 30: (1, 2)}
# the library's format enum -> ggml type id
GGML_OF_QUANT = {0: 2, 1: 8, 2: 12, 3: 14, 4: 3, 5: 6, 6: 7, 7: 10, 8: 11, 9: 13}


def _count(version, n):
    return struct.pack("<I" if version == 1 else "<Q", n)


def _string(version, s, v1_terminator=True):
    b = s if isinstance(s, bytes) else s.encode()
    if version == 1 and v1_terminator:
        b += b"\0"
    return _count(version, len(b)) + b


def _value(version, vtype, value):
    if vtype in _SCALAR:
        return struct.pack(_SCALAR[vtype], value)
    if vtype == STRING:
        return _string(version, value)
    if vtype == ARRAY:
        etype, items = value
        out = struct.pack("<I", etype) + _count(version, len(items))
        for it in items:
            out += _value(version, etype, it)
        return out
    raise ValueError(vtype)


def write_gguf(path, metadata, tensors, version=3, alignment=None, pad_tail=0):
    """metadata: [(key, value type, value)]; arrays are (ARRAY, (element type, [items])).
    tensors: [(name, dims outermost first, ggml type id, payload bytes)]."""
    align = alignment or 32
    out = b"GGUF" + struct.pack("<I", version) + _count(version, len(tensors)) + _count(version, len(metadata))
    for key, vtype, value in metadata:
        out += _string(version, key) + struct.pack("<I", vtype) + _value(version, vtype, value)
    offset = 0
    offsets = []
    for name, dims, gtype, payload in tensors:
        offsets.append(offset)
        out += _string(version, name) + struct.pack("<I", len(dims))
        for d in reversed(dims):            # stored innermost first
            out += _count(version, d)
        out += struct.pack("<I", gtype) + struct.pack("<Q", offset)
        offset += (len(payload) + align - 1) // align * align
    out += b"\0" * ((-len(out)) % align)
    for (name, dims, gtype, payload), off in zip(tensors, offsets):
        size = (len(payload) + align - 1) // align * align
        out += payload + b"\0" * (size - len(payload))
    out += b"\0" * pad_tail
    with open(path, "wb") as f:
        f.write(out)
    return out
