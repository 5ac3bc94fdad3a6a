"""Writes small GGUF files for the reader's tests: the format of src/ml/gguf/reader.cr:1-6 (magic, version,
counts, KV pairs, tensor infos, aligned data blob). Test infrastructure only."""
import struct

UINT8, INT8, UINT16, INT16, UINT32, INT32, FLOAT32, BOOL, STRING, ARRAY, UINT64, INT64, FLOAT64 = range(13)
_FMT = {UINT8: "<B", INT8: "<b", UINT16: "<H", INT16: "<h", UINT32: "<I", INT32: "<i", FLOAT32: "<f", UINT64: "<Q",
        INT64: "<q", FLOAT64: "<d"}


def _s(text):
    b = text.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _v(vtype, value, etype=None):
    if vtype in _FMT:
        return struct.pack(_FMT[vtype], value)
    if vtype == BOOL:
        return struct.pack("<B", 1 if value else 0)
    if vtype == STRING:
        return _s(value)
    if vtype == ARRAY:
        return struct.pack("<IQ", etype, len(value)) + b"".join(_v(etype, e) for e in value)
    raise ValueError(vtype)


def write_gguf(path, kv, tensors, version=3, alignment=None, magic=b"GGUF"):
    """kv: list of (key, vtype, value[, etype]); tensors: list of (name, dims, ggml type, bytes)."""
    align = alignment or 32
    kv = list(kv)
    if alignment is not None:
        kv.append(("general.alignment", UINT32, alignment))
    head = magic + struct.pack("<Iqq", version, len(tensors), len(kv))
    for item in kv:
        key, vtype, value = item[:3]
        head += _s(key) + struct.pack("<I", vtype) + _v(vtype, value, item[3] if len(item) > 3 else None)
    offsets, off = [], 0
    for name, dims, ttype, data in tensors:
        offsets.append(off)
        off = (off + len(data) + align - 1) // align * align
    for (name, dims, ttype, data), o in zip(tensors, offsets):
        head += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<q", d) for d in dims)
        head += struct.pack("<IQ", ttype, o)
    pad = (-len(head)) % align
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        for (name, dims, ttype, data), o in zip(tensors, offsets):
            f.write(bytes(data))
            f.write(b"\0" * ((-len(data)) % align))
    return len(head) + pad
