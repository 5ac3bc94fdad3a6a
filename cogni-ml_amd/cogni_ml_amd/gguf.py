"""GGUF file reader: metadata, tensor table and zero-copy tensor bytes out of an mmap.

The counterpart of the reference's ML::GGUF::GGUFFile (src/ml/gguf/reader.cr:130-391): same file format
(magic "GGUF", version 2 or 3, n_tensors:i64, n_kv:i64, KV pairs, tensor infos, data blob aligned to
general.alignment or 32), same accessors (tensor, read_tensor_raw, read_tensor_f32, get_string/get_int/get_float/
get_int_array/get_bool_array, mmap_region, data_offset) and the same errors for a wrong magic or version.
read_tensor_f32 dequantizes through the library's Dequant kernels (there is no CPU path); the loaders at the
bottom are the reference's load_qw / load_f32 (src/ml/gguf/qwen35_weights.cr:203-218).
"""
import mmap
import struct

import numpy as np

from .types import TensorType

MAGIC = b"GGUF"
VERSION = 3
ALIGNMENT = 32

# GGUF value types (reader.cr:17-31)
UINT8, INT8, UINT16, INT16, UINT32, INT32, FLOAT32, BOOL, STRING, ARRAY, UINT64, INT64, FLOAT64 = range(13)
_SCALAR = {UINT8: "<B", INT8: "<b", UINT16: "<H", INT16: "<h", UINT32: "<I", INT32: "<i", FLOAT32: "<f",
           UINT64: "<Q", INT64: "<q", FLOAT64: "<d"}


class GGUFError(RuntimeError):
    pass


class Value:
    """A metadata value together with its GGUF value type (the reference's typed union keeps UInt32 apart from
    Int64 and Float32 from Float64; the getters below depend on it)."""
    __slots__ = ("vtype", "value", "etype")

    def __init__(self, vtype, value, etype=None):
        self.vtype, self.value, self.etype = vtype, value, etype

    def __repr__(self):
        return "Value(%d, %r)" % (self.vtype, self.value)


class TensorInfo:
    """reader.cr:105-128."""

    def __init__(self, name, dims, ttype, offset):
        self.name, self.dims, self.type, self.offset = name, list(dims), TensorType(ttype), offset

    @property
    def n_elements(self):
        n = 1 if self.dims else 0
        for d in self.dims:
            n *= d
        return n

    @property
    def data_bytes(self):
        return self.type.data_bytes(self.n_elements)


class GGUFFile:
    def __init__(self, path):
        self.path = path
        self.version = 0
        self.metadata = {}          # key -> Value
        self.tensors = []
        self.data_offset = 0
        self._io = open(path, "rb")
        try:
            self._mm = mmap.mmap(self._io.fileno(), 0, access=mmap.ACCESS_READ)
        except (ValueError, OSError) as e:     # empty file or no mmap: nothing to parse either way
            self._io.close()
            raise GGUFError("Not a GGUF file: %s" % e)
        self._pos = 0
        try:
            self._parse_header()
        except Exception:
            self.close()
            raise
        self._by_name = {}
        for t in self.tensors:
            self._by_name.setdefault(t.name, t)      # Array#find returns the first match (reader.cr:219-221)
        self._bytes = np.frombuffer(self._mm, dtype=np.uint8)

    # ---- lifetime ---------------------------------------------------------------------------------------
    def close(self):
        self._bytes = None
        if self._mm is not None:
            try:
                self._mm.close()
            except BufferError:      # tensor views are still alive; the map goes when they do
                pass
            self._mm = None
        if not self._io.closed:
            self._io.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # ---- tensors ----------------------------------------------------------------------------------------
    def tensor(self, name):
        return self._by_name.get(name)

    def read_tensor_raw(self, info):
        """Zero-copy uint8 view of the tensor's bytes in the mmap (reader.cr:169-171, 183-195)."""
        off = self.data_offset + info.offset
        end = off + info.data_bytes
        if end > self._bytes.size:
            raise GGUFError("tensor %r ends at byte %d of a %d-byte file" % (info.name, end, self._bytes.size))
        return self._bytes[off:end]

    def read_tensor_f32(self, info):
        """Dequantized to float32 (reader.cr:162-166), computed by the library's dequantize kernels."""
        from . import quant
        return quant.dequantize(self.read_tensor_raw(info), info.type, info.n_elements)

    def mmap_region(self):
        """(numpy uint8 view of the whole file, size): the reference hands out the base pointer and size
        (reader.cr:177-181) so that one buffer can cover the file and tensors are addressed by offset."""
        return self._bytes, self._bytes.size

    # ---- metadata getters (reader.cr:224-276) -------------------------------------------------------------
    def get_string(self, key):
        v = self.metadata.get(key)
        return v.value if v is not None and v.vtype == STRING else None

    def get_int(self, key):
        v = self.metadata.get(key)
        return int(v.value) if v is not None and v.vtype in (INT32, UINT32, INT64, UINT64) else None

    def get_float(self, key):
        v = self.metadata.get(key)
        return float(v.value) if v is not None and v.vtype in (FLOAT32, FLOAT64) else None

    def get_int_array(self, key):
        v = self.metadata.get(key)
        if v is None or v.vtype != ARRAY:
            return None
        if v.etype not in (INT8, UINT8, INT16, UINT16, INT32, UINT32, INT64, UINT64):
            return None if v.value else []
        return [int(e) for e in v.value]

    def get_bool_array(self, key):
        v = self.metadata.get(key)
        if v is None or v.vtype != ARRAY:
            return None
        if v.etype != BOOL:
            return None if v.value else []
        return [bool(e) for e in v.value]

    # ---- parsing (reader.cr:278-391) ----------------------------------------------------------------------
    def _take(self, n):
        if n < 0 or self._pos + n > len(self._mm):
            raise GGUFError("unexpected end of file at byte %d" % self._pos)
        b = self._mm[self._pos:self._pos + n]
        self._pos += n
        return b

    def _scalar(self, vtype):
        fmt = _SCALAR[vtype]
        return struct.unpack(fmt, self._take(struct.calcsize(fmt)))[0]

    def _string(self):
        n = self._scalar(UINT64)
        n = n & 0xFFFFFFFF                      # the reference truncates the length to Int32 (reader.cr:340-341)
        if n >= 0x80000000 or n == 0:
            return ""
        return self._take(n).decode("utf-8", errors="replace")

    def _value(self, vtype):
        if vtype in _SCALAR:
            return Value(vtype, self._scalar(vtype))
        if vtype == BOOL:
            return Value(vtype, self._scalar(UINT8) != 0)
        if vtype == STRING:
            return Value(vtype, self._string())
        if vtype == ARRAY:
            etype = self._scalar(UINT32)
            n = self._scalar(UINT64) & 0xFFFFFFFF
            if etype in _SCALAR and etype != ARRAY:
                fmt = _SCALAR[etype]
                size = struct.calcsize(fmt)
                raw = self._take(n * size)
                vals = list(struct.unpack("<%d%s" % (n, fmt[1]), raw)) if n else []
            else:
                vals = [self._value(etype).value for _ in range(n)]
            return Value(ARRAY, vals, etype)
        raise GGUFError("unknown GGUF value type %d" % vtype)

    def _parse_header(self):
        magic = bytes(self._take(4)) if len(self._mm) >= 4 else bytes(self._mm[:])
        if magic != MAGIC:
            raise GGUFError("Not a GGUF file: magic=%r" % magic.decode("latin-1"))
        self.version = self._scalar(UINT32)
        if not 2 <= self.version <= 3:
            raise GGUFError("Unsupported GGUF version: %d" % self.version)
        n_tensors = self._scalar(INT64)
        n_kv = self._scalar(INT64)
        for _ in range(n_kv):
            key = self._string()
            vtype = self._scalar(UINT32)
            self.metadata[key] = self._value(vtype)
        for _ in range(n_tensors):
            name = self._string()
            n_dims = self._scalar(UINT32)
            dims = [self._scalar(INT64) for _ in range(n_dims)]
            ttype = self._scalar(UINT32)
            offset = self._scalar(UINT64)
            try:
                self.tensors.append(TensorInfo(name, dims, ttype, offset))
            except ValueError:
                raise GGUFError("tensor %r has unknown ggml type %d" % (name, ttype))
        align = self.metadata.get("general.alignment")
        alignment = int(align.value) if align is not None and align.vtype == UINT32 else ALIGNMENT
        self.data_offset = (self._pos + alignment - 1) & ~(alignment - 1)


# ---- loaders (src/ml/gguf/qwen35_weights.cr:203-218) -----------------------------------------------------------
def load_qw(gguf, name, route_prefix="qwen35"):
    """QuantWeight over the tensor's raw bytes: dims = [in_dim, out_dim], row-major with out_dim rows. The bytes are
    uploaded once; the host side keeps the mmap view, not a copy."""
    from . import quant
    info = gguf.tensor(name)
    if info is None:
        raise GGUFError("qwen35_weights: missing tensor %r" % name)
    raw = gguf.read_tensor_raw(info)
    in_dim = int(info.dims[0])
    out_dim = int(info.dims[1]) if len(info.dims) >= 2 else 1
    return quant.QuantWeight(raw, info.type, out_dim, in_dim, "%s:%s" % (route_prefix, name))


def load_f32(gguf, name):
    info = gguf.tensor(name)
    if info is None:
        raise GGUFError("qwen35_weights: missing tensor %r" % name)
    return gguf.read_tensor_f32(info)
