"""GGUF (version 3) container reader and writer for the tensors this backend consumes.

Layout (all little-endian): magic "GGUF", u32 version, u64 tensor_count, u64 kv_count; kv_count
(key string, u32 value type, value) pairs; tensor_count (name string, u32 n_dims, u64 dims[n_dims]
with dims[0] the contiguous one, u32 ggml type, u64 offset into the data section); padding to
`general.alignment` (default 32); the tensor data.  Strings are u64 length + UTF-8 bytes.

The reader memory-maps the file, so a quantized tensor goes from disk to `psn_weight_upload` without
a copy on the host.  No .gguf file ships with the reference tree
(/root/reference/apps/pylon/docs/2026-06-09-pylon-qwen35-local-inference-roadmap.md:84,141-142 only
names them), so the round trip through the writer here is what the tests check.
"""
from __future__ import annotations

import struct
from dataclasses import dataclass

import numpy as np

MAGIC = b"GGUF"
DEFAULT_ALIGNMENT = 32
MAX_DIMS = 4            # ggml tensors have at most four dimensions

# ggml tensor types this module knows: id -> (elements per block, bytes per block, name)
GGML_TYPES = {0: (1, 4, "F32"), 1: (1, 2, "F16"), 2: (32, 18, "Q4_0"), 8: (32, 34, "Q8_0"),
              12: (256, 144, "Q4_K"), 13: (256, 176, "Q5_K"), 14: (256, 210, "Q6_K")}

# metadata value types
U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_SCALAR = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<?", U64: "<Q", I64: "<q", F64: "<d"}


class GGUFError(ValueError):
    pass


@dataclass
class TensorInfo:
    name: str
    dims: tuple          # ggml order: dims[0] is the contiguous (K) dimension
    ggml_type: int
    offset: int          # into the data section
    nbytes: int

    @property
    def k(self) -> int:
        return int(self.dims[0])

    @property
    def n(self) -> int:
        n = 1
        for d in self.dims[1:]:
            n *= int(d)
        return n


def tensor_nbytes(ggml_type: int, dims) -> int:
    if ggml_type not in GGML_TYPES:
        raise GGUFError(f"ggml type {ggml_type} is not supported")
    be, bb, name = GGML_TYPES[ggml_type]
    if not 1 <= len(dims) <= MAX_DIMS or any(int(d) <= 0 for d in dims):
        raise GGUFError(f"{name}: dims {tuple(dims)} (want 1..{MAX_DIMS} positive dimensions)")
    if dims[0] % be:
        raise GGUFError(f"{name}: row length {dims[0]} is not a whole number of {be}-element blocks")
    rows = 1
    for d in dims[1:]:
        rows *= d
    return dims[0] // be * bb * rows


class _Cursor:
    def __init__(self, buf):
        self.buf, self.pos = buf, 0

    def take(self, fmt):
        size = struct.calcsize(fmt)
        if self.pos + size > len(self.buf):
            raise GGUFError("file ends inside the header")
        v = struct.unpack_from(fmt, self.buf, self.pos)[0]
        self.pos += size
        return v

    def string(self):
        n = self.take("<Q")
        if self.pos + n > len(self.buf):
            raise GGUFError("file ends inside a string")
        s = bytes(self.buf[self.pos:self.pos + n]).decode("utf-8")
        self.pos += n
        return s

    def remaining(self):
        return len(self.buf) - self.pos

    def count(self, min_bytes_each, what):
        """A u64 element count, checked against what the rest of the file could possibly hold."""
        n = self.take("<Q")
        if n * min_bytes_each > self.remaining():
            raise GGUFError(f"{what}: count {n} does not fit the remaining {self.remaining()} bytes")
        return n

    def value(self, vtype):
        if vtype in _SCALAR:
            return self.take(_SCALAR[vtype])
        if vtype == STRING:
            return self.string()
        if vtype == ARRAY:
            et = self.take("<I")
            if et == ARRAY:
                raise GGUFError("nested metadata arrays are not supported")
            if et != STRING and et not in _SCALAR:
                raise GGUFError(f"unknown metadata array element type {et}")
            count = self.count(8 if et == STRING else struct.calcsize(_SCALAR[et]), "metadata array")
            return [self.value(et) for _ in range(count)]
        raise GGUFError(f"unknown metadata value type {vtype}")


class GGUFFile:
    """A memory-mapped GGUF file: `metadata` (dict), `tensors` (name -> TensorInfo), `data(name)`."""

    def __init__(self, path: str):
        self.path = path
        self._map = np.memmap(path, dtype=np.uint8, mode="r")
        c = _Cursor(self._map)
        if bytes(self._map[:4]) != MAGIC:
            raise GGUFError("not a GGUF file (bad magic)")
        c.pos = 4
        self.version = c.take("<I")
        if self.version not in (2, 3):
            raise GGUFError(f"GGUF version {self.version} is not supported")
        n_tensors, n_kv = c.take("<Q"), c.take("<Q")
        # a key/value pair takes at least 8 + 4 + 1 bytes, a tensor entry at least 8 + 4 + 8 + 4 + 8
        if n_kv * 13 + n_tensors * 32 > c.remaining():
            raise GGUFError(f"header counts ({n_tensors} tensors, {n_kv} metadata pairs) do not fit the file")
        self.metadata = {}
        for _ in range(n_kv):
            key = c.string()
            self.metadata[key] = c.value(c.take("<I"))
        self.alignment = int(self.metadata.get("general.alignment", DEFAULT_ALIGNMENT))
        if self.alignment <= 0 or self.alignment & (self.alignment - 1):
            raise GGUFError(f"general.alignment = {self.alignment} is not a power of two")
        self.tensors = {}
        for _ in range(n_tensors):
            name = c.string()
            nd = c.take("<I")
            if not 1 <= nd <= MAX_DIMS:
                raise GGUFError(f"tensor {name}: {nd} dimensions (want 1..{MAX_DIMS})")
            dims = tuple(c.take("<Q") for _ in range(nd))
            if any(d <= 0 for d in dims):
                raise GGUFError(f"tensor {name}: dims {dims} contain a zero")
            gtype, off = c.take("<I"), c.take("<Q")
            nbytes = tensor_nbytes(gtype, dims) if gtype in GGML_TYPES else -1
            self.tensors[name] = TensorInfo(name, dims, gtype, off, nbytes)
        self.data_start = (c.pos + self.alignment - 1) // self.alignment * self.alignment
        for t in self.tensors.values():
            if t.nbytes >= 0 and (t.offset % self.alignment or self.data_start + t.offset + t.nbytes > len(self._map)):
                raise GGUFError(f"tensor {t.name}: misaligned or outside the file")

    def data(self, name: str) -> np.ndarray:
        """The tensor's bytes as a read-only uint8 view of the mapping."""
        t = self.tensors[name]
        if t.nbytes < 0:
            raise GGUFError(f"tensor {name}: ggml type {t.ggml_type} is not supported")
        start = self.data_start + t.offset
        return self._map[start:start + t.nbytes]

    def upload(self, backend, name: str):
        """Upload a quantized 2-D tensor [n, k]; returns backend.QuantizedTensor."""
        t = self.tensors[name]
        if t.ggml_type not in (2, 8, 12, 13, 14):
            raise GGUFError(f"tensor {name}: type {GGML_TYPES.get(t.ggml_type, (0, 0, t.ggml_type))[2]} is not a quantized weight format of this backend")
        return backend.upload_weight(t.ggml_type, self.data(name), t.n, t.k)


def _pack_string(s: str) -> bytes:
    b = s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _pack_value(vtype, v) -> bytes:
    if vtype in _SCALAR:
        return struct.pack(_SCALAR[vtype], v)
    if vtype == STRING:
        return _pack_string(v)
    if vtype == ARRAY:
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(_pack_value(et, i) for i in items)
    raise GGUFError(f"unknown metadata value type {vtype}")


def write_gguf(path: str, metadata: dict, tensors: list, alignment: int = DEFAULT_ALIGNMENT) -> None:
    """metadata: key -> (value type, value) (arrays: (ARRAY, (element type, list)));
    tensors: list of (name, dims in ggml order, ggml type, uint8 array of the tensor's bytes)."""
    md = dict(metadata)
    if alignment != DEFAULT_ALIGNMENT:
        md["general.alignment"] = (U32, alignment)
    head = MAGIC + struct.pack("<IQQ", 3, len(tensors), len(md))
    for key, (vt, v) in md.items():
        head += _pack_string(key) + struct.pack("<I", vt) + _pack_value(vt, v)
    offset, infos, blobs = 0, b"", []
    for name, dims, gtype, data in tensors:
        data = np.ascontiguousarray(data, dtype=np.uint8).reshape(-1)
        if data.size != tensor_nbytes(gtype, dims):
            raise GGUFError(f"tensor {name}: {data.size} bytes given, {tensor_nbytes(gtype, dims)} expected")
        infos += _pack_string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", gtype, offset)
        blobs.append((offset, data))
        offset = (offset + data.size + alignment - 1) // alignment * alignment
    head += infos
    pad = (-len(head)) % alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        pos = 0
        for off, data in blobs:
            f.write(b"\0" * (off - pos))
            f.write(data.tobytes())
            pos = off + data.size
