"""GGML tensor types as the reference's GGUF loader names them.

Mirrors `GGMLType` / `from_u32` / `type_size` of
example-cli/src/model/formats/gguf.rs:78-144 (same ids, same bytes per block).
"""
from __future__ import annotations

import enum


class GGMLType(enum.IntEnum):
    F32 = 0
    F16 = 1
    Q4_0 = 2
    Q4_1 = 3
    Q5_0 = 6
    Q5_1 = 7
    Q8_0 = 8
    Q8_1 = 9
    Q2_K = 10
    Q3_K = 11
    Q4_K = 12
    Q5_K = 13
    Q6_K = 14
    Q8_K = 15
    I8 = 16
    I16 = 17
    I32 = 18

    @classmethod
    def from_u32(cls, value: int) -> "GGMLType":
        try:
            return cls(value)
        except ValueError:
            raise ValueError("Unknown GGML type: %d" % value) from None

    def type_size(self) -> int:
        """Bytes per block (per element for the plain types)."""
        return _TYPE_SIZE[self]

    def block_elems(self) -> int:
        """Elements per block."""
        if self in (GGMLType.Q2_K, GGMLType.Q3_K, GGMLType.Q4_K, GGMLType.Q5_K, GGMLType.Q6_K, GGMLType.Q8_K):
            return 256
        if self in (GGMLType.Q4_0, GGMLType.Q4_1, GGMLType.Q5_0, GGMLType.Q5_1, GGMLType.Q8_0, GGMLType.Q8_1):
            return 32
        return 1

    def row_bytes(self, n_cols: int) -> int:
        be = self.block_elems()
        if n_cols % be:
            raise ValueError("n_cols=%d is not a multiple of the block size %d" % (n_cols, be))
        return n_cols // be * self.type_size()


_TYPE_SIZE = {
    GGMLType.F32: 4, GGMLType.I32: 4, GGMLType.F16: 2, GGMLType.I16: 2, GGMLType.I8: 1,
    GGMLType.Q4_0: 18, GGMLType.Q4_1: 20, GGMLType.Q5_0: 22, GGMLType.Q5_1: 24, GGMLType.Q8_0: 34,
    GGMLType.Q8_1: 36, GGMLType.Q2_K: 84,   # the public ggml block (16 + 64 + 2 * 2); the reference's table lists 82
    GGMLType.Q3_K: 110, GGMLType.Q4_K: 144, GGMLType.Q5_K: 176,
    GGMLType.Q6_K: 210, GGMLType.Q8_K: 292,
}


# ---------------------------------------------------------------------------------------------------------
# GGUF v3 container: reader mirroring `GGUFLoader` (example-cli/src/model/formats/gguf.rs:146-407) and a
# writer for synthetic model files.  All integers little-endian.  The reader finishes what the reference's
# `load_tensor_data` leaves unimplemented (gguf.rs:401-406): raw bytes of a tensor are read at
# tensor_data_offset + offset with the real block byte count and handed on untouched.

import struct
from dataclasses import dataclass, field
from typing import Any, BinaryIO, Dict, Iterable, List, Optional, Tuple

import numpy as np

GGUF_MAGIC = 0x46554747      # "GGUF"
GGUF_VERSION = 3
DEFAULT_ALIGNMENT = 32

# value type ids of the metadata section (gguf.rs:269-301)
(VT_UINT8, VT_INT8, VT_UINT16, VT_INT16, VT_UINT32, VT_INT32, VT_FLOAT32, VT_BOOL, VT_STRING, VT_ARRAY, VT_UINT64,
 VT_INT64, VT_FLOAT64) = range(13)
_SCALAR_FMT = {VT_UINT8: "<B", VT_INT8: "<b", VT_UINT16: "<H", VT_INT16: "<h", VT_UINT32: "<I", VT_INT32: "<i",
               VT_FLOAT32: "<f", VT_UINT64: "<Q", VT_INT64: "<q", VT_FLOAT64: "<d"}
_VT_NAMES = ("UInt8", "Int8", "UInt16", "Int16", "UInt32", "Int32", "Float32", "Bool", "String", "Array", "UInt64",
             "Int64", "Float64")


class GGUFError(ValueError):
    """Malformed container (the reference's `anyhow::bail!` cases)."""


@dataclass(frozen=True)
class GGUFValue:
    """One metadata value: `kind` is the GGUF value-type id, `value` the decoded Python object
    (arrays: list of GGUFValue, as the reference nests them)."""
    kind: int
    value: Any

    @property
    def kind_name(self) -> str:
        return _VT_NAMES[self.kind]

    def as_str(self) -> Optional[str]:
        return self.value if self.kind == VT_STRING else None

    def as_u32(self) -> Optional[int]:
        # UInt32, or UInt64 truncated (gguf.rs:52-58)
        if self.kind == VT_UINT32:
            return self.value
        if self.kind == VT_UINT64:
            return self.value & 0xFFFFFFFF
        return None

    def as_u64(self) -> Optional[int]:
        return self.value if self.kind in (VT_UINT64, VT_UINT32) else None

    def as_f32(self) -> Optional[float]:
        return self.value if self.kind in (VT_FLOAT32, VT_FLOAT64) else None

    def as_list(self) -> Optional[list]:
        return [v.value for v in self.value] if self.kind == VT_ARRAY else None


@dataclass(frozen=True)
class GGUFHeader:
    magic: int
    version: int
    tensor_count: int
    metadata_kv_count: int


@dataclass(frozen=True)
class GGUFTensorInfo:
    name: str
    n_dims: int
    dims: Tuple[int, ...]        # dims[0] is the contiguous (column / K) dimension
    ggml_type: GGMLType
    offset: int                  # relative to tensor_data_offset

    @property
    def n_elems(self) -> int:
        n = 1
        for d in self.dims:
            n *= d
        return n

    @property
    def n_cols(self) -> int:
        return self.dims[0] if self.dims else 1

    @property
    def n_rows(self) -> int:
        return self.n_elems // self.n_cols if self.n_cols else 0

    @property
    def n_bytes(self) -> int:
        return self.n_rows * self.ggml_type.row_bytes(self.n_cols)


class _Reader:
    def __init__(self, f: BinaryIO):
        self.f = f

    def take(self, n: int) -> bytes:
        b = self.f.read(n)
        if len(b) != n:
            raise GGUFError("unexpected end of file (wanted %d bytes, got %d)" % (n, len(b)))
        return b

    def scalar(self, fmt: str):
        return struct.unpack(fmt, self.take(struct.calcsize(fmt)))[0]

    def string(self) -> str:
        n = self.scalar("<Q")
        try:
            return self.take(n).decode("utf-8")
        except UnicodeDecodeError:
            raise GGUFError("Invalid UTF-8 in string") from None

    def value(self, vt: int) -> GGUFValue:
        if vt in _SCALAR_FMT:
            return GGUFValue(vt, self.scalar(_SCALAR_FMT[vt]))
        if vt == VT_BOOL:
            return GGUFValue(vt, self.scalar("<B") != 0)
        if vt == VT_STRING:
            return GGUFValue(vt, self.string())
        if vt == VT_ARRAY:
            et = self.scalar("<I")
            n = self.scalar("<Q")
            return GGUFValue(vt, [self.value(et) for _ in range(n)])
        raise GGUFError("Unknown value type: %d" % vt)


class GGUFLoader:
    """Parse header, metadata and tensor table of a GGUF file (same accessors as the reference's loader:
    header / metadata / tensors / get_metadata / find_tensor / get_tensor / tensor_names), and read tensors'
    raw bytes.  Data starts at the first multiple of the alignment after the tensor table; the alignment is
    `general.alignment` when the file states one, else 32 (the reference hard-codes 32, gguf.rs:189)."""

    def __init__(self, path):
        self.path = str(path)
        try:
            self._f = open(self.path, "rb")
        except OSError as e:
            raise GGUFError("Failed to open GGUF file: %s (%s)" % (self.path, e)) from None
        r = _Reader(self._f)
        magic = r.scalar("<I")
        if magic != GGUF_MAGIC:
            raise GGUFError("Invalid GGUF magic number: 0x%08x (expected 0x%08x)" % (magic, GGUF_MAGIC))
        version = r.scalar("<I")
        self.version_mismatch = version != GGUF_VERSION     # the reference only warns (gguf.rs:216-222)
        self.header = GGUFHeader(magic, version, r.scalar("<Q"), r.scalar("<Q"))
        self.metadata: Dict[str, GGUFValue] = {}
        for _ in range(self.header.metadata_kv_count):
            key = r.string()
            self.metadata[key] = r.value(r.scalar("<I"))
        self.tensors: List[GGUFTensorInfo] = []
        for _ in range(self.header.tensor_count):
            name = r.string()
            nd = r.scalar("<I")
            dims = tuple(r.scalar("<Q") for _ in range(nd))
            t = r.scalar("<I")
            try:
                gt = GGMLType.from_u32(t)
            except ValueError as e:
                raise GGUFError(str(e)) from None
            self.tensors.append(GGUFTensorInfo(name, nd, dims, gt, r.scalar("<Q")))
        al = self.metadata.get("general.alignment")
        self.alignment = (al.as_u32() or DEFAULT_ALIGNMENT) if al is not None else DEFAULT_ALIGNMENT
        pos = self._f.tell()
        self.tensor_data_offset = -(-pos // self.alignment) * self.alignment
        self._f.seek(0, 2)
        self.file_size = self._f.tell()

    # --- the reference's public accessors
    def get_metadata(self, key: str) -> Optional[GGUFValue]:
        return self.metadata.get(key)

    def find_tensor(self, name: str) -> Optional[GGUFTensorInfo]:
        for t in self.tensors:
            if t.name == name:
                return t
        return None

    get_tensor = find_tensor

    def tensor_names(self) -> List[str]:
        return [t.name for t in self.tensors]

    # --- tensor payloads
    def load_tensor_data(self, tensor_name: str) -> np.ndarray:
        """Raw bytes of one tensor, exactly as stored (quantized blocks are not decoded on the host)."""
        t = self.find_tensor(tensor_name)
        if t is None:
            raise GGUFError("Tensor not found: %s" % tensor_name)
        start = self.tensor_data_offset + t.offset
        if start + t.n_bytes > self.file_size:
            raise GGUFError("Tensor %s runs past the end of the file (%d + %d > %d)" % (t.name, start, t.n_bytes, self.file_size))
        self._f.seek(start)
        return np.frombuffer(_Reader(self._f).take(t.n_bytes), dtype=np.uint8)

    def load_f32(self, tensor_name: str) -> np.ndarray:
        """F32 / F16 / I8 / I16 / I32 tensors decoded to f32 (tensor_loader.rs:144-211,255-269)."""
        t = self.find_tensor(tensor_name)
        raw = self.load_tensor_data(tensor_name)
        np_t = {GGMLType.F32: "<f4", GGMLType.F16: "<f2", GGMLType.I8: "i1", GGMLType.I16: "<i2", GGMLType.I32: "<i4"}.get(t.ggml_type)
        if np_t is None:
            raise GGUFError("load_f32: %s holds %s blocks; upload them raw instead" % (t.name, t.ggml_type.name))
        return raw.view(np_t).astype(np.float32)

    def close(self) -> None:
        if self._f:
            self._f.close()
            self._f = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def _pack_value(vt: int, v) -> bytes:
    if vt in _SCALAR_FMT:
        return struct.pack(_SCALAR_FMT[vt], v)
    if vt == VT_BOOL:
        return struct.pack("<B", 1 if v else 0)
    if vt == VT_STRING:
        b = v.encode("utf-8")
        return struct.pack("<Q", len(b)) + b
    if vt == VT_ARRAY:
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(_pack_value(et, x) for x in items)
    raise GGUFError("Unknown value type: %d" % vt)


class GGUFWriter:
    """Write a GGUF v3 file: `add_kv(key, value_type, value)` (arrays: value = (element_type, items)),
    `add_tensor(name, ggml_type, dims, raw)` with dims[0] the contiguous dimension, then `write(path)`."""

    def __init__(self, alignment: int = DEFAULT_ALIGNMENT, state_alignment: bool = False):
        self.alignment = alignment
        self.kvs: List[Tuple[str, int, Any]] = []
        self.tensors: List[Tuple[str, GGMLType, Tuple[int, ...], np.ndarray]] = []
        if state_alignment or alignment != DEFAULT_ALIGNMENT:
            self.add_kv("general.alignment", VT_UINT32, alignment)

    def add_kv(self, key: str, vt: int, value) -> None:
        self.kvs.append((key, vt, value))

    def add_tensor(self, name: str, ggml_type: int, dims: Iterable[int], raw) -> None:
        gt = GGMLType(int(ggml_type))
        dims = tuple(int(d) for d in dims)
        raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        info = GGUFTensorInfo(name, len(dims), dims, gt, 0)
        if raw.nbytes != info.n_bytes:
            raise GGUFError("%s: %d bytes given, %s%r needs %d" % (name, raw.nbytes, gt.name, dims, info.n_bytes))
        self.tensors.append((name, gt, dims, raw))

    def write(self, path) -> None:
        head = struct.pack("<IIQQ", GGUF_MAGIC, GGUF_VERSION, len(self.tensors), len(self.kvs))
        for key, vt, v in self.kvs:
            head += _pack_value(VT_STRING, key) + struct.pack("<I", vt) + _pack_value(vt, v)
        off = 0
        offs = []
        for name, gt, dims, raw in self.tensors:
            offs.append(off)
            head += _pack_value(VT_STRING, name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
            head += struct.pack("<IQ", int(gt), off)
            off = -(-(off + raw.nbytes) // self.alignment) * self.alignment
        with open(path, "wb") as f:
            f.write(head)
            f.write(b"\0" * (-len(head) % self.alignment))
            base = f.tell()
            for (name, gt, dims, raw), o in zip(self.tensors, offs):
                f.write(b"\0" * (base + o - f.tell()))
                f.write(raw.tobytes())
