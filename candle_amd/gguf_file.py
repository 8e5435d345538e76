"""GGUF files: header, metadata and tensor directory, tensors loaded into device buffers, and the writer.

Host-side mirror of candle-core/src/quantized/gguf_file.rs (``Content::read``, ``Content::tensor``, ``TensorInfo::read``,
``Value``, ``write``) with the same limits and error texts, so that the reference's tests for the format
(candle-core/tests/gguf_tests.rs) read the same here.  Readers are binary file objects (``read`` / ``seek`` / ``tell``),
the counterpart of ``R: Read + Seek``.  Tensor data goes from the file to HBM as the raw blocks
(``QStorage.from_data``, mod.rs:94-133); nothing is converted on the way.
"""
from __future__ import annotations

import enum
import struct
from typing import BinaryIO, Dict, List, Sequence, Tuple

from .quantized import GgmlDType, QStorage, QTensor

DEFAULT_ALIGNMENT = 32                      # gguf_file.rs:10

# gguf_file.rs:16-19
GGUF_MAX_STRING_LENGTH = 1 << 30
GGUF_MAX_ARRAY_ELEMENTS = 1 << 30
GGUF_MAX_TENSOR_DIMS = 4
GGUF_MAX_VALUE_DEPTH = 64


class GgufError(ValueError):
    """What the reference reports through ``crate::bail!``."""


def _read_exact(reader: BinaryIO, n: int) -> bytes:
    b = reader.read(n)
    if len(b) != n:
        raise GgufError("failed to fill whole buffer")          # std::io::ErrorKind::UnexpectedEof
    return b


def _u8(r):  return _read_exact(r, 1)[0]
def _u32(r): return struct.unpack("<I", _read_exact(r, 4))[0]
def _u64(r): return struct.unpack("<Q", _read_exact(r, 8))[0]


def _file_size(reader: BinaryIO) -> int:
    cur = reader.tell()
    end = reader.seek(0, 2)
    reader.seek(cur)
    return end


def _remaining_bytes(reader: BinaryIO, file_size: int) -> int:
    return max(file_size - reader.tell(), 0)                     # gguf_file.rs:23-26


class VersionedMagic(enum.Enum):
    """gguf_file.rs:51-79."""
    GgufV1 = 1
    GgufV2 = 2
    GgufV3 = 3

    @staticmethod
    def read(reader: BinaryIO) -> "VersionedMagic":
        magic = _u32(reader)
        if magic not in (0x46554747, 0x47475546):
            raise GgufError(f"unknown magic 0x{magic:08x}")
        version = _u32(reader)
        if version not in (1, 2, 3):
            raise GgufError(f"gguf: unsupported magic/version Gguf/{version}")
        return VersionedMagic(version)

    def length_prefix_size(self) -> int:
        return 4 if self is VersionedMagic.GgufV1 else 8


def _read_length(reader: BinaryIO, magic: VersionedMagic) -> int:
    return _u32(reader) if magic is VersionedMagic.GgufV1 else _u64(reader)    # gguf_file.rs:28-33


def _read_string(reader: BinaryIO, magic: VersionedMagic, file_size: int) -> str:
    """gguf_file.rs:130-151."""
    n = _read_length(reader, magic)
    if n > GGUF_MAX_STRING_LENGTH:
        raise GgufError(f"gguf: string length {n} exceeds max {GGUF_MAX_STRING_LENGTH}")
    remaining = _remaining_bytes(reader, file_size)
    if n > remaining:
        raise GgufError(f"gguf: string length {n} exceeds remaining file bytes {remaining}")
    v = _read_exact(reader, n)
    return v.rstrip(b"\x00").decode("utf-8", errors="replace")   # trailing NULs dropped, invalid utf-8 replaced


class ValueType(enum.IntEnum):
    """The on-disk codes (gguf_file.rs:410-448)."""
    U8 = 0
    I8 = 1
    U16 = 2
    I16 = 3
    U32 = 4
    I32 = 5
    F32 = 6
    Bool = 7
    String = 8
    Array = 9
    U64 = 10
    I64 = 11
    F64 = 12

    @staticmethod
    def from_u32(v: int) -> "ValueType":
        try:
            return ValueType(v)
        except ValueError:
            raise GgufError(f"unrecognized value-type {v:#08x}") from None

    def to_u32(self) -> int:
        return int(self)

    def min_disk_size(self, magic: VersionedMagic) -> int:
        """gguf_file.rs:452-462."""
        if self in (ValueType.U8, ValueType.I8, ValueType.Bool):
            return 1
        if self in (ValueType.U16, ValueType.I16):
            return 2
        if self in (ValueType.U32, ValueType.I32, ValueType.F32):
            return 4
        if self in (ValueType.U64, ValueType.I64, ValueType.F64):
            return 8
        if self is ValueType.String:
            return magic.length_prefix_size()
        return 4 + magic.length_prefix_size()


_SCALAR_FMT = {ValueType.U8: "<B", ValueType.I8: "<b", ValueType.U16: "<H", ValueType.I16: "<h", ValueType.U32: "<I",
               ValueType.I32: "<i", ValueType.U64: "<Q", ValueType.I64: "<q", ValueType.F32: "<f", ValueType.F64: "<d"}


class Value:
    """A metadata value with its GGUF type (gguf_file.rs:185-408).  ``v`` is an int / float / bool / str, or a list of
    ``Value`` for an array."""
    __slots__ = ("type", "v")

    def __init__(self, value_type: ValueType, v):
        self.type, self.v = ValueType(value_type), v

    # constructors named after the enum variants
    @staticmethod
    def U8(v): return Value(ValueType.U8, int(v))
    @staticmethod
    def I8(v): return Value(ValueType.I8, int(v))
    @staticmethod
    def U16(v): return Value(ValueType.U16, int(v))
    @staticmethod
    def I16(v): return Value(ValueType.I16, int(v))
    @staticmethod
    def U32(v): return Value(ValueType.U32, int(v))
    @staticmethod
    def I32(v): return Value(ValueType.I32, int(v))
    @staticmethod
    def U64(v): return Value(ValueType.U64, int(v))
    @staticmethod
    def I64(v): return Value(ValueType.I64, int(v))
    @staticmethod
    def F32(v): return Value(ValueType.F32, float(v))
    @staticmethod
    def F64(v): return Value(ValueType.F64, float(v))
    @staticmethod
    def Bool(v): return Value(ValueType.Bool, bool(v))
    @staticmethod
    def String(v): return Value(ValueType.String, str(v))
    @staticmethod
    def Array(v): return Value(ValueType.Array, list(v))

    def value_type(self) -> ValueType:
        return self.type

    def __repr__(self) -> str:
        return f"{self.type.name}({self.v!r})"

    def __eq__(self, other) -> bool:
        return isinstance(other, Value) and self.type == other.type and self.v == other.v

    def _expect(self, t: ValueType, what: str):
        if self.type != t:
            raise GgufError(f"not a {what} {self!r}")
        return self.v

    def to_u8(self): return self._expect(ValueType.U8, "u8")
    def to_i8(self): return self._expect(ValueType.I8, "i8")
    def to_u16(self): return self._expect(ValueType.U16, "u16")
    def to_i16(self): return self._expect(ValueType.I16, "i16")
    def to_u32(self): return self._expect(ValueType.U32, "u32")
    def to_i32(self): return self._expect(ValueType.I32, "i32")
    def to_i64(self): return self._expect(ValueType.I64, "i64")
    def to_f32(self): return self._expect(ValueType.F32, "f32")
    def to_f64(self): return self._expect(ValueType.F64, "f64")
    def to_bool(self): return self._expect(ValueType.Bool, "bool")
    def to_vec(self): return self._expect(ValueType.Array, "vec")
    def to_string(self): return self._expect(ValueType.String, "string")

    def to_u64(self) -> int:
        """Also upcasts the integral types that cannot truncate (gguf_file.rs:268-279)."""
        if self.type in (ValueType.U64, ValueType.U8, ValueType.U16, ValueType.U32, ValueType.Bool):
            return int(self.v)
        raise GgufError(f"not a u64 or upcastable to u64 {self!r}")

    @staticmethod
    def read(reader: BinaryIO, value_type: ValueType, magic: VersionedMagic, depth: int, file_size: int) -> "Value":
        """gguf_file.rs:323-374."""
        if depth > GGUF_MAX_VALUE_DEPTH:
            raise GgufError(f"gguf: value nesting depth exceeds max {GGUF_MAX_VALUE_DEPTH}")
        if value_type in _SCALAR_FMT:
            fmt = _SCALAR_FMT[value_type]
            return Value(value_type, struct.unpack(fmt, _read_exact(reader, struct.calcsize(fmt)))[0])
        if value_type is ValueType.Bool:
            b = _u8(reader)
            if b > 1:
                raise GgufError(f"unexpected bool value {b}")
            return Value(ValueType.Bool, b == 1)
        if value_type is ValueType.String:
            return Value(ValueType.String, _read_string(reader, magic, file_size))
        inner = ValueType.from_u32(_u32(reader))
        n = _read_length(reader, magic)
        if n > GGUF_MAX_ARRAY_ELEMENTS:
            raise GgufError(f"gguf: array length {n} exceeds max {GGUF_MAX_ARRAY_ELEMENTS}")
        needed = n * inner.min_disk_size(magic)
        remaining = _remaining_bytes(reader, file_size)
        if needed > remaining:
            raise GgufError(f"gguf: array of {n} elements needs at least {needed} bytes, only {remaining} remaining")
        return Value(ValueType.Array, [Value.read(reader, inner, magic, depth + 1, file_size) for _ in range(n)])

    def write(self, w: BinaryIO) -> None:
        """gguf_file.rs:376-407."""
        if self.type in _SCALAR_FMT:
            w.write(struct.pack(_SCALAR_FMT[self.type], self.v))
        elif self.type is ValueType.Bool:
            w.write(struct.pack("<B", 1 if self.v else 0))
        elif self.type is ValueType.String:
            _write_string(w, self.v)
        else:
            if not self.v:
                inner = ValueType.U32                            # does not matter, the array is empty
            else:
                kinds = {e.value_type() for e in self.v}
                if len(kinds) != 1:
                    raise GgufError(f"multiple value-types in the same array {sorted(k.name for k in kinds)}")
                inner = kinds.pop()
            w.write(struct.pack("<IQ", inner.to_u32(), len(self.v)))
            for e in self.v:
                e.write(w)


class TensorInfo:
    """gguf_file.rs:81-120."""
    __slots__ = ("ggml_dtype", "shape", "offset")

    def __init__(self, ggml_dtype: GgmlDType, shape: Sequence[int], offset: int):
        self.ggml_dtype, self.shape, self.offset = GgmlDType(ggml_dtype), tuple(int(d) for d in shape), int(offset)

    def elem_count(self) -> int:
        n = 1
        for d in self.shape:
            n *= d
        return n

    def size_in_bytes(self) -> int:
        tensor_elems, block_size = self.elem_count(), self.ggml_dtype.block_size()
        if tensor_elems % block_size:
            raise GgufError(f"the number of elements {tensor_elems} is not divisible by the block size {block_size}")
        return tensor_elems // block_size * self.ggml_dtype.type_size()

    def read_bytes(self, reader: BinaryIO, tensor_data_offset: int) -> bytes:
        """The raw blocks of the tensor, after the bounds check of gguf_file.rs:96-110."""
        size_in_bytes = self.size_in_bytes()
        tensor_start = tensor_data_offset + self.offset
        remaining = max(_file_size(reader) - tensor_start, 0)
        if size_in_bytes > remaining:
            raise GgufError(f"tensor needs {size_in_bytes} bytes at offset {tensor_start}, only {remaining} remaining in file")
        reader.seek(tensor_start)
        return _read_exact(reader, size_in_bytes)

    def read(self, reader: BinaryIO, tensor_data_offset: int, device) -> QTensor:
        """The tensor as raw blocks in HBM (ggml_file.rs qtensor_from_ggml -> QStorage::from_data)."""
        raw = self.read_bytes(reader, tensor_data_offset)
        return QTensor.new(QStorage.from_data(raw, device, self.ggml_dtype), self.shape)


class Content:
    """gguf_file.rs:122-128, 464-560."""

    def __init__(self, magic: VersionedMagic, metadata: Dict[str, Value], tensor_infos: Dict[str, TensorInfo], tensor_data_offset: int):
        self.magic, self.metadata, self.tensor_infos, self.tensor_data_offset = magic, metadata, tensor_infos, tensor_data_offset

    @staticmethod
    def read(reader: BinaryIO) -> "Content":
        file_size = _file_size(reader)
        magic = VersionedMagic.read(reader)
        tensor_count = _read_length(reader, magic)
        metadata_kv_count = _read_length(reader, magic)
        if tensor_count > GGUF_MAX_ARRAY_ELEMENTS:
            raise GgufError(f"gguf: tensor_count {tensor_count} exceeds max {GGUF_MAX_ARRAY_ELEMENTS}")
        if metadata_kv_count > GGUF_MAX_ARRAY_ELEMENTS:
            raise GgufError(f"gguf: metadata_kv_count {metadata_kv_count} exceeds max {GGUF_MAX_ARRAY_ELEMENTS}")
        # counts that cannot fit in the file at minimum entry size (gguf_file.rs:488-503)
        prefix = magic.length_prefix_size()
        needed = metadata_kv_count * (prefix + 4 + 1) + tensor_count * (prefix + 4 + 4 + 8)
        remaining = _remaining_bytes(reader, file_size)
        if needed > remaining:
            raise GgufError(f"gguf: header declares {tensor_count} tensors and {metadata_kv_count} metadata entries, "
                            f"needs at least {needed} bytes, only {remaining} remaining")
        metadata: Dict[str, Value] = {}
        for _ in range(metadata_kv_count):
            key = _read_string(reader, magic, file_size)
            value_type = ValueType.from_u32(_u32(reader))
            metadata[key] = Value.read(reader, value_type, magic, 0, file_size)
        tensor_infos: Dict[str, TensorInfo] = {}
        for _ in range(tensor_count):
            name = _read_string(reader, magic, file_size)
            n_dimensions = _u32(reader)
            if n_dimensions > GGUF_MAX_TENSOR_DIMS:
                raise GgufError(f"gguf: tensor '{name}' has {n_dimensions} dimensions, max is {GGUF_MAX_TENSOR_DIMS}")
            if magic is VersionedMagic.GgufV1:
                dims = list(struct.unpack(f"<{n_dimensions}I", _read_exact(reader, 4 * n_dimensions)))
            else:
                dims = list(struct.unpack(f"<{n_dimensions}Q", _read_exact(reader, 8 * n_dimensions)))
            dims.reverse()                                       # the file lists the fastest dimension first
            ggml_dtype = GgmlDType.from_u32(_u32(reader))
            offset = _u64(reader)
            tensor_infos[name] = TensorInfo(ggml_dtype, dims, offset)
        position = reader.tell()
        alignment = DEFAULT_ALIGNMENT
        a = metadata.get("general.alignment")
        if a is not None and a.type in (ValueType.U8, ValueType.U16, ValueType.U32):
            alignment = a.v
        elif a is not None and a.type in (ValueType.I8, ValueType.I16, ValueType.I32) and a.v >= 0:
            alignment = a.v
        if alignment == 0:
            raise GgufError("attempt to divide by zero")         # the reference panics on a zero alignment
        tensor_data_offset = -(-position // alignment) * alignment
        return Content(magic, metadata, tensor_infos, tensor_data_offset)

    def tensor(self, reader: BinaryIO, name: str, device) -> QTensor:
        info = self.tensor_infos.get(name)
        if info is None:
            raise GgufError(f"cannot find tensor info for {name}")
        return info.read(reader, self.tensor_data_offset, device)

    def tensor_bytes(self, reader: BinaryIO, name: str) -> Tuple[TensorInfo, bytes]:
        """The directory entry and the raw blocks of a tensor, left on the host (for callers that place the blocks
        themselves, e.g. a model that keeps all its weights in one allocation)."""
        info = self.tensor_infos.get(name)
        if info is None:
            raise GgufError(f"cannot find tensor info for {name}")
        return info, info.read_bytes(reader, self.tensor_data_offset)


def _write_string(w: BinaryIO, s: str) -> None:
    b = s.encode("utf-8")
    w.write(struct.pack("<Q", len(b)))
    w.write(b)


def write(w: BinaryIO, metadata: Sequence[Tuple[str, Value]], tensors: Sequence[Tuple[str, object]]) -> None:
    """gguf_file.rs:569-638: a version-2 file, tensor data aligned to 32 bytes.  A tensor is anything with ``shape()``,
    ``dtype()``, ``storage_size_in_bytes()`` and ``data()`` (``QTensor``)."""
    w.write(struct.pack("<IIQQ", 0x46554747, 2, len(tensors), len(metadata)))
    for name, value in metadata:
        _write_string(w, name)
        w.write(struct.pack("<I", value.value_type().to_u32()))
        value.write(w)
    offset = 0
    offsets: List[int] = []
    for name, tensor in tensors:
        _write_string(w, name)
        dims = tuple(tensor.shape())
        w.write(struct.pack("<I", len(dims)))
        for dim in reversed(dims):
            w.write(struct.pack("<Q", dim))
        w.write(struct.pack("<IQ", GgmlDType(tensor.dtype()).to_u32(), offset))
        offsets.append(offset)
        size_in_bytes = tensor.storage_size_in_bytes()
        offset += size_in_bytes + (31 - (31 + size_in_bytes) % 32)
    pos = w.tell()
    w.write(bytes(31 - (31 + pos) % 32))
    tensor_start_pos = w.tell()
    for off, (_name, tensor) in zip(offsets, tensors):
        pos = w.tell()
        if tensor_start_pos + off != pos:
            raise GgufError(f"internal error, unexpected current position {tensor_start_pos} {off} {pos}")
        data = tensor.data()
        w.write(data)
        w.write(bytes(31 - (31 + len(data)) % 32))
