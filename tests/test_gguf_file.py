"""The GGUF reader / writer (candle_amd/gguf_file.py) against the reference's own tests of the format
(candle-core/tests/gguf_tests.rs: every case below builds the same bytes and expects the same outcome) and against
what the format fixes: every value type survives a write -> read round trip, tensor offsets are 32-byte aligned and the
directory reproduces names, shapes (fastest dimension first on disk), types and bytes."""
import io
import struct

import numpy as np
import pytest

from candle_amd import gguf_file as gf
from candle_amd.quantized import GgmlDType

GGUF_MAGIC = b"GGUF"


def header(tensor_count, metadata_kv_count, version=3):
    return GGUF_MAGIC + struct.pack("<IQQ", version, tensor_count, metadata_kv_count)


def length_prefixed(s: bytes) -> bytes:
    return struct.pack("<Q", len(s)) + s


def assert_rejects(buf: bytes, msg_contains: str):
    with pytest.raises(gf.GgufError) as e:
        gf.Content.read(io.BytesIO(buf))
    assert msg_contains in str(e.value), str(e.value)


# ---- gguf_tests.rs, case by case ----
def test_empty_header_loads():
    c = gf.Content.read(io.BytesIO(header(0, 0)))
    assert c.metadata == {} and c.tensor_infos == {}


def test_rejects_oversized_metadata_kv_count():
    assert_rejects(header(0, 1 << 31), "metadata_kv_count")


def test_rejects_oversized_tensor_count():
    assert_rejects(header(1 << 31, 0), "tensor_count")


def test_rejects_oversized_string_length():
    assert_rejects(header(1, 0) + struct.pack("<Q", 1 << 31) + bytes(64), "string length")


def test_rejects_oversized_array_length():
    buf = header(0, 1) + length_prefixed(b"k") + struct.pack("<IIQ", 9, 0, 1 << 31) + bytes(64)
    assert_rejects(buf, "array length")


def test_rejects_oversized_n_dimensions():
    buf = header(1, 0) + length_prefixed(b"t") + struct.pack("<I", 0xFFFFFFFF) + bytes(64)
    assert_rejects(buf, "dimensions")


def test_rejects_deeply_nested_arrays():
    buf = header(0, 1) + length_prefixed(b"k") + struct.pack("<I", 9)
    for _ in range(256):
        buf += struct.pack("<IQ", 9, 1)
    buf += struct.pack("<IQ", 0, 0)
    assert_rejects(buf, "nesting depth")


def test_empty_v1_header_loads():
    gf.Content.read(io.BytesIO(GGUF_MAGIC + struct.pack("<III", 1, 0, 0)))


def test_rejects_tensor_size_exceeding_file():
    buf = header(1, 0) + length_prefixed(b"t") + struct.pack("<IQIQ", 1, 1_073_741_824, 0, 0)
    r = io.BytesIO(buf)
    c = gf.Content.read(r)
    with pytest.raises(gf.GgufError) as e:
        c.tensor_bytes(r, "t")
    assert "remaining" in str(e.value)


def test_rejects_string_length_above_remaining_file_bytes():
    assert_rejects(header(1, 0) + struct.pack("<Q", 1 << 20) + bytes(64), "string length")


# ---- the rest of the reader's contract ----
def test_unknown_magic_and_version():
    assert_rejects(b"GGML" + struct.pack("<IQQ", 3, 0, 0), "unknown magic")
    assert_rejects(header(0, 0, version=4), "unsupported magic/version")


def test_header_counts_must_fit_the_file():
    assert_rejects(header(3, 0), "needs at least")


def test_unknown_value_type_and_bool_byte():
    assert_rejects(header(0, 1) + length_prefixed(b"k") + struct.pack("<I", 13) + bytes(8), "unrecognized value-type")
    assert_rejects(header(0, 1) + length_prefixed(b"k") + struct.pack("<IB", 7, 2), "unexpected bool value")


def test_strings_drop_trailing_nuls_and_survive_bad_utf8():
    buf = header(0, 2) + length_prefixed(b"a\x00\x00") + struct.pack("<I", 8) + length_prefixed(b"x\xffy") + \
        length_prefixed(b"b") + struct.pack("<IB", 7, 1)
    c = gf.Content.read(io.BytesIO(buf))
    assert c.metadata["a"].to_string() == "x�y" and c.metadata["b"].to_bool() is True


def test_v1_uses_32_bit_lengths_and_dimensions():
    buf = GGUF_MAGIC + struct.pack("<III", 1, 1, 1)
    buf += struct.pack("<I", 1) + b"k" + struct.pack("<II", 4, 77)                       # k: U32 = 77
    buf += struct.pack("<I", 1) + b"t" + struct.pack("<III", 2, 256, 3) + struct.pack("<IQ", 12, 0)
    c = gf.Content.read(io.BytesIO(buf))
    assert c.metadata["k"].to_u32() == 77
    t = c.tensor_infos["t"]
    assert t.shape == (3, 256) and t.ggml_dtype == GgmlDType.Q4K and t.size_in_bytes() == 3 * 144


def test_alignment_key_moves_the_tensor_data():
    for val, want in ((gf.Value.U32(64), 64), (gf.Value.I16(16), 16), (gf.Value.I32(-8), 32), (gf.Value.U64(128), 32)):
        w = io.BytesIO()
        gf.write(w, [("general.alignment", val)], [])
        end_of_directory = w.getvalue().rfind(b"general.alignment") + len("general.alignment") + 4 + val.type.min_disk_size(gf.VersionedMagic.GgufV2)
        c = gf.Content.read(io.BytesIO(w.getvalue()))
        assert c.tensor_data_offset == -(-end_of_directory // want) * want


def test_value_accessors_and_upcasts():
    v = gf.Value.U16(9)
    assert v.to_u16() == 9 and v.to_u64() == 9
    assert gf.Value.Bool(True).to_u64() == 1
    for bad in (lambda: v.to_u32(), lambda: gf.Value.I32(1).to_u64(), lambda: gf.Value.String("s").to_f32()):
        with pytest.raises(gf.GgufError):
            bad()


class HostTensor:
    """Stand-in for a QTensor on a machine without a GPU: the four things the writer asks of a tensor."""

    def __init__(self, dtype, shape, data):
        self._dtype, self._shape, self._data = GgmlDType(dtype), tuple(shape), bytes(data)

    def shape(self): return self._shape
    def dtype(self): return self._dtype
    def storage_size_in_bytes(self): return len(self._data)
    def data(self): return self._data


def test_write_read_round_trip():
    rng = np.random.default_rng(3)
    md = [("general.architecture", gf.Value.String("llama")), ("u8", gf.Value.U8(200)), ("i8", gf.Value.I8(-7)), ("u16", gf.Value.U16(65000)),
          ("i16", gf.Value.I16(-30000)), ("u32", gf.Value.U32(4_000_000_000)), ("i32", gf.Value.I32(-5)), ("u64", gf.Value.U64(1 << 40)),
          ("i64", gf.Value.I64(-(1 << 40))), ("f32", gf.Value.F32(1.5)), ("f64", gf.Value.F64(-2.25)), ("flag", gf.Value.Bool(False)),
          ("empty", gf.Value.Array([])), ("tokens", gf.Value.Array([gf.Value.String("a"), gf.Value.String("bc")])),
          ("nested", gf.Value.Array([gf.Value.Array([gf.Value.I32(1), gf.Value.I32(2)]), gf.Value.Array([gf.Value.I32(3)])]))]
    tensors = [("blk.0.attn_q.weight", HostTensor(GgmlDType.Q4K, (4, 512), rng.integers(0, 256, 4 * 2 * 144, dtype=np.uint8).tobytes())),
               ("output_norm.weight", HostTensor(GgmlDType.F32, (7,), np.arange(7, dtype=np.float32).tobytes())),
               ("w6", HostTensor(GgmlDType.Q6K, (2, 3, 256), rng.integers(0, 256, 6 * 210, dtype=np.uint8).tobytes()))]
    w = io.BytesIO()
    gf.write(w, md, tensors)
    r = io.BytesIO(w.getvalue())
    c = gf.Content.read(r)
    assert c.magic is gf.VersionedMagic.GgufV2 and c.tensor_data_offset % 32 == 0
    assert c.metadata == dict(md)
    assert c.metadata["empty"].to_vec() == [] and c.metadata["nested"].to_vec()[0].to_vec()[1].to_i32() == 2
    for name, t in tensors:
        info, raw = c.tensor_bytes(r, name)
        assert info.shape == t.shape() and info.ggml_dtype == t.dtype() and raw == t.data() and info.offset % 32 == 0
    # the fastest dimension comes first on disk
    pos = w.getvalue().find(b"w6") + 2
    assert struct.unpack("<IQQQ", w.getvalue()[pos:pos + 28]) == (3, 256, 3, 2)
    with pytest.raises(gf.GgufError):
        c.tensor_bytes(r, "missing")
    with pytest.raises(gf.GgufError):
        gf.write(io.BytesIO(), [("mixed", gf.Value.Array([gf.Value.U8(1), gf.Value.I8(1)]))], [])


def test_tensor_elements_must_fill_whole_blocks():
    with pytest.raises(gf.GgufError) as e:
        gf.TensorInfo(GgmlDType.Q4K, (3, 100), 0).size_in_bytes()
    assert "not divisible by the block size" in str(e.value)
