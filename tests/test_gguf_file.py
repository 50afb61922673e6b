"""GGUF container: writer and reader round-trip each other and follow the published layout."""
import struct

import numpy as np
import pytest

from oracle import gguf_oracle as go
from sensenova_u1_amd.gguf_file import (GGML_QUANT_SIZES, GGMLQuantizationType, GGUFReader, GGUFValueType, GGUFWriter,
                                        write_gguf)


def test_round_trip_all_supported_types(tmp_path):
    rng = np.random.default_rng(0)
    f32 = rng.standard_normal((3, 5)).astype(np.float32)
    f16 = rng.standard_normal((7,)).astype(np.float16)
    q8 = go.quantize_q8_0(rng.standard_normal((4, 64)).astype(np.float32))
    q4 = rng.integers(0, 256, (2, 2 * 144), dtype=np.uint8)
    q6 = rng.integers(0, 256, (3, 210), dtype=np.uint8)
    path = str(tmp_path / "t.gguf")
    w = GGUFWriter(path)
    w.add_metadata("test.int", 7)
    w.add_metadata("test.str", "héllo")
    w.add_metadata("test.arr", (GGUFValueType.INT32, [1, 2, 3]), GGUFValueType.ARRAY)
    for name, arr, t in [("a.weight", f32, 0), ("b.bias", f16, 1), ("c.weight", q8, 8), ("d.weight", q4, 12),
                         ("e.weight", q6, 14)]:
        w.add_tensor(name, arr, t)
    w.write()
    with GGUFReader(path) as r:
        assert r.version == 3 and r.fields["test.int"] == 7 and r.fields["test.str"] == "héllo"
        assert r.fields["test.arr"] == [1, 2, 3] and r.fields["general.architecture"] == "sensenova_u1"
        got = {t.name: t for t in r.tensors}
        assert [t.name for t in r.tensors] == ["a.weight", "b.bias", "c.weight", "d.weight", "e.weight"]
        assert np.array_equal(got["a.weight"].data, f32) and got["a.weight"].tensor_type == GGMLQuantizationType.F32
        assert np.array_equal(got["b.bias"].data, f16)
        assert np.array_equal(got["c.weight"].data, q8) and got["c.weight"].data.dtype == np.uint8
        assert got["c.weight"].shape == [64, 4]                  # ggml order: fastest dim first
        assert got["d.weight"].data.shape == (2, 288) and got["d.weight"].shape == [512, 2]
        assert np.array_equal(got["e.weight"].data, q6) and got["e.weight"].n_elements == 3 * 256
        for t in r.tensors:
            assert t.data_offset % 32 == 0                       # default alignment
            copy = t.data.copy()                                 # what the loader does


def test_header_bytes_follow_the_spec(tmp_path):
    path = str(tmp_path / "h.gguf")
    write_gguf(path, [("w", np.zeros((2, 34), dtype=np.uint8), 8)])
    raw = open(path, "rb").read()
    magic, version, n_tensors, n_kv = struct.unpack_from("<IIQQ", raw, 0)
    assert raw[:4] == b"GGUF" and magic == 0x46554747 and version == 3 and n_tensors == 1 and n_kv == 1
    # after the single KV pair: name "w", n_dims 2, dims (32, 2), type 8, offset 0
    tail = raw[raw.index(b"\x01\x00\x00\x00\x00\x00\x00\x00w"):]
    (n_dims,) = struct.unpack_from("<I", tail, 9)
    d0, d1 = struct.unpack_from("<QQ", tail, 13)
    ttype, off = struct.unpack_from("<IQ", tail, 29)
    assert (n_dims, d0, d1, ttype, off) == (2, 32, 2, 8, 0)
    assert len(raw) % 32 == 0


def test_custom_alignment_and_v2(tmp_path):
    path = str(tmp_path / "a.gguf")
    w = GGUFWriter(path, alignment=64)
    w.add_tensor("x", np.arange(5, dtype=np.float32), 0)
    w.add_tensor("y", np.arange(3, dtype=np.float32), 0)
    w.write()
    with GGUFReader(path) as r:
        assert r.alignment == 64 and all(t.data_offset % 64 == 0 for t in r.tensors)
        assert np.array_equal(r.tensors[1].data, np.arange(3, dtype=np.float32))
    raw = bytearray(open(path, "rb").read())
    raw[4:8] = struct.pack("<I", 2)
    open(path, "wb").write(raw)
    with GGUFReader(path) as r:
        assert r.version == 2


def test_reader_rejects_garbage(tmp_path):
    bad = tmp_path / "bad.gguf"
    bad.write_bytes(b"NOPE" + b"\x00" * 64)
    with pytest.raises(ValueError, match="magic"):
        GGUFReader(str(bad))
    bad.write_bytes(struct.pack("<IIQQ", 0x46554747, 9, 0, 0))
    with pytest.raises(ValueError, match="version"):
        GGUFReader(str(bad))
    good = tmp_path / "good.gguf"
    write_gguf(str(good), [("w", np.zeros((4, 68), dtype=np.uint8), 8)])
    raw = good.read_bytes()
    bad.write_bytes(raw[:len(raw) - 40])                         # payload cut short
    with pytest.raises(ValueError, match="past the end|truncated"):
        GGUFReader(str(bad))
    bad.write_bytes(raw[:30])                                    # header cut short
    with pytest.raises(ValueError):
        GGUFReader(str(bad))
    bad.write_bytes(b"")
    with pytest.raises(ValueError):
        GGUFReader(str(bad))


def test_writer_rejects_bad_rows(tmp_path):
    w = GGUFWriter(str(tmp_path / "x.gguf"))
    with pytest.raises(ValueError):
        w.add_tensor("w", np.zeros((2, 35), dtype=np.uint8), 8)
    with pytest.raises(TypeError):
        w.add_tensor("w", np.zeros((2, 34), dtype=np.float32), 8)


def test_quant_sizes_table():
    assert GGML_QUANT_SIZES[GGMLQuantizationType.Q8_0] == (32, 34)
    assert GGML_QUANT_SIZES[GGMLQuantizationType.Q4_K] == (256, 2 + 2 + 12 + 128)
    assert GGML_QUANT_SIZES[GGMLQuantizationType.Q6_K] == (256, 128 + 64 + 16 + 2)
    assert GGML_QUANT_SIZES[GGMLQuantizationType.Q5_K] == (256, 2 + 2 + 12 + 32 + 128)
    assert int(GGMLQuantizationType.Q8_0) == 8 and int(GGMLQuantizationType.Q4_K) == 12 and int(GGMLQuantizationType.Q6_K) == 14
