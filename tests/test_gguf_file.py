"""GGUF container: writer and reader round-trip each other and follow the published layout."""
import struct

import numpy as np
import pytest

from oracle import gguf_oracle as go
from sensenova_u1_amd.gguf_file import (GGML_QUANT_SIZES, GGMLQuantizationType, GGUFReader, GGUFValueType, GGUFWriter,
                                        NativeGGUFReader, write_gguf)

READERS = [GGUFReader, NativeGGUFReader]     # pure Python, and the C++ reader inside libsngguf.so


@pytest.mark.parametrize("Reader", READERS)
def test_round_trip_all_supported_types(tmp_path, Reader):
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
    with Reader(path) as r:
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


@pytest.mark.parametrize("Reader", READERS)
def test_custom_alignment_and_v2(tmp_path, Reader):
    path = str(tmp_path / "a.gguf")
    w = GGUFWriter(path, alignment=64)
    w.add_tensor("x", np.arange(5, dtype=np.float32), 0)
    w.add_tensor("y", np.arange(3, dtype=np.float32), 0)
    w.write()
    with Reader(path) as r:
        assert r.alignment == 64 and all(t.data_offset % 64 == 0 for t in r.tensors)
        assert np.array_equal(r.tensors[1].data, np.arange(3, dtype=np.float32))
    raw = bytearray(open(path, "rb").read())
    raw[4:8] = struct.pack("<I", 2)
    open(path, "wb").write(raw)
    with Reader(path) as r:
        assert r.version == 2


@pytest.mark.parametrize("Reader", READERS)
def test_reader_rejects_garbage(tmp_path, Reader):
    bad = tmp_path / "bad.gguf"
    bad.write_bytes(b"NOPE" + b"\x00" * 64)
    with pytest.raises(ValueError, match="magic"):
        Reader(str(bad))
    bad.write_bytes(struct.pack("<IIQQ", 0x46554747, 9, 0, 0))
    with pytest.raises(ValueError, match="version"):
        Reader(str(bad))
    good = tmp_path / "good.gguf"
    write_gguf(str(good), [("w", np.zeros((4, 68), dtype=np.uint8), 8)])
    raw = good.read_bytes()
    bad.write_bytes(raw[:len(raw) - 40])                         # payload cut short
    with pytest.raises(ValueError, match="past the end|truncated"):
        Reader(str(bad))
    bad.write_bytes(raw[:30])                                    # header cut short
    with pytest.raises(ValueError):
        Reader(str(bad))
    bad.write_bytes(b"")
    with pytest.raises(ValueError):
        Reader(str(bad))


def _rich_file(path):
    """Every metadata value type, nested and string arrays, scalar / 1-d / 3-d tensors of several types."""
    rng = np.random.default_rng(5)
    w = GGUFWriter(path)
    for key, vt, val in [("m.u8", GGUFValueType.UINT8, 200), ("m.i8", GGUFValueType.INT8, -100),
                         ("m.u16", GGUFValueType.UINT16, 60000), ("m.i16", GGUFValueType.INT16, -30000),
                         ("m.u32", GGUFValueType.UINT32, 4000000000), ("m.i32", GGUFValueType.INT32, -2000000000),
                         ("m.f32", GGUFValueType.FLOAT32, 0.5), ("m.bool", GGUFValueType.BOOL, True),
                         ("m.u64", GGUFValueType.UINT64, 2 ** 63 + 5), ("m.i64", GGUFValueType.INT64, -2 ** 62),
                         ("m.f64", GGUFValueType.FLOAT64, 1e300), ("m.empty", GGUFValueType.STRING, "")]:
        w.add_metadata(key, val, vt)
    w.add_metadata("m.strs", (GGUFValueType.STRING, ["a", "", "längere Zeichenkette"]), GGUFValueType.ARRAY)
    w.add_metadata("m.none", (GGUFValueType.FLOAT32, []), GGUFValueType.ARRAY)
    tensors = [("s", np.array(3.5, dtype=np.float32).reshape(()), 0), ("v", rng.standard_normal(11).astype(np.float16), 1),
               ("c", rng.integers(0, 256, (2, 3, 2 * 18), dtype=np.uint8), 2), ("i", np.arange(6, dtype=np.int32).reshape(2, 3), 26),
               ("k", rng.integers(0, 256, (5, 110), dtype=np.uint8), 11), ("z", np.zeros((0, 34), dtype=np.uint8), 8)]
    for name, arr, t in tensors:
        w.add_tensor(name, arr, t)
    w.write()
    return tensors


def test_native_reader_agrees_with_python_reader(tmp_path):
    path = str(tmp_path / "rich.gguf")
    tensors = _rich_file(path)
    with GGUFReader(path) as a, NativeGGUFReader(path) as b:
        assert a.fields == b.fields and list(a.fields) == list(b.fields)
        assert b.fields["m.u64"] == 2 ** 63 + 5 and b.fields["m.strs"] == ["a", "", "längere Zeichenkette"]
        assert (a.version, a.alignment, len(a.tensors)) == (b.version, b.alignment, len(b.tensors))
        for ta, tb, (name, arr, t) in zip(a.tensors, b.tensors, tensors):
            assert (ta.name, ta.tensor_type, ta.shape, ta.n_elements, ta.n_bytes, ta.data_offset) == \
                   (tb.name, tb.tensor_type, tb.shape, tb.n_elements, tb.n_bytes, tb.data_offset)
            assert tb.name == name and int(tb.tensor_type) == t
            assert ta.data.dtype == tb.data.dtype and ta.data.shape == tb.data.shape
            assert np.array_equal(ta.data, tb.data) and np.array_equal(tb.data.reshape(arr.shape), arr)
            assert not tb.data.flags.writeable


def test_native_read_into(tmp_path):
    """Multi-threaded payload copy: several tensors, one larger than a copy piece, out of file order."""
    import torch
    rng = np.random.default_rng(6)
    big = rng.integers(0, 256, (300, 1024 // 32 * 34 * 32), dtype=np.uint8)     # 10.4 MB > one 8 MiB piece
    small = rng.standard_normal((5, 7)).astype(np.float32)
    path = str(tmp_path / "big.gguf")
    write_gguf(path, [("big", big, 8), ("small", small, 0), ("empty", np.zeros((0, 34), dtype=np.uint8), 8)])
    with NativeGGUFReader(path) as r:
        out_small = np.empty_like(small)
        out_big = torch.empty(big.shape, dtype=torch.uint8)
        out_empty = torch.empty((0, 34), dtype=torch.uint8)
        for threads in (1, 4, 100):
            out_small[:] = 0
            out_big.zero_()
            r.read_into([1, 2, 0], [out_small, out_empty, out_big], threads=threads)
            assert np.array_equal(out_small, small) and np.array_equal(out_big.numpy(), big)
        with pytest.raises(ValueError, match="needs"):
            r.read_into([0], [np.empty(10, dtype=np.uint8)])
        assert r._lib.sngguf_file_read_tensors(r._handle, None, None, 0, 1) == 0
        tmp = np.empty(4, dtype=np.uint8)
    # a bad index is refused, not followed
    import ctypes
    with NativeGGUFReader(path) as r:
        idx = (ctypes.c_int64 * 1)(7)
        dst = (ctypes.c_void_p * 1)(tmp.ctypes.data)
        assert r._lib.sngguf_file_read_tensors(r._handle, idx, dst, 1, 1) == -2


def test_native_reader_survives_every_truncation_and_bit_flips(tmp_path):
    """A small file cut at every length and with single bytes of the header / infos overwritten: the
    C++ parser must either parse or refuse with ValueError, never read outside the mapping."""
    path = str(tmp_path / "rich.gguf")
    _rich_file(path)
    raw = open(path, "rb").read()
    bad = str(tmp_path / "cut.gguf")
    n_ok = 0
    for n in range(0, len(raw)):
        open(bad, "wb").write(raw[:n])
        try:
            with NativeGGUFReader(bad) as r:
                for t in r.tensors:
                    t.data.sum()
            n_ok += 1
        except ValueError:
            pass
    assert n_ok == 0                     # the last tensor with bytes ("k") ends the file: every cut loses something
    with GGUFReader(path) as ref:
        header_end = min(t.data_offset for t in ref.tensors)
    rng = np.random.default_rng(7)
    parsed = 0
    for _ in range(600):
        buf = bytearray(raw)
        pos = int(rng.integers(4, header_end))
        buf[pos] = int(rng.integers(0, 256))
        open(bad, "wb").write(buf)
        try:
            with NativeGGUFReader(bad) as r:
                for t in r.tensors:
                    t.data.sum()
                parsed += 1
        except ValueError:
            pass
    assert parsed > 0                    # e.g. a changed metadata value still parses
    with pytest.raises(OSError):
        NativeGGUFReader(str(tmp_path / "does_not_exist.gguf"))


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
