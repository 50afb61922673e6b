"""Minimal GGUF (v2 / v3) container reader and writer.

The reference parses files with the third-party ``gguf`` package
(``src/sensenova_u1/utils/gguf_loader.py:29-33``: ``GGUFReader(path).tensors`` with ``.name``,
``.tensor_type`` and ``.data``).  This module provides those three attributes, the
``GGMLQuantizationType`` numbering and ``GGML_QUANT_SIZES`` from the public GGUF
specification, so that the loader needs no external package; the writer exists so that tests
and tools can produce files.  ``NativeGGUFReader`` gives the same view through the C++ reader
of libsngguf.so (``sngguf_file_*``) and is what the checkpoint loader uses; ``GGUFReader`` is
the pure-Python counterpart.

Layout (little endian): magic ``GGUF``, u32 version, u64 tensor count, u64 metadata count,
metadata key/values, tensor infos (name, u32 n_dims, u64 dims fastest-first, u32 type, u64
offset), padding to ``general.alignment`` (default 32), tensor data.
"""
from __future__ import annotations

import ctypes
import mmap
import os
import struct
from enum import IntEnum
from typing import Any, Iterable

import numpy as np

GGUF_MAGIC = 0x46554747
GGUF_DEFAULT_ALIGNMENT = 32


class GGMLQuantizationType(IntEnum):
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
    IQ2_XXS = 16
    IQ2_XS = 17
    IQ3_XXS = 18
    IQ1_S = 19
    IQ4_NL = 20
    IQ3_S = 21
    IQ2_S = 22
    IQ4_XS = 23
    I8 = 24
    I16 = 25
    I32 = 26
    I64 = 27
    F64 = 28
    IQ1_M = 29
    BF16 = 30


# type -> (elements per block, bytes per block)
GGML_QUANT_SIZES: dict[GGMLQuantizationType, tuple[int, int]] = {
    GGMLQuantizationType.F32: (1, 4),
    GGMLQuantizationType.F16: (1, 2),
    GGMLQuantizationType.Q4_0: (32, 18),
    GGMLQuantizationType.Q4_1: (32, 20),
    GGMLQuantizationType.Q5_0: (32, 22),
    GGMLQuantizationType.Q5_1: (32, 24),
    GGMLQuantizationType.Q8_0: (32, 34),
    GGMLQuantizationType.Q8_1: (32, 36),
    GGMLQuantizationType.Q2_K: (256, 84),
    GGMLQuantizationType.Q3_K: (256, 110),
    GGMLQuantizationType.Q4_K: (256, 144),
    GGMLQuantizationType.Q5_K: (256, 176),
    GGMLQuantizationType.Q6_K: (256, 210),
    GGMLQuantizationType.Q8_K: (256, 292),
    GGMLQuantizationType.I8: (1, 1),
    GGMLQuantizationType.I16: (1, 2),
    GGMLQuantizationType.I32: (1, 4),
    GGMLQuantizationType.I64: (1, 8),
    GGMLQuantizationType.F64: (1, 8),
    GGMLQuantizationType.BF16: (1, 2),
}

_PLAIN_DTYPES = {
    GGMLQuantizationType.F32: np.float32,
    GGMLQuantizationType.F16: np.float16,
    GGMLQuantizationType.F64: np.float64,
    GGMLQuantizationType.I8: np.int8,
    GGMLQuantizationType.I16: np.int16,
    GGMLQuantizationType.I32: np.int32,
    GGMLQuantizationType.I64: np.int64,
}


class GGUFValueType(IntEnum):
    UINT8 = 0
    INT8 = 1
    UINT16 = 2
    INT16 = 3
    UINT32 = 4
    INT32 = 5
    FLOAT32 = 6
    BOOL = 7
    STRING = 8
    ARRAY = 9
    UINT64 = 10
    INT64 = 11
    FLOAT64 = 12


_SCALAR_FMT = {
    GGUFValueType.UINT8: "<B", GGUFValueType.INT8: "<b", GGUFValueType.UINT16: "<H", GGUFValueType.INT16: "<h",
    GGUFValueType.UINT32: "<I", GGUFValueType.INT32: "<i", GGUFValueType.FLOAT32: "<f", GGUFValueType.BOOL: "<?",
    GGUFValueType.UINT64: "<Q", GGUFValueType.INT64: "<q", GGUFValueType.FLOAT64: "<d",
}


class ReaderTensor:
    """One tensor of a GGUF file: ``name``, ``tensor_type``, ``shape`` (ggml order, fastest dim
    first) and ``data`` - a read-only numpy view into the mapped file.  Quantized tensors come
    as uint8 with the row length in bytes; F32/F16 and integer types come typed."""

    __slots__ = ("name", "tensor_type", "shape", "n_elements", "n_bytes", "data_offset", "data")

    def __init__(self, name, tensor_type, shape, n_elements, n_bytes, data_offset, data):
        self.name = name
        self.tensor_type = tensor_type
        self.shape = shape
        self.n_elements = n_elements
        self.n_bytes = n_bytes
        self.data_offset = data_offset
        self.data = data


class GGUFReader:
    """Parses header, metadata and tensor infos; tensor payloads stay memory-mapped."""

    def __init__(self, path: str):
        self._file = open(path, "rb")
        try:
            self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        except ValueError as exc:  # empty file
            self._file.close()
            raise ValueError(f"{path}: not a GGUF file (empty)") from exc
        self._buf = memoryview(self._map)
        self._pos = 0
        self.fields: dict[str, Any] = {}
        self.tensors: list[ReaderTensor] = []
        try:
            self._parse(path)
        except (struct.error, IndexError) as exc:
            raise ValueError(f"{path}: truncated or corrupt GGUF file") from exc

    # -- low-level reads
    def _unpack(self, fmt: str):
        size = struct.calcsize(fmt)
        if self._pos + size > len(self._buf):
            raise IndexError("read past end of file")
        (v,) = struct.unpack_from(fmt, self._buf, self._pos)
        self._pos += size
        return v

    def _string(self) -> str:
        n = self._unpack("<Q")
        if self._pos + n > len(self._buf):
            raise IndexError("string past end of file")
        s = bytes(self._buf[self._pos:self._pos + n]).decode("utf-8", errors="replace")
        self._pos += n
        return s

    def _value(self, vtype: int):
        vtype = GGUFValueType(vtype)
        if vtype == GGUFValueType.STRING:
            return self._string()
        if vtype == GGUFValueType.ARRAY:
            item_type = self._unpack("<I")
            count = self._unpack("<Q")
            return [self._value(item_type) for _ in range(count)]
        return self._unpack(_SCALAR_FMT[vtype])

    def _parse(self, path: str) -> None:
        if self._unpack("<I") != GGUF_MAGIC:
            raise ValueError(f"{path}: bad magic, not a GGUF file")
        self.version = self._unpack("<I")
        if self.version not in (2, 3):
            raise ValueError(f"{path}: unsupported GGUF version {self.version}")
        n_tensors = self._unpack("<Q")
        n_kv = self._unpack("<Q")
        for _ in range(n_kv):
            key = self._string()
            self.fields[key] = self._value(self._unpack("<I"))
        infos = []
        for _ in range(n_tensors):
            name = self._string()
            n_dims = self._unpack("<I")
            dims = [self._unpack("<Q") for _ in range(n_dims)]
            ttype = self._unpack("<I")
            offset = self._unpack("<Q")
            infos.append((name, dims, ttype, offset))
        self.alignment = int(self.fields.get("general.alignment", GGUF_DEFAULT_ALIGNMENT))
        self.data_offset = (self._pos + self.alignment - 1) // self.alignment * self.alignment
        for name, dims, ttype, offset in infos:
            try:
                qtype = GGMLQuantizationType(ttype)
            except ValueError as exc:
                raise ValueError(f"{path}: tensor {name} has unknown ggml type {ttype}") from exc
            if qtype not in GGML_QUANT_SIZES:
                raise ValueError(f"{path}: tensor {name} has ggml type {qtype.name} whose block size is not known")
            block, tsize = GGML_QUANT_SIZES[qtype]
            n_elem = int(np.prod(dims, dtype=np.int64)) if dims else 1
            if dims and dims[0] % block != 0:
                raise ValueError(f"{path}: tensor {name}: row length {dims[0]} is not a multiple of block size {block}")
            n_bytes = n_elem // block * tsize
            start = self.data_offset + offset
            if start + n_bytes > len(self._buf):
                raise ValueError(f"{path}: tensor {name} runs past the end of the file")
            np_dims = list(reversed(dims)) if dims else [1]
            if qtype in _PLAIN_DTYPES:
                arr = np.frombuffer(self._buf, dtype=_PLAIN_DTYPES[qtype], count=n_elem, offset=start).reshape(np_dims)
            else:
                np_dims[-1] = np_dims[-1] // block * tsize
                arr = np.frombuffer(self._buf, dtype=np.uint8, count=n_bytes, offset=start).reshape(np_dims)
            self.tensors.append(ReaderTensor(name, qtype, list(dims), n_elem, n_bytes, start, arr))

    def close(self) -> None:
        self.tensors = []
        self._buf.release()
        try:
            self._map.close()
        except BufferError:
            pass  # numpy views handed out earlier still pin the mapping; it goes with them
        self._file.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


class _TensorInfo(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char_p), ("ggml_type", ctypes.c_int32), ("n_dims", ctypes.c_int32),
                ("dims", ctypes.c_int64 * 4), ("n_elements", ctypes.c_int64), ("n_bytes", ctypes.c_int64),
                ("file_offset", ctypes.c_int64), ("data", ctypes.c_void_p)]


class _MetadataInfo(ctypes.Structure):
    _fields_ = [("key", ctypes.c_char_p), ("value_type", ctypes.c_int32), ("item_type", ctypes.c_int32),
                ("count", ctypes.c_int64), ("value", ctypes.c_void_p), ("value_bytes", ctypes.c_int64)]


def _decode_value(buf: bytes, pos: int, vtype: int):
    """One encoded GGUF metadata value at ``buf[pos:]`` -> (python value, next position)."""
    vtype = GGUFValueType(vtype)
    if vtype == GGUFValueType.STRING:
        (n,) = struct.unpack_from("<Q", buf, pos)
        return buf[pos + 8:pos + 8 + n].decode("utf-8", errors="replace"), pos + 8 + n
    if vtype == GGUFValueType.ARRAY:
        item_type, count = struct.unpack_from("<IQ", buf, pos)
        pos += 12
        items = []
        for _ in range(count):
            v, pos = _decode_value(buf, pos, item_type)
            items.append(v)
        return items, pos
    fmt = _SCALAR_FMT[vtype]
    (v,) = struct.unpack_from(fmt, buf, pos)
    return v, pos + struct.calcsize(fmt)


class NativeGGUFReader:
    """The same view of a file as ``GGUFReader`` (``version``, ``alignment``, ``fields``, ``tensors``
    with numpy views into the mapping), parsed and mapped by the C++ reader inside libsngguf.so.
    ``read_into`` copies payloads to caller-chosen host buffers with several threads."""

    def __init__(self, path: str):
        from . import ops
        self._lib = ops.load_library()
        handle = ctypes.c_void_p()
        err = ctypes.create_string_buffer(1024)
        rc = self._lib.sngguf_file_open(os.fsencode(path), ctypes.byref(handle), err, len(err))
        if rc != 0:
            msg = err.value.decode("utf-8", errors="replace")
            if rc == -7:
                raise OSError(msg)
            raise ValueError(msg if msg.startswith(path) else f"{path}: {msg}")
        self._handle = handle
        self.version = self._lib.sngguf_file_version(handle)
        self.alignment = self._lib.sngguf_file_alignment(handle)
        self.fields: dict[str, Any] = {}
        info = _MetadataInfo()
        for i in range(self._lib.sngguf_file_metadata_count(handle)):
            self._lib.sngguf_file_metadata(handle, i, ctypes.byref(info))
            raw = ctypes.string_at(info.value, info.value_bytes)
            self.fields[info.key.decode("utf-8", errors="replace")] = _decode_value(raw, 0, info.value_type)[0]
        self.tensors: list[ReaderTensor] = []
        tinfo = _TensorInfo()
        for i in range(self._lib.sngguf_file_tensor_count(handle)):
            self._lib.sngguf_file_tensor(handle, i, ctypes.byref(tinfo))
            name = tinfo.name.decode("utf-8", errors="replace")
            try:
                qtype = GGMLQuantizationType(tinfo.ggml_type)
            except ValueError as exc:
                self.close()
                raise ValueError(f"{path}: tensor {name} has unknown ggml type {tinfo.ggml_type}") from exc
            block, tsize = GGML_QUANT_SIZES[qtype]
            dims = [int(tinfo.dims[d]) for d in range(tinfo.n_dims)]
            np_dims = list(reversed(dims)) if dims else [1]
            if tinfo.n_bytes:
                flat = np.ctypeslib.as_array(ctypes.cast(tinfo.data, ctypes.POINTER(ctypes.c_uint8)), shape=(tinfo.n_bytes,))
            else:
                flat = np.empty((0,), dtype=np.uint8)
            flat.flags.writeable = False
            if qtype in _PLAIN_DTYPES:
                arr = flat.view(_PLAIN_DTYPES[qtype]).reshape(np_dims)
            else:
                np_dims[-1] = np_dims[-1] // block * tsize
                arr = flat.reshape(np_dims)
            self.tensors.append(ReaderTensor(name, qtype, dims, int(tinfo.n_elements), int(tinfo.n_bytes),
                                             int(tinfo.file_offset), arr))

    def read_into(self, indices, buffers, threads: int = 8) -> None:
        """Copy the payloads of tensors ``indices`` (positions in ``tensors``) into ``buffers``:
        objects with the buffer protocol or ``data_ptr()`` (torch tensors), each at least as large."""
        n = len(indices)
        idx = (ctypes.c_int64 * n)(*indices)
        dst = (ctypes.c_void_p * n)()
        for i, (t, b) in enumerate(zip(indices, buffers)):
            need = self.tensors[t].n_bytes
            if hasattr(b, "data_ptr"):
                have, ptr = b.numel() * b.element_size(), b.data_ptr()
                if not b.is_contiguous() or b.device.type != "cpu":
                    raise ValueError("read_into needs contiguous host tensors")
            else:
                view = np.asarray(b)
                if not view.flags.c_contiguous or not view.flags.writeable:
                    raise ValueError("read_into needs contiguous writable buffers")
                have, ptr = view.nbytes, view.ctypes.data
            if have < need:
                raise ValueError(f"buffer for tensor {self.tensors[t].name} holds {have} bytes, needs {need}")
            dst[i] = ptr
        rc = self._lib.sngguf_file_read_tensors(self._handle, idx, dst, n, int(threads))
        if rc != 0:
            raise RuntimeError(f"sngguf_file_read_tensors failed: {rc}")

    def close(self) -> None:
        """Unmaps the file: arrays in ``tensors`` must not be used afterwards."""
        self.tensors = []
        if getattr(self, "_handle", None):
            self._lib.sngguf_file_close(self._handle)
            self._handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class GGUFWriter:
    """Writes a GGUF v3 file.  ``add_tensor(name, array, tensor_type)``: plain types take a typed
    array of the logical shape, quantized types take uint8 rows of packed blocks
    ``[..., row_bytes]``."""

    def __init__(self, path: str, arch: str = "sensenova_u1", alignment: int = GGUF_DEFAULT_ALIGNMENT):
        self.path = path
        self.alignment = alignment
        self._kv: list[tuple[str, GGUFValueType, Any]] = [("general.architecture", GGUFValueType.STRING, arch)]
        if alignment != GGUF_DEFAULT_ALIGNMENT:
            self._kv.append(("general.alignment", GGUFValueType.UINT32, alignment))
        self._tensors: list[tuple[str, list[int], GGMLQuantizationType, np.ndarray]] = []

    def add_metadata(self, key: str, value, vtype: GGUFValueType | None = None) -> None:
        if vtype is None:
            if isinstance(value, bool):
                vtype = GGUFValueType.BOOL
            elif isinstance(value, int):
                vtype = GGUFValueType.INT64
            elif isinstance(value, float):
                vtype = GGUFValueType.FLOAT64
            elif isinstance(value, str):
                vtype = GGUFValueType.STRING
            else:
                raise TypeError(f"cannot infer GGUF value type of {type(value)}")
        self._kv.append((key, vtype, value))

    def add_tensor(self, name: str, array: np.ndarray, tensor_type: GGMLQuantizationType | int) -> None:
        qtype = GGMLQuantizationType(tensor_type)
        block, tsize = GGML_QUANT_SIZES[qtype]
        arr = np.ascontiguousarray(array)
        if qtype in _PLAIN_DTYPES:
            arr = arr.astype(_PLAIN_DTYPES[qtype], copy=False)
            shape = list(arr.shape)
        else:
            if arr.dtype != np.uint8:
                raise TypeError(f"{name}: quantized tensors are given as uint8 packed rows")
            if arr.shape[-1] % tsize != 0:
                raise ValueError(f"{name}: row of {arr.shape[-1]} bytes is not a multiple of {tsize}")
            shape = list(arr.shape)
            shape[-1] = shape[-1] // tsize * block
        self._tensors.append((name, list(reversed(shape)), qtype, arr))

    @staticmethod
    def _pack_string(s: str) -> bytes:
        b = s.encode("utf-8")
        return struct.pack("<Q", len(b)) + b

    def _pack_value(self, vtype: GGUFValueType, value) -> bytes:
        if vtype == GGUFValueType.STRING:
            return self._pack_string(value)
        if vtype == GGUFValueType.ARRAY:
            item_type, items = value
            return struct.pack("<IQ", int(item_type), len(items)) + b"".join(
                self._pack_value(GGUFValueType(item_type), v) for v in items)
        return struct.pack(_SCALAR_FMT[vtype], value)

    def write(self) -> None:
        head = struct.pack("<IIQQ", GGUF_MAGIC, 3, len(self._tensors), len(self._kv))
        for key, vtype, value in self._kv:
            head += self._pack_string(key) + struct.pack("<I", int(vtype)) + self._pack_value(vtype, value)
        offset = 0
        offsets = []
        for name, dims, qtype, arr in self._tensors:
            offsets.append(offset)
            head += self._pack_string(name) + struct.pack("<I", len(dims))
            head += b"".join(struct.pack("<Q", d) for d in dims)
            head += struct.pack("<IQ", int(qtype), offset)
            offset += (arr.nbytes + self.alignment - 1) // self.alignment * self.alignment
        pad = (-len(head)) % self.alignment
        with open(self.path, "wb") as f:
            f.write(head + b"\x00" * pad)
            for (_, _, _, arr), off in zip(self._tensors, offsets):
                f.write(arr.tobytes())
                f.write(b"\x00" * ((-arr.nbytes) % self.alignment))


def write_gguf(path: str, tensors: Iterable[tuple[str, np.ndarray, int]], metadata: dict | None = None) -> None:
    """Convenience: write ``(name, array, ggml_type)`` triples to ``path``."""
    w = GGUFWriter(path)
    for k, v in (metadata or {}).items():
        w.add_metadata(k, v)
    for name, arr, t in tensors:
        w.add_tensor(name, arr, t)
    w.write()
