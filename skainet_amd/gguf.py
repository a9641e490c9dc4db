"""GGUF container reader (64-bit offsets, memory-mapped) and a minimal writer for tests.

Same container semantics as the reference reader (gguf/src/commonMain/kotlin/sk/ai/net/gguf/GGUFReader.kt):
magic 0x46554747 little-endian (:159-165, Constants.kt:10), versions 2 and 3 (:141-157), u64 tensor and KV counts
(:116-139), KV records = key string, u32 type, value (:285-318, :187-250), tensor infos = name, u32 n_dims,
u64 dims[], u32 ggml type, u64 offset (:252-283), data section aligned to general.alignment or 32 (:104-111),
element count = product of dims, byte count = n_elems * type_size / block (:354-360), dims reversed for
row-major shapes (:356), quantized tensors handed out as raw block bytes with the last axis in bytes
(Quants.kt:10-20).  Where the reference stops -- Int offsets (< 2 GiB), boxing every byte, no F16, six of the
eleven scalar KV types -- this reader goes on: int64 offsets over an mmap, zero-copy tensor views, all scalar types.
"""
from __future__ import annotations

import mmap
import struct

import numpy as np

GGUF_MAGIC = 0x46554747
SUPPORTED_VERSIONS = (2, 3)
DEFAULT_ALIGNMENT = 32

# GGUFValueType (Constants.kt:92-106)
_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
T_STRING, T_ARRAY = 8, 9

# (block elems, block bytes), GGML_QUANT_SIZES (Constants.kt:58-90)
QUANT_SIZES = {
    0: (1, 4), 1: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 40),
    10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292),
    16: (256, 66), 17: (256, 74), 18: (256, 98), 19: (256, 50), 20: (32, 18), 21: (256, 110), 22: (256, 82),
    23: (256, 136), 24: (1, 1), 25: (1, 2), 26: (1, 4), 27: (1, 8), 28: (1, 8), 29: (256, 56), 30: (1, 2),
    34: (256, 54), 35: (256, 66),
}
_DENSE = {0: np.float32, 1: np.float16, 24: np.int8, 25: np.int16, 26: np.int32, 27: np.int64, 28: np.float64}
TYPE_NAMES = {0: "F32", 1: "F16", 8: "Q8_0", 12: "Q4_K", 14: "Q6_K", 30: "BF16"}


class ReaderTensor:
    def __init__(self, name, ggml_type, dims, n_bytes, data_offset, data):
        self.name, self.tensor_type, self.dims = name, ggml_type, tuple(dims)
        self.shape = tuple(reversed(dims))  # row-major: GGUF stores the fastest axis first
        self.n_elements = int(np.prod(dims, dtype=np.int64)) if dims else 1
        self.n_bytes, self.data_offset, self.data = n_bytes, data_offset, data

    @property
    def byte_shape(self):
        """quantShapeToByteShape: the last axis in bytes for block types."""
        block, tsize = QUANT_SIZES[self.tensor_type]
        if self.shape[-1] % block:
            raise ValueError(
                f"Quantized tensor row size ({self.shape[-1]}) is not a multiple of "
                f"{TYPE_NAMES.get(self.tensor_type, self.tensor_type)} block size ({block})"
            )
        return self.shape[:-1] + (self.shape[-1] // block * tsize,)


class GGUFReader:
    def __init__(self, path):
        self._f = open(path, "rb")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        self.fields, self.tensors = {}, []
        self.alignment = DEFAULT_ALIGNMENT
        mm = self._mm
        if len(mm) < 24 or struct.unpack_from("<I", mm, 0)[0] != GGUF_MAGIC:
            raise ValueError("GGUF magic invalid")
        self.version = struct.unpack_from("<I", mm, 4)[0]
        if self.version not in SUPPORTED_VERSIONS:
            raise ValueError(f"Unsupported GGUF version: {self.version}")
        n_tensors, n_kv = struct.unpack_from("<QQ", mm, 8)
        off = 24
        for _ in range(n_kv):
            key, off = self._string(off)
            (vtype,) = struct.unpack_from("<I", mm, off)
            value, off = self._value(off + 4, vtype)
            if key in self.fields:  # the reference keeps duplicates under name_offset (GGUFReader.kt:168-176)
                key = f"{key}_{off}"
            self.fields[key] = value
        infos = []
        names = set()
        for _ in range(n_tensors):
            name, off = self._string(off)
            (n_dims,) = struct.unpack_from("<I", mm, off)
            dims = struct.unpack_from(f"<{n_dims}Q", mm, off + 4)
            ggml_type, t_off = struct.unpack_from("<IQ", mm, off + 4 + 8 * n_dims)
            off += 4 + 8 * n_dims + 12
            if name in names:
                raise ValueError(f"buildTensors: Found duplicated tensor with name {name}")
            names.add(name)
            infos.append((name, ggml_type, dims, t_off))
        align = self.fields.get("general.alignment")
        if isinstance(align, int) and align > 0:
            self.alignment = align
        self.data_offset = off + (-off % self.alignment)
        for name, ggml_type, dims, t_off in infos:
            if ggml_type not in QUANT_SIZES:
                raise ValueError("Invalid ggmlType")
            block, tsize = QUANT_SIZES[ggml_type]
            n_elems = int(np.prod(dims, dtype=np.int64)) if dims else 1
            n_bytes = n_elems * tsize // block
            start = self.data_offset + t_off
            if start + n_bytes > len(mm):
                raise ValueError(f"tensor {name} extends past the end of the file")
            raw = np.frombuffer(mm, dtype=np.uint8, count=n_bytes, offset=start)
            if ggml_type in _DENSE:
                data = raw.view(_DENSE[ggml_type]).reshape(tuple(reversed(dims)))
            else:
                data = raw  # block bytes, exactly what the device kernels read
            self.tensors.append(ReaderTensor(name, ggml_type, dims, n_bytes, start, data))

    def _string(self, off):
        (n,) = struct.unpack_from("<Q", self._mm, off)
        return self._mm[off + 8:off + 8 + n].decode("utf-8"), off + 8 + n

    def _value(self, off, vtype):
        if vtype == T_STRING:
            return self._string(off)
        if vtype in _SCALARS:
            fmt = _SCALARS[vtype]
            return struct.unpack_from(fmt, self._mm, off)[0], off + struct.calcsize(fmt)
        if vtype == T_ARRAY:
            itype, n = struct.unpack_from("<IQ", self._mm, off)
            off += 12
            out = []
            for _ in range(n):
                v, off = self._value(off, itype)
                out.append(v)
            return out, off
        raise ValueError(f"GGUFValueType {vtype} not defined")

    def tensor(self, name):
        for t in self.tensors:
            if t.name == name:
                return t
        raise KeyError(name)

    def close(self):
        self.tensors = []
        try:
            self._mm.close()
        except BufferError:  # views of the map are still alive; the map goes with them
            pass
        self._f.close()


def write_gguf(path, fields, tensors, alignment=DEFAULT_ALIGNMENT):
    """Minimal GGUF v3 writer: fields = {key: str | int (u32) | float (f32)}, tensors = [(name, ggml_type, shape, bytes-like)]
    with `shape` row-major (it is stored reversed, as GGUF wants)."""

    def s(x):
        b = x.encode("utf-8")
        return struct.pack("<Q", len(b)) + b

    head = struct.pack("<IIQQ", GGUF_MAGIC, 3, len(tensors), len(fields))
    for k, v in fields.items():
        head += s(k)
        if isinstance(v, str):
            head += struct.pack("<I", T_STRING) + s(v)
        elif isinstance(v, bool):
            head += struct.pack("<I?", 7, v)
        elif isinstance(v, int):
            head += struct.pack("<II", 4, v)
        elif isinstance(v, float):
            head += struct.pack("<If", 6, v)
        else:
            raise TypeError(f"unsupported field value {v!r}")
    blobs, off = [], 0
    for name, ggml_type, shape, data in tensors:
        raw = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        dims = tuple(reversed(shape))
        head += s(name) + struct.pack(f"<I{len(dims)}QIQ", len(dims), *dims, ggml_type, off)
        blobs.append((off, raw))
        off += raw.size + (-raw.size % alignment)
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * (-len(head) % alignment))
        base = f.tell()
        for o, raw in blobs:
            f.seek(base + o)
            f.write(raw.tobytes())
        f.truncate(base + off)
