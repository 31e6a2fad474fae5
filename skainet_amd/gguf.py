"""GGUF files on disk -> packed weights on the device, without a copy in between.

Host-side mirror of the reference's streaming reader
(/root/reference/skainet-io/skainet-io-gguf/src/commonMain/kotlin/sk/ainet/io/gguf/StreamingGGUFReader.kt:217-368:
magic, version 2 / 3, metadata key-values, tensor infos with offsets relative to the aligned data section,
`general.alignment` override; value types Constants.kt:142-156; block geometry Constants.kt:102-130). The file is
memory-mapped and a tensor is handed to `skainet_hip_weight_upload` as a view of the mapping -- the bytes of a
Q4_K / Q6_K / Q8_0 tensor are already in the canonical row-major block order the kernels read
(`loadTensorViewMapped`, StreamingGGUFReader.kt:153), so nothing is repacked.

`GGUFWriter` writes the same format (used by the tests and to export synthetic models); it is not a converter.
"""
from __future__ import annotations

import mmap
import struct
from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np

GGUF_MAGIC = 0x46554747
SUPPORTED_VERSIONS = (2, 3)
DEFAULT_ALIGNMENT = 32

# ggml type id -> (name, elements per block, bytes per block)      (Constants.kt:25-54, 102-130)
GGML_TYPES = {
    0: ("F32", 1, 4), 1: ("F16", 1, 2), 2: ("Q4_0", 32, 18), 3: ("Q4_1", 32, 20), 6: ("Q5_0", 32, 22), 7: ("Q5_1", 32, 24),
    8: ("Q8_0", 32, 34), 9: ("Q8_1", 32, 36), 10: ("Q2_K", 256, 84), 11: ("Q3_K", 256, 110), 12: ("Q4_K", 256, 144),
    13: ("Q5_K", 256, 176), 14: ("Q6_K", 256, 210), 15: ("Q8_K", 256, 292), 24: ("I8", 1, 1), 25: ("I16", 1, 2),
    26: ("I32", 1, 4), 27: ("I64", 1, 8), 28: ("F64", 1, 8), 30: ("BF16", 1, 2),
}
TYPE_ID = {v[0]: k for k, v in GGML_TYPES.items()}
DEVICE_ENCODINGS = ("Q8_0", "Q4_K", "Q6_K", "Q4_0", "Q5_0", "Q5_1", "Q5_K")      # what the kernels consume packed

# metadata value types (Constants.kt:142-156)
_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
_STRING, _ARRAY = 8, 9


class GGUFError(ValueError):
    pass


@dataclass
class TensorInfo:
    name: str
    shape: tuple          # ggml order: shape[0] is the contiguous (input / column) dimension
    type_id: int
    type_name: str
    n_elements: int
    n_bytes: int
    offset: int           # absolute file offset of the first byte

    @property
    def rows(self) -> int:
        """Output rows of a 2-D weight (everything but the contiguous dimension)."""
        return self.n_elements // self.shape[0] if self.shape else 0

    @property
    def cols(self) -> int:
        return self.shape[0] if self.shape else 0


class GGUFReader:
    """Parses the header once; tensor bytes are views of a read-only memory mapping (no copy until upload)."""

    def __init__(self, path: str):
        self.path = path
        self._file = open(path, "rb")
        try:
            self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        except ValueError as e:                       # empty file
            self._file.close()
            raise GGUFError(f"{path}: not a GGUF file ({e})")
        self._buf = memoryview(self._map)
        self.fields: Dict[str, object] = {}
        self.tensors: List[TensorInfo] = []
        self.alignment = DEFAULT_ALIGNMENT
        self._pos = 0
        try:
            self._parse()
        except (struct.error, IndexError, UnicodeDecodeError) as e:
            self.close()
            raise GGUFError(f"{path}: truncated or corrupt GGUF header ({e})")
        except GGUFError:
            self.close()
            raise
        self._by_name = {t.name: t for t in self.tensors}

    # ------------------------------------------------------------------ parsing
    def _take(self, fmt: str):
        n = struct.calcsize(fmt)
        if self._pos + n > len(self._buf):
            raise GGUFError("unexpected end of file in the header")
        v = struct.unpack_from(fmt, self._buf, self._pos)[0]
        self._pos += n
        return v

    def _string(self) -> str:
        n = self._take("<Q")
        if self._pos + n > len(self._buf):
            raise GGUFError("string runs past the end of the file")
        s = bytes(self._buf[self._pos:self._pos + n]).decode("utf-8")
        self._pos += n
        return s

    def _value(self, vtype: int):
        if vtype in _SCALARS:
            return self._take(_SCALARS[vtype])
        if vtype == _STRING:
            return self._string()
        if vtype == _ARRAY:
            etype = self._take("<I")
            count = self._take("<Q")
            if etype in _SCALARS and etype != 7:
                dt = np.dtype(_SCALARS[etype])
                end = self._pos + count * dt.itemsize
                if end > len(self._buf):
                    raise GGUFError("array runs past the end of the file")
                out = np.frombuffer(self._buf, dtype=dt, count=count, offset=self._pos).copy()
                self._pos = end
                return out
            if count > len(self._buf):
                raise GGUFError("array length exceeds the file size")
            return [self._value(etype) for _ in range(count)]
        raise GGUFError(f"unknown metadata value type {vtype}")

    def _parse(self) -> None:
        magic = self._take("<I")
        if magic != GGUF_MAGIC:
            raise GGUFError(f"invalid GGUF magic: expected 0x{GGUF_MAGIC:x}, got 0x{magic:x}")
        self.version = self._take("<I")
        if self.version not in SUPPORTED_VERSIONS:
            raise GGUFError(f"unsupported GGUF version {self.version} (supported: {SUPPORTED_VERSIONS})")
        n_tensors = self._take("<Q")
        n_kv = self._take("<Q")
        for _ in range(n_kv):
            key = self._string()
            self.fields[key] = self._value(self._take("<I"))
        a = self.fields.get("general.alignment")
        if isinstance(a, int) and a > 0:
            self.alignment = a
        raw = []
        for _ in range(n_tensors):
            name = self._string()
            nd = self._take("<I")
            shape = tuple(self._take("<Q") for _ in range(nd))
            raw.append((name, shape, self._take("<I"), self._take("<Q")))
        data_start = (self._pos + self.alignment - 1) // self.alignment * self.alignment
        by_offset = sorted(r[3] for r in raw)
        for name, shape, tid, rel in raw:
            n_el = int(np.prod(shape, dtype=np.int64)) if shape else 0
            if tid in GGML_TYPES:
                tname, bs, nb = GGML_TYPES[tid]
                if shape and shape[0] % bs != 0:
                    raise GGUFError(f"tensor {name}: row length {shape[0]} is not a multiple of the {tname} block ({bs})")
                n_bytes = n_el // bs * nb
            else:                                     # unknown type: raw bytes up to the next tensor (reader's fallback)
                tname = f"UNKNOWN_{tid}"
                later = [o for o in by_offset if o > rel]
                n_bytes = (later[0] - rel) if later else max(0, len(self._buf) - data_start - rel)
            off = data_start + rel
            if off + n_bytes > len(self._buf):
                raise GGUFError(f"tensor {name}: data [{off}, {off + n_bytes}) runs past the end of the file")
            self.tensors.append(TensorInfo(name, shape, tid, tname, n_el, n_bytes, off))
        self.data_offset = data_start

    # ------------------------------------------------------------------ access
    def names(self) -> List[str]:
        return [t.name for t in self.tensors]

    def info(self, name: str) -> TensorInfo:
        try:
            return self._by_name[name]
        except KeyError:
            raise KeyError(f"tensor not found: {name}")

    def tensor_bytes(self, name: str) -> np.ndarray:
        """The tensor's bytes as a read-only uint8 view of the mapping."""
        t = self.info(name)
        return np.frombuffer(self._buf, dtype=np.uint8, count=t.n_bytes, offset=t.offset)

    def tensor_f32(self, name: str) -> np.ndarray:
        """A dense tensor (F32 / F16 / BF16) as float32 in ggml order reversed to row-major [rows..., cols]."""
        t = self.info(name)
        raw = self.tensor_bytes(name)
        if t.type_name == "F32":
            a = raw.view("<f4").astype(np.float32)
        elif t.type_name == "F16":
            a = raw.view("<f2").astype(np.float32)
        elif t.type_name == "BF16":
            a = (raw.view("<u2").astype(np.uint32) << 16).view(np.float32)
        else:
            raise GGUFError(f"tensor {name} is {t.type_name}, not a dense float tensor")
        return a.reshape(tuple(reversed(t.shape)))

    def upload(self, name: str):
        """`DeviceWeight` for a packed 2-D tensor, uploaded straight from the mapping (canonical row-major blocks)."""
        from . import kernels
        t = self.info(name)
        if t.type_name not in DEVICE_ENCODINGS:
            raise GGUFError(f"tensor {name} is {t.type_name}; the device kernels take {DEVICE_ENCODINGS}")
        if len(t.shape) != 2:
            raise GGUFError(f"tensor {name} has shape {t.shape}; a matmul weight is 2-D")
        return kernels.DeviceWeight.upload(t.type_name, self.tensor_bytes(name), t.rows, t.cols)

    def close(self) -> None:
        self._by_name = {}
        buf, self._buf = getattr(self, "_buf", None), None
        if buf is not None:
            try:
                buf.release()
            except BufferError:
                pass                                   # a caller still holds an array view of the mapping
        m, self._map = getattr(self, "_map", None), None
        if m is not None:
            try:
                m.close()
            except BufferError:
                pass                                   # a caller still holds a view; the mapping goes with it
        f, self._file = getattr(self, "_file", None), None
        if f is not None:
            f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
        return False


class GGUFWriter:
    """Writes a version-3 GGUF file: metadata, tensor infos, aligned tensor data."""

    def __init__(self, alignment: int = DEFAULT_ALIGNMENT):
        self.alignment = alignment
        self._kv: List[bytes] = []
        self._tensors: List[tuple] = []
        if alignment != DEFAULT_ALIGNMENT:
            self.add_u32("general.alignment", alignment)

    @staticmethod
    def _str(s: str) -> bytes:
        b = s.encode("utf-8")
        return struct.pack("<Q", len(b)) + b

    def add_u32(self, key: str, v: int) -> None:
        self._kv.append(self._str(key) + struct.pack("<II", 4, v))

    def add_f32(self, key: str, v: float) -> None:
        self._kv.append(self._str(key) + struct.pack("<If", 6, v))

    def add_string(self, key: str, v: str) -> None:
        self._kv.append(self._str(key) + struct.pack("<I", _STRING) + self._str(v))

    def add_array_i32(self, key: str, values) -> None:
        a = np.asarray(values, dtype="<i4")
        self._kv.append(self._str(key) + struct.pack("<IIQ", _ARRAY, 5, a.size) + a.tobytes())

    def add_array_string(self, key: str, values) -> None:
        body = b"".join(self._str(v) for v in values)
        self._kv.append(self._str(key) + struct.pack("<IIQ", _ARRAY, _STRING, len(values)) + body)

    def add_tensor(self, name: str, type_name: str, shape_rows_cols, data: np.ndarray) -> None:
        """`shape_rows_cols` is row-major (rows..., cols); it is stored in ggml order (cols first)."""
        tid = TYPE_ID[type_name]
        _, bs, nb = GGML_TYPES[tid]
        data = np.ascontiguousarray(data)
        n_el = int(np.prod(shape_rows_cols))
        if data.nbytes != n_el // bs * nb:
            raise GGUFError(f"tensor {name}: {data.nbytes} bytes given, shape {shape_rows_cols} as {type_name} needs {n_el // bs * nb}")
        self._tensors.append((name, tuple(reversed(tuple(shape_rows_cols))), tid, data.view(np.uint8).reshape(-1)))

    def write(self, path: str) -> None:
        head = struct.pack("<IIQQ", GGUF_MAGIC, 3, len(self._tensors), len(self._kv)) + b"".join(self._kv)
        infos, rel = [], 0
        for name, shape, tid, data in self._tensors:
            infos.append(self._str(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape) +
                         struct.pack("<IQ", tid, rel))
            rel = (rel + data.size + self.alignment - 1) // self.alignment * self.alignment
        head += b"".join(infos)
        with open(path, "wb") as f:
            f.write(head)
            f.write(b"\0" * (-len(head) % self.alignment))
            for _, _, _, data in self._tensors:
                f.write(data.tobytes())
                f.write(b"\0" * (-data.size % self.alignment))
