"""Reading and writing safetensors files without any library.

Format: 8 bytes little-endian header length N, N bytes of JSON mapping each
tensor name to {"dtype", "shape", "data_offsets": [begin, end]} (offsets
relative to the end of the header), then the data.  The checks are those of
the reference's reader (/root/reference/core/include/sonicboom/safetensors/reader.h:19-204):
a sane header length, well-formed JSON, offsets inside the file, a byte count
that matches shape and dtype; errors say which of file / format / truncation
went wrong and where.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, Tuple

import numpy as np

# dtype name -> (bytes per element, numpy dtype used to carry the raw bits)
DTYPES = {
    "F64": (8, np.float64), "F32": (4, np.float32), "F16": (2, np.float16), "BF16": (2, np.uint16),
    "I64": (8, np.int64), "I32": (4, np.int32), "I16": (2, np.int16), "I8": (1, np.int8),
    "U8": (1, np.uint8), "BOOL": (1, np.uint8),
}
MAX_HEADER = 100 * 1024 * 1024


class SafetensorsError(ValueError):
    """category is "io", "format" or "truncated"."""

    def __init__(self, category: str, message: str):
        super().__init__(f"{category}: {message}")
        self.category = category


@dataclass(frozen=True)
class TensorInfo:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    begin: int      # absolute file offsets
    end: int


class SafetensorsFile:
    """A memory-mapped safetensors file; ``tensors`` maps names to :class:`TensorInfo`."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._f = open(path, "rb")
        except OSError as e:
            raise SafetensorsError("io", f"{path}: {e.strerror or e}") from None
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise SafetensorsError("truncated", f"{path}: {size} bytes, no room for the header length")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n > MAX_HEADER or 8 + n > size:
            raise SafetensorsError("truncated" if n <= MAX_HEADER else "format",
                                   f"{path}: header length {n} does not fit the file of {size} bytes")
        raw = self._f.read(n)
        try:
            header = json.loads(raw.decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError("format", f"{path}: header is not valid JSON ({e})") from None
        if not isinstance(header, dict):
            raise SafetensorsError("format", f"{path}: header must be a JSON object")
        base = 8 + n
        self.metadata = header.pop("__metadata__", {}) or {}
        self.tensors: Dict[str, TensorInfo] = {}
        spans = []
        for name, e in header.items():
            try:
                dtype, shape, (b, en) = e["dtype"], tuple(int(s) for s in e["shape"]), e["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError("format", f"{path}: malformed entry for tensor {name}") from None
            if dtype not in DTYPES:
                raise SafetensorsError("format", f"{path}: tensor {name} has unknown dtype {dtype}")
            count = 1
            for s in shape:
                count *= s
            if en - b != count * DTYPES[dtype][0] or b < 0:
                raise SafetensorsError(
                    "format", f"{path}: tensor {name} spans {en - b} bytes, shape {list(shape)} {dtype} needs "
                              f"{count * DTYPES[dtype][0]}")
            if base + en > size:
                raise SafetensorsError(
                    "truncated", f"{path}: tensor {name} ends at byte {base + en}, the file has {size}")
            spans.append((b, en, name))
            self.tensors[name] = TensorInfo(name, dtype, shape, base + b, base + en)
        spans.sort()
        for (b0, e0, n0), (b1, e1, n1) in zip(spans, spans[1:]):
            if b1 < e0:
                raise SafetensorsError("format", f"{path}: tensors {n0} and {n1} overlap")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def raw(self, name: str) -> np.ndarray:
        """A private copy of the tensor's bits in the carrier dtype (BF16 as uint16)."""
        info = self.tensors[name]
        arr = np.frombuffer(self._mm, dtype=DTYPES[info.dtype][1], count=(info.end - info.begin) // DTYPES[info.dtype][0],
                            offset=info.begin)
        return np.array(arr, copy=True).reshape(info.shape)

    def close(self) -> None:
        if self._mm is not None:
            self._mm.close()
            self._mm = None
        self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """Round float32 to bfloat16 bits, to nearest even, NaN kept quiet
    (/root/reference/core/include/sonicboom/dtype.h:42-46)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = ((u + (0x7FFF + ((u >> 16) & 1))) >> 16).astype(np.uint16)
    return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), rounded)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def write_safetensors(path: str, tensors: Iterable[Tuple[str, str, np.ndarray]], metadata=None) -> None:
    """Write (name, dtype name, array of raw bits in the carrier dtype) triples."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for name, dtype, arr in tensors:
        size, carrier = DTYPES[dtype]
        arr = np.ascontiguousarray(arr, dtype=carrier)
        nbytes = arr.size * size
        header[name] = {"dtype": dtype, "shape": list(arr.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        blobs.append(arr)
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * ((8 - len(raw) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(raw)))
        f.write(raw)
        for arr in blobs:
            f.write(arr.tobytes())
    os.replace(tmp, path)
