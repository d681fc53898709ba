"""Reader and writer for the safetensors container, with nothing that executes file content.

Layout of a file: an unsigned 64-bit little-endian header length ``N``, ``N`` bytes of JSON
``{name: {"dtype": "BF16", "shape": [...], "data_offsets": [begin, end]}, ...}`` (plus an optional
``"__metadata__"`` object), then the raw little-endian tensor bytes that the offsets index.
The reader memory-maps the file and returns numpy views, so a tensor is only paged in when it is
copied to the device. bfloat16 has no numpy type: such tensors come back as ``uint16`` bit patterns
with the logical dtype beside them.
"""

from __future__ import annotations

import json
import mmap
import struct
from dataclasses import dataclass
from pathlib import Path
from typing import Iterator, Mapping

import numpy as np

# safetensors dtype tag -> (numpy dtype that holds the bits, item size)
_NUMPY_OF_TAG: dict[str, np.dtype] = {
    "F64": np.dtype("<f8"),
    "F32": np.dtype("<f4"),
    "F16": np.dtype("<f2"),
    "BF16": np.dtype("<u2"),
    "I64": np.dtype("<i8"),
    "I32": np.dtype("<i4"),
    "I16": np.dtype("<i2"),
    "I8": np.dtype("i1"),
    "U8": np.dtype("u1"),
    "BOOL": np.dtype("?"),
}
_MAX_HEADER = 100 * 1024 * 1024


class SafetensorsFormatError(ValueError):
    """The file is not a well-formed safetensors container."""


@dataclass(frozen=True)
class TensorEntry:
    """One tensor of a file: its tag (``"BF16"``, ``"F32"``, ...), shape and raw bits."""

    name: str
    tag: str
    shape: tuple[int, ...]
    bits: np.ndarray  # view into the mapped file, dtype per _NUMPY_OF_TAG, already shaped

    @property
    def is_float(self) -> bool:
        return self.tag in ("F64", "F32", "F16", "BF16")

    @property
    def is_integer(self) -> bool:
        return self.tag in ("I64", "I32", "I16", "I8", "U8")


class SafetensorsFile:
    """A memory-mapped safetensors file. Use as a context manager or call :meth:`close`."""

    def __init__(self, path: str | Path) -> None:
        self.path = Path(path)
        self._fh = open(self.path, "rb")
        try:
            head = self._fh.read(8)
            if len(head) != 8:
                raise SafetensorsFormatError(f"{self.path}: shorter than the 8-byte length field")
            (n,) = struct.unpack("<Q", head)
            size = self.path.stat().st_size
            if n > _MAX_HEADER or 8 + n > size:
                raise SafetensorsFormatError(f"{self.path}: header length {n} exceeds the file")
            try:
                header = json.loads(self._fh.read(n).decode("utf-8"))
            except (UnicodeDecodeError, json.JSONDecodeError) as exc:
                raise SafetensorsFormatError(f"{self.path}: header is not JSON: {exc}") from exc
            if not isinstance(header, dict):
                raise SafetensorsFormatError(f"{self.path}: header is not a JSON object")
            self.metadata: dict[str, str] = dict(header.pop("__metadata__", None) or {})
            self._data_start = 8 + n
            self._data_len = size - self._data_start
            self._header = header
            self._validate()
            self._map = (
                mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None
            )
        except Exception:
            self._fh.close()
            raise

    def _validate(self) -> None:
        for name, info in self._header.items():
            if not isinstance(info, dict) or not {"dtype", "shape", "data_offsets"} <= set(info):
                raise SafetensorsFormatError(f"{self.path}: malformed entry for {name!r}")
            tag = info["dtype"]
            if tag not in _NUMPY_OF_TAG:
                raise SafetensorsFormatError(f"{self.path}: {name!r} has unknown dtype {tag!r}")
            begin, end = info["data_offsets"]
            count = 1
            for s in info["shape"]:
                count *= int(s)
            if not 0 <= begin <= end <= self._data_len:
                raise SafetensorsFormatError(f"{self.path}: {name!r} lies outside the data section")
            if end - begin != count * _NUMPY_OF_TAG[tag].itemsize:
                raise SafetensorsFormatError(
                    f"{self.path}: {name!r} has {end - begin} bytes but shape {info['shape']} of {tag}"
                )

    def names(self) -> list[str]:
        return list(self._header)

    def shape_of(self, name: str) -> tuple[int, ...]:
        return tuple(int(s) for s in self._header[name]["shape"])

    def tag_of(self, name: str) -> str:
        return str(self._header[name]["dtype"])

    def get(self, name: str) -> TensorEntry:
        info = self._header[name]
        tag = info["dtype"]
        shape = tuple(int(s) for s in info["shape"])
        begin, end = info["data_offsets"]
        dt = _NUMPY_OF_TAG[tag]
        count = (end - begin) // dt.itemsize
        if count == 0:
            bits = np.zeros(shape, dtype=dt)
        else:
            bits = np.frombuffer(
                self._map, dtype=dt, count=count, offset=self._data_start + begin
            ).reshape(shape)
        return TensorEntry(name, tag, shape, bits)

    def __iter__(self) -> Iterator[TensorEntry]:
        for name in self._header:
            yield self.get(name)

    def close(self) -> None:
        # numpy views keep the map alive; closing is best effort.
        try:
            if self._map is not None:
                self._map.close()
        except BufferError:
            pass
        self._fh.close()

    def __enter__(self) -> "SafetensorsFile":
        return self

    def __exit__(self, *exc: object) -> None:
        self.close()


def float32_to_bfloat16_bits(values: np.ndarray) -> np.ndarray:
    """Round float32 to bfloat16 (nearest, ties to even); returns the uint16 bit patterns."""
    u = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32)
    rounded = u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    out = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), rounded >> np.uint32(16))
    return out.astype(np.uint16)


def bfloat16_bits_to_float32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def write_safetensors(
    path: str | Path,
    tensors: Mapping[str, tuple[str, np.ndarray]],
    metadata: Mapping[str, str] | None = None,
) -> None:
    """Write ``{name: (tag, array)}``; a ``"BF16"`` array is given as uint16 bit patterns.

    Tensors are laid out in name order without gaps (the format allows none); the header is
    padded with spaces so that the data section starts on an 8-byte boundary.
    """
    header: dict[str, object] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    blobs: list[np.ndarray] = []  # written straight from the arrays' memory, no second copy
    offset = 0
    for name in sorted(tensors):
        tag, arr = tensors[name]
        if tag not in _NUMPY_OF_TAG:
            raise SafetensorsFormatError(f"unknown dtype tag {tag!r} for {name!r}")
        dt = _NUMPY_OF_TAG[tag]
        arr = np.ascontiguousarray(arr)
        if arr.dtype.itemsize != dt.itemsize:
            raise SafetensorsFormatError(f"{name!r}: array of {arr.dtype} cannot be stored as {tag}")
        raw = np.ascontiguousarray(arr.astype(dt, copy=False) if arr.dtype != dt else arr)
        header[name] = {"dtype": tag, "shape": list(arr.shape), "data_offsets": [offset, offset + raw.nbytes]}
        blobs.append(raw)
        offset += raw.nbytes
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    text += b" " * ((-len(text)) % 8)
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(text)))
        fh.write(text)
        for b in blobs:
            if b.nbytes:
                fh.write(memoryview(b.reshape(-1)).cast("B"))
