"""Reading and writing safetensors files without a library.

The format: 8 bytes little-endian header length N, N bytes of JSON
`{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}`, then the raw
little-endian payload that the offsets index.  The reference never parses this format itself:
it converts checkpoints offline into a format of its own (scripts/convert_model.py:23-46) and
checks header, byte counts against shapes, duplicates, truncation and trailing bytes on load
(src/weight_store.cpp:168-260).  The same checks are made here, with the same error codes.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass

import torch

from ..errors import EngineError, ErrorCode

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {value: key for key, value in _DTYPES.items()}
_MAX_HEADER = 100 * 1024 * 1024


def _bad(message: str) -> EngineError:
    return EngineError(ErrorCode.INVALID_FORMAT, message)


@dataclass(frozen=True)
class StoredTensor:
    name: str
    dtype: torch.dtype
    shape: tuple[int, ...]
    begin: int      # offsets into the file, payload included
    end: int


class SafetensorsFile:
    """One file, memory-mapped; `tensor(name)` gives a CPU tensor that views the mapping."""

    def __init__(self, path: str):
        self.path = path
        try:
            handle = open(path, "rb")
        except OSError as error:
            raise EngineError(ErrorCode.IO, f"unable to open weights: {path} ({error.strerror})") from None
        with handle:                       # (the mapping made at the end keeps the file open by itself)
            self._read(handle, path)

    def _read(self, handle, path: str) -> None:
        size = os.fstat(handle.fileno()).st_size
        if size < 8:
            raise _bad(f"{path}: shorter than a safetensors header")
        (header_length,) = struct.unpack("<Q", handle.read(8))
        if header_length > _MAX_HEADER or 8 + header_length > size:
            raise _bad(f"{path}: header length {header_length} does not fit the file")
        try:
            header = json.loads(handle.read(header_length).decode("utf-8"),
                                object_pairs_hook=self._no_duplicates)
        except (ValueError, UnicodeDecodeError) as error:
            raise _bad(f"{path}: header is not valid JSON ({error})") from None
        if not isinstance(header, dict):
            raise _bad(f"{path}: header is not a JSON object")
        payload_begin = 8 + header_length
        self.metadata = header.pop("__metadata__", {}) or {}
        self.tensors: dict[str, StoredTensor] = {}
        spans = []
        for name, entry in header.items():
            try:
                dtype_name, shape, (begin, end) = entry["dtype"], entry["shape"], entry["data_offsets"]
                shape = tuple(int(extent) for extent in shape)
                begin, end = int(begin), int(end)
            except (KeyError, TypeError, ValueError):
                raise _bad(f"{path}: malformed entry for tensor '{name}'") from None
            if dtype_name not in _DTYPES:
                raise EngineError(ErrorCode.INVALID_DTYPE, f"{path}: tensor '{name}' has unsupported dtype {dtype_name}")
            dtype = _DTYPES[dtype_name]
            count = 1
            for extent in shape:
                if extent < 0:
                    raise _bad(f"{path}: tensor '{name}' has a negative extent")
                count *= extent
            item = torch.empty((), dtype=dtype).element_size()
            if begin < 0 or end < begin or end - begin != count * item:
                raise EngineError(ErrorCode.INVALID_SHAPE,
                                  f"{path}: tensor '{name}' holds {end - begin} bytes, its shape {list(shape)} needs {count * item}")
            if payload_begin + end > size:
                raise _bad(f"{path}: tensor '{name}' reaches past the end of the file (truncated?)")
            self.tensors[name] = StoredTensor(name, dtype, shape, payload_begin + begin, payload_begin + end)
            spans.append((begin, end, name))
        spans.sort()
        cursor = 0
        for begin, end, name in spans:
            if begin < cursor:
                raise _bad(f"{path}: tensor '{name}' overlaps another tensor")
            cursor = end
        if payload_begin + cursor != size and spans:
            raise _bad(f"{path}: {size - payload_begin - cursor} bytes after the last tensor")
        self._map = mmap.mmap(handle.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    @staticmethod
    def _no_duplicates(pairs):
        seen = {}
        for key, value in pairs:
            if key in seen:
                raise ValueError(f"tensor '{key}' is listed twice")
            seen[key] = value
        return seen

    def tensor(self, name: str) -> torch.Tensor:
        stored = self.tensors[name]
        count = 1
        for extent in stored.shape:
            count *= extent
        if count == 0:
            return torch.empty(stored.shape, dtype=stored.dtype)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")     # the mapping is read-only; nothing writes through the view
            flat = torch.frombuffer(self._map, dtype=stored.dtype, count=count, offset=stored.begin)
        return flat.view(stored.shape)


def write_safetensors(path: str, tensors: dict[str, torch.Tensor], metadata: dict[str, str] | None = None) -> None:
    """Writes the tensors in name order, each at an 8-byte-aligned offset of a padded header."""
    header: dict = {}
    if metadata:
        header["__metadata__"] = {str(key): str(value) for key, value in metadata.items()}
    cursor = 0
    ordered = sorted(tensors)
    for name in ordered:
        tensor = tensors[name]
        if tensor.dtype not in _NAMES:
            raise EngineError(ErrorCode.INVALID_DTYPE, f"cannot store dtype {tensor.dtype} of '{name}'")
        size = tensor.numel() * tensor.element_size()
        header[name] = {"dtype": _NAMES[tensor.dtype], "shape": list(tensor.shape), "data_offsets": [cursor, cursor + size]}
        cursor += size
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    text += b" " * ((-len(text)) % 8)
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(text)))
        handle.write(text)
        for name in ordered:
            tensor = tensors[name].detach().cpu().contiguous()
            handle.write(tensor.view(torch.uint8).numpy().tobytes() if tensor.numel() else b"")
