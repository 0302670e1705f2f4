"""Reading and writing the safetensors container, with the checks a loader owes its caller.

Layout of a file: an 8-byte little-endian header length, a JSON header that maps each
tensor name to ``{"dtype", "shape", "data_offsets": [begin, end]}`` (offsets relative to
the end of the header), then the raw little-endian tensor bytes.

The checks follow the habits of the reference's model-file parser
(crates/vipera-core/src/gguf/mod.rs:143-293): sizes are bounded before anything is
trusted, a tensor must lie inside the file, tensors must not overlap, names are unique,
and every error names the file and the entry it is about.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
import warnings
from dataclasses import dataclass
from typing import Dict, Iterable, List, Tuple

import torch

from ..errors import IoError, ParseError, UnsupportedError

_DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "F64": (torch.float64, 8),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {dtype: name for name, (dtype, _) in _DTYPES.items()}
_MAX_HEADER = 100 * 1024 * 1024


@dataclass(frozen=True)
class TensorInfo:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    begin: int  # absolute byte offset in the file
    end: int
    path: str

    @property
    def torch_dtype(self) -> torch.dtype:
        return _DTYPES[self.dtype][0]

    @property
    def is_32bit_float(self) -> bool:
        return self.dtype == "F32"


class SafetensorsFile:
    """One ``.safetensors`` file: its parsed header and lazy access to the tensor bytes."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._handle = open(path, "rb")
            size = os.fstat(self._handle.fileno()).st_size
        except OSError as err:
            raise IoError(f"cannot read {path}: {err.strerror or err}") from None
        if size < 8:
            raise ParseError(f"{path}: {size} bytes is too short for a safetensors header")
        (header_len,) = struct.unpack("<Q", self._handle.read(8))
        if header_len > _MAX_HEADER or 8 + header_len > size:
            raise ParseError(
                f"{path}: header length {header_len} does not fit the file of {size} bytes"
            )
        raw = self._handle.read(header_len)
        try:
            header = json.loads(raw.decode("utf-8"), object_pairs_hook=_no_duplicates(path))
        except (UnicodeDecodeError, json.JSONDecodeError) as err:
            raise ParseError(f"{path}: header is not valid JSON: {err}") from None
        if not isinstance(header, dict):
            raise ParseError(f"{path}: header must be a JSON object")
        data_start = 8 + header_len
        self.metadata = header.pop("__metadata__", {}) or {}
        self.tensors: Dict[str, TensorInfo] = {}
        spans: List[Tuple[int, int, str]] = []
        for name, entry in header.items():
            info = _parse_entry(path, name, entry, data_start, size)
            self.tensors[name] = info
            if info.end > info.begin:
                spans.append((info.begin, info.end, name))
        spans.sort()
        for (_, end_a, name_a), (begin_b, _, name_b) in zip(spans, spans[1:]):
            if begin_b < end_a:
                raise ParseError(f"{path}: tensors \"{name_a}\" and \"{name_b}\" overlap")
        self._map = mmap.mmap(self._handle.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def read(self, name: str) -> torch.Tensor:
        """The tensor as a CPU tensor that views the mapped file (copy before the file is closed)."""
        info = self.tensors[name]
        count = 1
        for dim in info.shape:
            count *= dim
        if count == 0:
            return torch.empty(info.shape, dtype=info.torch_dtype)
        with warnings.catch_warnings():  # the map is read-only on purpose; nothing writes through the view
            warnings.simplefilter("ignore", UserWarning)
            flat = torch.frombuffer(self._map, dtype=info.torch_dtype, count=count, offset=info.begin)
        return flat.reshape(info.shape)

    def close(self) -> None:
        # The map may still be referenced by tensors that view it; it is released with them.
        self._handle.close()


def _no_duplicates(path: str):
    def hook(pairs):
        seen = {}
        for key, value in pairs:
            if key in seen:
                raise ParseError(f"{path}: name \"{key}\" appears twice in the header")
            seen[key] = value
        return seen

    return hook


def _parse_entry(path: str, name: str, entry, data_start: int, size: int) -> TensorInfo:
    if not isinstance(entry, dict):
        raise ParseError(f"{path}: entry of tensor \"{name}\" is not an object")
    dtype = entry.get("dtype")
    shape = entry.get("shape")
    offsets = entry.get("data_offsets")
    if dtype not in _DTYPES:
        raise UnsupportedError(f"{path}: tensor \"{name}\" has dtype {dtype!r}, which is not implemented")
    if not isinstance(shape, list) or any(isinstance(d, bool) or not isinstance(d, int) or d < 0 for d in shape):
        raise ParseError(f"{path}: tensor \"{name}\" has shape {shape!r}, expected a list of sizes")
    if (
        not isinstance(offsets, list)
        or len(offsets) != 2
        or any(isinstance(o, bool) or not isinstance(o, int) or o < 0 for o in offsets)
        or offsets[0] > offsets[1]
    ):
        raise ParseError(f"{path}: tensor \"{name}\" has data_offsets {offsets!r}, expected [begin, end]")
    count = 1
    for dim in shape:
        count *= dim
    want = count * _DTYPES[dtype][1]
    if offsets[1] - offsets[0] != want:
        raise ParseError(
            f"{path}: tensor \"{name}\" of shape {shape} and dtype {dtype} needs {want} bytes "
            f"but its data_offsets span {offsets[1] - offsets[0]}"
        )
    begin, end = data_start + offsets[0], data_start + offsets[1]
    if end > size:
        raise ParseError(f"{path}: tensor \"{name}\" ends at byte {end}, past the file's {size}")
    return TensorInfo(name, dtype, tuple(shape), begin, end, path)


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata=None) -> None:
    """Write ``(name, tensor)`` pairs in the given order; tensors are CPU and contiguous."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    kept: List[torch.Tensor] = []
    for name, tensor in tensors:
        if name in header:
            raise ParseError(f"{path}: tensor \"{name}\" given twice")
        if tensor.dtype not in _NAMES:
            raise UnsupportedError(f"tensor \"{name}\" has dtype {tensor.dtype}, which cannot be written")
        tensor = tensor.detach().cpu().contiguous()
        nbytes = tensor.numel() * tensor.element_size()
        header[name] = {
            "dtype": _NAMES[tensor.dtype],
            "shape": list(tensor.shape),
            "data_offsets": [offset, offset + nbytes],
        }
        offset += nbytes
        kept.append(tensor)
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * (-(8 + len(raw)) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as handle:
        handle.write(struct.pack("<Q", len(raw)))
        handle.write(raw)
        for tensor in kept:
            if tensor.numel():
                handle.write(tensor.reshape(-1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
