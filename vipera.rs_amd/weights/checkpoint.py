"""A model folder's tensors by name, and the one check of them against what a model declares.

The reference finds a tensor by name and fails on the first problem with a text that
names the tensor, what was found and what was expected
(crates/vipera-backend-cpu/src/model.rs:4383-4458).  Here every problem of a folder is
collected into one error: tensors that are missing, tensors nobody asked for, and
tensors of the wrong shape.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from ..errors import InvalidArgumentError, IoError, ParseError
from .safetensors_io import SafetensorsFile, TensorInfo

MATRIX = "matrix"   # converted to the run's dtype when it is loaded (see kept_dtype)
VECTOR = "vector"   # norm weights, biases: kept in 32-bit
INT_TABLE = "int_table"  # integer tables: kept as int32


@dataclass(frozen=True)
class TensorSpec:
    """A tensor that a part needs: its name, shape, how it is kept, and how random weights fill it."""

    name: str
    shape: Tuple[int, ...]
    role: str = MATRIX
    init: str = "normal"      # "normal" N(0, std) | "one_plus_normal" 1 + N(0, std) | "zeros" | "ones"
    std: float = 0.02
    optional: bool = False    # a folder need not hold it; when it does, its shape is checked and it is loaded


class WeightsError(InvalidArgumentError):
    """The folder's tensors do not match the model; lists every mismatch."""

    def __init__(self, where: str, missing: Sequence[str], unexpected: Sequence[str],
                 wrong: Sequence[Tuple[str, Tuple[int, ...], Tuple[int, ...]]]):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shapes = list(wrong)
        lines = [f"{where} does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shapes:
            shown = ", ".join(
                f"{name} is {list(found)}, expected {list(want)}" for name, found, want in self.wrong_shapes
            )
            lines.append(f"  wrong shapes ({len(self.wrong_shapes)}): {shown}")
        super().__init__("\n".join(lines))


class Checkpoint:
    """All tensors of a model folder: ``model.safetensors`` or the shards an index file names."""

    def __init__(self, folder: str):
        self.folder = folder
        self.files: List[SafetensorsFile] = []
        self.tensors: Dict[str, Tuple[SafetensorsFile, TensorInfo]] = {}
        index_path = os.path.join(folder, "model.safetensors.index.json")
        single = os.path.join(folder, "model.safetensors")
        if os.path.exists(single):
            paths = [single]
        elif os.path.exists(index_path):
            try:
                with open(index_path) as handle:
                    index = json.load(handle)
                shard_names = sorted(set(index["weight_map"].values()))
            except (OSError, ValueError, KeyError, AttributeError, TypeError) as err:
                raise ParseError(f"{index_path}: cannot read the shard index: {err}") from None
            paths = []
            root = os.path.realpath(folder)
            for name in shard_names:
                # a shard is a file of this folder: an index is not let to point anywhere else
                path = os.path.realpath(os.path.join(root, name)) if isinstance(name, str) else ""
                if not isinstance(name, str) or os.path.isabs(name) or os.path.dirname(path) != root:
                    raise ParseError(f"{index_path}: shard name {name!r} does not name a file of this folder")
                paths.append(path)
        else:
            raise IoError(f"{folder} holds neither model.safetensors nor model.safetensors.index.json")
        for path in paths:
            shard = SafetensorsFile(path)
            self.files.append(shard)
            for name, info in shard.tensors.items():
                if name in self.tensors:
                    other = self.tensors[name][1].path
                    raise ParseError(f"tensor \"{name}\" appears in both {other} and {path}")
                self.tensors[name] = (shard, info)

    def names(self) -> List[str]:
        return list(self.tensors)

    def info(self, name: str) -> TensorInfo:
        return self.tensors[name][1]

    def read(self, name: str) -> torch.Tensor:
        shard, _ = self.tensors[name]
        return shard.read(name)

    def check(self, specs: Iterable[TensorSpec]) -> None:
        """Raise one :class:`WeightsError` that lists everything wrong, or return."""
        wanted = {spec.name: spec for spec in specs}
        missing = [name for name, spec in wanted.items() if name not in self.tensors and not spec.optional]
        unexpected = [name for name in self.tensors if name not in wanted]
        wrong = []
        for name, spec in wanted.items():
            if name in self.tensors:
                found = self.tensors[name][1].shape
                if tuple(found) != tuple(spec.shape):
                    wrong.append((name, tuple(found), tuple(spec.shape)))
        if missing or unexpected or wrong:
            raise WeightsError(self.folder, missing, unexpected, wrong)

    def close(self) -> None:
        for shard in self.files:
            shard.close()


def kept_dtype(spec: TensorSpec, stored: torch.dtype, run_dtype: torch.dtype, keep_float32: bool = False) -> torch.dtype:
    """The dtype a tensor has on the device.

    A matrix is converted once, when it is loaded, to the run's dtype, whatever floating-point type the folder
    stores it in (32-bit, 16-bit float or bfloat16; to bfloat16 by rounding to nearest even): the run's kernels and
    the memory a plan predicts are then those of the run's dtype, not of the file's.  ``keep_float32``: a matrix
    stored in 32-bit stays in 32-bit in a bfloat16 run (its products then go through the 32-bit FMA kernel, at a
    fraction of the speed).  Vectors (norm weights, biases) are always 32-bit, which widens a 16-bit one exactly and
    leaves a 32-bit one as it is; integer tables become int32.
    """
    if spec.role == INT_TABLE:
        return torch.int32
    if spec.role == VECTOR:
        return torch.float32
    if run_dtype == torch.float32 or (keep_float32 and stored == torch.float32):
        return torch.float32
    return run_dtype


def kept_bytes(checkpoint: Checkpoint, specs: Sequence[TensorSpec], run_dtype: torch.dtype,
               keep_float32: bool = False) -> int:
    """Device bytes of the tensors that :func:`load_tensors` would load from ``checkpoint``, from its headers alone.
    A required tensor that the folder does not hold (yet) counts as if it were stored in the run's dtype."""
    total = 0
    for spec in specs:
        present = spec.name in checkpoint.tensors
        if not present and spec.optional:
            continue
        count = 1
        for dim in spec.shape:
            count *= int(dim)
        stored = checkpoint.info(spec.name).torch_dtype if present else run_dtype
        total += count * torch.empty(0, dtype=kept_dtype(spec, stored, run_dtype, keep_float32)).element_size()
    return total


def load_tensors(checkpoint: Checkpoint, specs: Sequence[TensorSpec], run_dtype: torch.dtype,
                 device: torch.device, progress=None, keep_float32: bool = False) -> Dict[str, torch.Tensor]:
    """Check the folder against ``specs`` and copy every tensor to the device in its kept dtype (an optional
    tensor that the folder does not hold is left out).  A tensor goes up as it is stored and is converted on the
    device."""
    checkpoint.check(specs)
    out: Dict[str, torch.Tensor] = {}
    for spec in specs:
        if spec.name not in checkpoint.tensors:
            continue
        stored = checkpoint.read(spec.name)
        dtype = kept_dtype(spec, stored.dtype, run_dtype, keep_float32)
        if not (stored.dtype.is_floating_point or spec.role == INT_TABLE):
            raise InvalidArgumentError(
                f"tensor \"{spec.name}\" is stored as {stored.dtype}, expected a floating-point dtype"
            )
        on_device = stored.to(device=device, copy=True)
        out[spec.name] = (on_device if on_device.dtype == dtype else on_device.to(dtype)).contiguous()
        if progress is not None:
            progress(spec.name)
    return out
