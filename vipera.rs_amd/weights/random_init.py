"""Seeded random weights: a model folder written from a configuration and a seed.

The reference has no such mode (its tests need a real model file and skip without one,
crates/vipera-backend-cpu/tests/batch.rs:117-125).  Every tensor draws from a stream of its
own, keyed by the seed and the tensor's name, so the values do not depend on the order
in which tensors are generated.  The stream is counter-based: element ``i`` of a tensor is a
function of (key, i) alone, which a device kernel can reproduce.

    z   = splitmix64_finalizer(key + (i + 1) * 0x9E3779B97F4A7C15)
    u1  = (high 32 bits of z + 0.5) / 2^32          in (0, 1)
    u2  = (low 32 bits of z) / 2^32                 in [0, 1)
    n   = sqrt(-2 ln u1) * cos(2 pi u2)             standard normal, computed in 64-bit
"""
from __future__ import annotations

import os
from typing import Dict, Iterable, Sequence

import numpy as np
import torch

from ..config.base import ModelConfig
from .checkpoint import INT_TABLE, MATRIX, TensorSpec
from .safetensors_io import write_safetensors

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_MASK = (1 << 64) - 1


def tensor_key(seed: int, name: str) -> int:
    """64-bit key of a tensor's stream: FNV-1a of the name, mixed with the seed."""
    h = 0xCBF29CE484222325
    for byte in name.encode("utf-8"):
        h = ((h ^ byte) * 0x100000001B3) & _MASK
    z = (h ^ ((seed * 0x9E3779B97F4A7C15) & _MASK)) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def standard_normal(key: int, count: int) -> np.ndarray:
    """``count`` standard normals of the stream ``key`` as float64."""
    with np.errstate(over="ignore"):
        index = np.arange(1, count + 1, dtype=np.uint64)
        z = np.uint64(key) + index * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    u1 = ((z >> np.uint64(32)).astype(np.float64) + 0.5) / 4294967296.0
    u2 = (z & np.uint64(0xFFFFFFFF)).astype(np.float64) / 4294967296.0
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)


def random_tensor(spec: TensorSpec, seed: int, dtype: torch.dtype) -> torch.Tensor:
    count = 1
    for dim in spec.shape:
        count *= dim
    if spec.role == INT_TABLE:
        return torch.zeros(spec.shape, dtype=torch.int32)
    if spec.init == "zeros":
        values = np.zeros(count, dtype=np.float32)
    elif spec.init == "ones":
        values = np.ones(count, dtype=np.float32)
    else:
        normal = standard_normal(tensor_key(seed, spec.name), count) * spec.std
        if spec.init == "one_plus_normal":
            normal = 1.0 + normal
        elif spec.init != "normal":
            raise ValueError(f"tensor \"{spec.name}\": unknown init {spec.init!r}")
        values = normal.astype(np.float32)
    return torch.from_numpy(values).reshape(spec.shape).to(dtype)


def random_tensors(specs: Iterable[TensorSpec], seed: int, dtype: torch.dtype):
    for spec in specs:
        if not spec.optional:
            yield spec.name, random_tensor(spec, seed, dtype)


def write_random_model(folder: str, config: ModelConfig, specs: Sequence[TensorSpec], seed: int,
                       dtype: torch.dtype = torch.float32) -> str:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` with seeded random weights."""
    os.makedirs(folder, exist_ok=True)
    config.save(folder)
    write_safetensors(
        os.path.join(folder, "model.safetensors"),
        random_tensors(specs, seed, dtype),
        metadata={"format": "pt", "seed": seed},
    )
    return folder


def random_device_tensors(specs: Sequence[TensorSpec], seed: int, run_dtype: torch.dtype, device):
    """Seeded random weights made on the device, for models too large to write to a folder first.

    The same counter-based streams as :func:`random_tensor`, evaluated by the ``fill_normal`` kernel;
    values agree with the host's up to the last bit of the device's ``log`` and ``cos``.
    """
    from ..ops import kernels
    from .checkpoint import kept_dtype

    out: Dict[str, torch.Tensor] = {}
    for spec in specs:
        if spec.optional:
            continue
        dtype = kept_dtype(spec, run_dtype, run_dtype)
        tensor = torch.empty(spec.shape, dtype=dtype, device=device)
        if spec.role == INT_TABLE or spec.init == "zeros":
            tensor.zero_()
        elif spec.init == "ones":
            tensor.fill_(1.0)
        else:
            kernels.fill_normal(tensor, tensor_key(seed, spec.name), spec.std,
                                1.0 if spec.init == "one_plus_normal" else 0.0)
        out[spec.name] = tensor
    return out
