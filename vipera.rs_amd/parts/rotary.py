"""Rotary position encoding, NeoX layout: pairs ``(i, i + rotary_dim / 2)`` of each head.

Reference: crates/vipera-backend-cpu/src/model.rs:4192-4251.  ``inv_i = 1 / base^(2i / head_dim)``
in 32-bit; the angle is ``float(pos) * inv_i`` in 32-bit; ``x[i] = lo*c - hi*s``,
``x[i + half] = lo*s + hi*c``.  The table of ``inv_i`` is computed once on the host with 32-bit
operations and kept on the device; the angle and its sine and cosine are computed in the kernel, or for
a step of many tokens once per step into a table that all layers with these frequencies read.
"""
from __future__ import annotations

from typing import List

import numpy as np
import torch

from ..config.base import PartSpec
from ..errors import InvalidArgumentError
from ..ops import kernels
from .base import PositionEncoding, register_position


ANGLE_TABLE_MIN_TOKENS = 128   # steps with at least this many tokens share one table of sines and cosines


def neox_inverse_frequencies(rotary_dim: int, base: float) -> np.ndarray:
    index = np.arange(rotary_dim // 2, dtype=np.float32)
    exponent = (np.float32(2.0) * index) / np.float32(rotary_dim)
    return (np.float32(1.0) / np.power(np.float32(base), exponent, dtype=np.float32)).astype(np.float32)


class RotaryNeox(PositionEncoding):
    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        self.head_dim = int(spec.params["head_dim"])
        self.rotary_dim = int(spec.params.get("rotary_dim", self.head_dim))
        self.base = float(spec.params["base"])
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.head_dim:
            raise InvalidArgumentError(
                f"rotary_dim {self.rotary_dim} must be even and at most head_dim {self.head_dim}")
        table = neox_inverse_frequencies(self.rotary_dim, self.base)
        self.inv_freq = torch.from_numpy(table).to(runtime.device)

    def fused_rotary(self):
        return self.inv_freq, self.rotary_dim

    def step_angles(self, batch):
        # a prompt's tokens times all heads times all layers would compute the same few sines again and
        # again; a few decoded tokens are cheaper without the extra launch
        if batch.num_tokens < ANGLE_TABLE_MIN_TOKENS or not self.rotary_dim:
            return None
        key = ("rope_angles", self.base, self.rotary_dim)
        table = batch.shared.get(key)
        if table is None:
            table = batch.shared[key] = kernels.rope_angles(batch.positions, self.inv_freq, batch.num_tokens)
        return table

    def apply(self, qkv, batch, heads, kv_heads, head_dim):
        kernels.rope_kvwrite(qkv, batch.positions, self.inv_freq, self.rotary_dim, None, None,
                             batch.entry_of_token, None, heads, kv_heads, head_dim)


class NoPosition(PositionEncoding):
    """No position encoding: queries and keys stay as projected."""

    def fused_rotary(self):
        return None, 0

    def apply(self, qkv, batch, heads, kv_heads, head_dim):
        return None


register_position("rotary_neox", RotaryNeox)
register_position("none", NoPosition)
