"""Gated feed-forward (SwiGLU): ``x += (up(h) * silu(gate(h))) Wd^T``.

Reference: crates/vipera-backend-cpu/src/model.rs:672-680, 1159-1198; ``silu(z) = z / (1 + exp(-z))``
(model.rs:4368-4370).  Gate and up run as one product over ``[Wg; Wu]``.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..config.base import PartSpec
from ..errors import UnsupportedError
from ..ops import kernels
from ..ops.linear import linear
from ..weights.checkpoint import MATRIX, TensorSpec
from .attention import _cat
from .base import FeedForward, register_ffn


class GatedMLP(FeedForward):
    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        self.hidden = int(spec.params["hidden"])
        self.inter = int(spec.params["intermediate"])
        if spec.params.get("activation", "silu") != "silu":
            raise UnsupportedError(f"activation {spec.params.get('activation')!r} is not implemented; only \"silu\"")
        self.w_gate_up = self.w_down = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        base = f"{prefix}{spec.params['name']}."
        hidden, inter = int(spec.params["hidden"]), int(spec.params["intermediate"])
        return [
            TensorSpec(base + "gate_proj.weight", (inter, hidden), MATRIX),
            TensorSpec(base + "up_proj.weight", (inter, hidden), MATRIX),
            TensorSpec(base + "down_proj.weight", (hidden, inter), MATRIX),
        ]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        base = f"{self.prefix}{self.spec.params['name']}."
        self.w_gate_up = _cat([tensors[base + "gate_proj.weight"], tensors[base + "up_proj.weight"]])
        self.w_down = tensors[base + "down_proj.weight"]

    def forward(self, h, batch, residual) -> None:
        tokens = h.shape[0]
        gate_up = self.runtime.empty((tokens, 2 * self.inter))
        linear(h, self.w_gate_up, None, gate_up)
        act = self.runtime.empty((tokens, self.inter))
        kernels.swiglu(gate_up, act)
        linear(act, self.w_down, None, residual, accumulate=True)


register_ffn("gated_mlp", GatedMLP)
