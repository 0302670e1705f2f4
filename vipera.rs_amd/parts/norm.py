"""RMSNorm: ``out = (x * rsqrt(mean(x^2) + eps)) * weight`` with the sum in 32-bit.

Reference: crates/vipera-backend-cpu/src/model.rs:4282-4288 (eps inside the square root, added to
the mean; multiply order ``(x * inv) * w``).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..config.base import PartSpec
from ..ops import kernels
from ..weights.checkpoint import VECTOR, TensorSpec
from .base import Norm, NormHandoff, register_norm


class RMSNorm(Norm):
    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        self.width = int(spec.params["width"])
        self.eps = float(spec.params["eps"])
        self.weight: Optional[torch.Tensor] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        return [TensorSpec(f"{prefix}{spec.params['name']}.weight", (int(spec.params["width"]),), VECTOR,
                           "one_plus_normal")]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[f"{self.prefix}{self.spec.params['name']}.weight"]

    def handoff(self, tokens: int) -> Optional[NormHandoff]:
        if self.runtime.dtype != torch.bfloat16 or self.weight is None or self.weight.dtype != torch.float32:
            return None
        return NormHandoff(self.weight, self.eps, self.runtime.empty((tokens, self.width)),
                           torch.empty(kernels.follow_sumsq_floats(self.width, tokens), dtype=torch.float32,
                                       device=self.weight.device))

    def forward(self, x, out=None, rows=None):
        count = x.shape[0] if rows is None else rows.numel()
        if out is None:
            out = self.runtime.empty((count, self.width))
        kernels.rmsnorm(x, self.weight, self.eps, out, rows)
        return out


register_norm("rmsnorm", RMSNorm)
