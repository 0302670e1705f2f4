"""Gated feed-forward (SwiGLU): ``x += (up(h) * silu(gate(h))) Wd^T``.

Reference: crates/vipera-backend-cpu/src/model.rs:672-680, 1159-1198; ``silu(z) = z / (1 + exp(-z))``
(model.rs:4368-4370).  Gate and up run as one product over a fused weight; with bfloat16 weights its
rows are interleaved in groups of 16 so that the product's epilogue can apply the gate.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..config.base import PartSpec
from ..errors import UnsupportedError
from ..ops import kernels
from ..ops.linear import gated_plan, interleave_gate_up, linear, linear_follow, linear_gated
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
        self.interleaved = False

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
        gate, up = tensors[base + "gate_proj.weight"], tensors[base + "up_proj.weight"]
        # all-bfloat16 weights of a width the kernels can pair are interleaved, so that the product's
        # epilogue can apply the gate; anything else stays [gate; up]
        self.interleaved = (gate.dtype == torch.bfloat16 and up.dtype == torch.bfloat16 and self.inter % 16 == 0)
        self.w_gate_up = interleave_gate_up(gate, up) if self.interleaved else _cat([gate, up])
        self.w_down = tensors[base + "down_proj.weight"]

    def _dividing_plan(self, tokens: int):
        """0 or 3 where the gate/up product of ``tokens`` rows runs on a kernel that can divide by the norm in front
        of it (the kernel with resident activations, the tiled kernel), else None."""
        if not (self.interleaved and self.w_gate_up.dtype == torch.bfloat16 and self.runtime.dtype == torch.bfloat16):
            return None
        if tokens > 64:  # no product before the norm leaves its first half for more than 64 tokens
            return None
        plan = gated_plan(tokens, *self.w_gate_up.shape, kernels.compute_units(self.w_gate_up.device))
        return plan if plan in (0, 3) and (plan == 3 or tokens <= 16) else None

    def accepts_handoff(self, tokens: int) -> bool:
        return self._dividing_plan(tokens) is not None

    fills_handoff = True

    def forward(self, h, batch, residual, handoff=None, outgoing=None) -> None:
        tokens = residual.shape[0]
        act = self.runtime.empty((tokens, self.inter))
        if handoff is not None and self._dividing_plan(tokens) == 0:
            kernels.gemm_bf16_gated_scaled(handoff.scaled, self.w_gate_up, act, handoff.sumsq, handoff.groups, handoff.eps)
        elif handoff is not None:
            kernels.gemm_bf16_gated_tile_scaled(handoff.scaled, self.w_gate_up, act, handoff.sumsq, handoff.groups,
                                                handoff.eps)
        else:
            linear_gated(h, self.w_gate_up, act, self.interleaved)
        if outgoing is not None:
            # the down product also prepares the next layer's first norm where its kernel can
            outgoing.groups = linear_follow(act, self.w_down, None, residual, outgoing.gain, outgoing.scaled, outgoing.sumsq)
        else:
            linear(act, self.w_down, None, residual, accumulate=True)


register_ffn("gated_mlp", GatedMLP)
