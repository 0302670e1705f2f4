"""Grouped-query attention over the paged cache.

Order of work as in the reference's batched pass (crates/vipera-backend-cpu/src/model.rs:1005-1126):
``q, k, v = h W^T + b``; rotate q and k; write K (rotated) and V of every token of the step into the
cache; attend causally by count (a token at position p reads positions ``<= p`` of its own request,
or the last ``window`` of them); ``x += attn Wo^T``.  The three projections run as one product over
the concatenated weight ``[Wq; Wk; Wv]``, whose rows equal the separate products' rows.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ..config.base import PartSpec
from ..errors import InvalidArgumentError, UnsupportedError
from ..ops import kernels
from ..ops.attention import paged_attention
from ..ops.linear import linear, linear_follow, split_qkv_plan, streams_in_wave_order
from ..weights.checkpoint import MATRIX, VECTOR, TensorSpec
from .base import KVCacheSpec, Mixer, register_mixer


def _cat(tensors: List[torch.Tensor]) -> torch.Tensor:
    dtypes = {t.dtype for t in tensors}
    if len(dtypes) > 1:  # a matrix kept in 32-bit pulls its companions up with it
        tensors = [t.float() for t in tensors]
    return torch.cat(tensors, dim=0).contiguous()


class Attention(Mixer):
    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        p = spec.params
        self.hidden = int(p["hidden"])
        self.heads = int(p["heads"])
        self.kv_heads = int(p["kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.window = int(p.get("window") or 0)
        self.qkv_bias = bool(p.get("qkv_bias", False))
        self.out_bias = bool(p.get("out_bias", False))
        scale = p.get("scale")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        if self.heads % self.kv_heads:
            raise InvalidArgumentError(f"heads {self.heads} is not a multiple of kv_heads {self.kv_heads}")
        self.q_width = self.heads * self.head_dim
        self.kv_width = self.kv_heads * self.head_dim
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        p = spec.params
        base = f"{prefix}{p['name']}."
        hidden, hd = int(p["hidden"]), int(p["head_dim"])
        q, kv = int(p["heads"]) * hd, int(p["kv_heads"]) * hd
        specs: List[TensorSpec] = []
        for name, rows in (("q", q), ("k", kv), ("v", kv)):
            specs.append(TensorSpec(f"{base}{name}_proj.weight", (rows, hidden), MATRIX))
            if p.get("qkv_bias"):
                specs.append(TensorSpec(f"{base}{name}_proj.bias", (rows,), VECTOR))
        specs.append(TensorSpec(base + "o_proj.weight", (hidden, q), MATRIX))
        if p.get("out_bias"):
            specs.append(TensorSpec(base + "o_proj.bias", (hidden,), VECTOR))
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        base = f"{self.prefix}{self.spec.params['name']}."
        self.w_qkv = _cat([tensors[base + f"{n}_proj.weight"] for n in "qkv"])
        if self.qkv_bias:
            self.b_qkv = torch.cat([tensors[base + f"{n}_proj.bias"] for n in "qkv"]).contiguous()
        self.w_o = tensors[base + "o_proj.weight"]
        if self.out_bias:
            self.b_o = tensors[base + "o_proj.bias"]

    @classmethod
    def declare_cache(cls, spec: PartSpec):
        p = spec.params
        return KVCacheSpec(int(p["kv_heads"]), int(p["head_dim"]), int(p.get("window") or 0)), None

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype: torch.dtype) -> None:
        p = spec.params
        heads, kv_heads, head_dim = int(p["heads"]), int(p["kv_heads"]), int(p["head_dim"])
        if head_dim > kernels.ATTENTION_MAX_HEAD_DIM:
            raise UnsupportedError(f"attention: head_dim {head_dim} is above the kernels' limit of "
                                   f"{kernels.ATTENTION_MAX_HEAD_DIM}")
        if heads + 2 * kv_heads > kernels.ATTENTION_MAX_HEADS:
            raise UnsupportedError(f"attention: {heads} query heads with {kv_heads} key/value heads are above the "
                                   f"kernels' limit of {kernels.ATTENTION_MAX_HEADS} heads in all")

    fills_handoff = True

    def _fused(self, tokens: int, position, batch) -> Optional[str]:
        """How product, rotation and cache write of a step of ``tokens`` run as one launch sequence without a
        rotation kernel, if they do: "stream" (up to 16 tokens, one kernel) or "split" (up to 64 tokens, K split
        over workgroups and the kernel that adds the ranges rotates).  All bfloat16, a full rotation computed in the
        kernel (no table of the step's angles)."""
        fused = position.fused_rotary()
        n, k = self.w_qkv.shape
        if not (fused is not None and fused[1] == self.head_dim and self.runtime.dtype == torch.bfloat16
                and self.w_qkv.dtype == torch.bfloat16 and self.head_dim % 2 == 0 and k % 8 == 0
                and position.step_angles(batch) is None):
            return None
        if tokens <= 16 and streams_in_wave_order(tokens, n, k, rotates=True) and n * k * 2 < 2 ** 31:
            return "stream"
        if self.head_dim % 8 == 0 and split_qkv_plan(tokens, n, k) is not None:
            return "split"
        return None

    def accepts_handoff(self, tokens: int, position, batch) -> bool:
        # the fused products can divide by the norm themselves
        return self._fused(tokens, position, batch) is not None

    def forward(self, h, batch, cache, state, position, residual, reads_only: bool = False, handoff=None,
                incoming=None) -> None:
        tokens = residual.shape[0]
        how = self._fused(tokens, position, batch)
        if incoming is not None and how is None:
            raise UnsupportedError("attention was handed a split norm for a step whose product cannot divide by it")
        scaled = {} if incoming is None else {"sumsq": incoming.sumsq, "groups": incoming.groups, "eps": incoming.eps}
        if incoming is not None:
            h = incoming.scaled
        qkv = self.runtime.empty((tokens, self.q_width + 2 * self.kv_width))
        table = batch.block_tables[cache.group]
        fused = position.fused_rotary()
        inv_freq, rotary_dim = fused if fused is not None else (None, 0)
        angles = position.step_angles(batch) if rotary_dim else None
        caches = (None, None, batch.entry_of_token, None) if reads_only else (cache.k, cache.v, batch.entry_of_token, table)
        if how == "stream" and kernels.gemm_bf16_qkv_rope_supported(h, self.w_qkv, qkv, self.head_dim):
            kernels.gemm_bf16_qkv_rope(h, self.w_qkv, self.b_qkv, qkv, batch.positions, inv_freq, *caches, self.heads,
                                       self.kv_heads, self.head_dim, **scaled)
        elif how == "split" and kernels.gemm_bf16_supported(h, self.w_qkv, qkv):
            ranges, rows_per_wave = split_qkv_plan(tokens, *self.w_qkv.shape)
            kernels.gemm_bf16_mid_qkv_rope(h, self.w_qkv, self.b_qkv, qkv, ranges, rows_per_wave, batch.positions, inv_freq,
                                           *caches, self.heads, self.kv_heads, self.head_dim, **scaled)
        else:
            if incoming is not None:
                raise UnsupportedError("attention was handed a split norm for operands its fused product does not take")
            linear(h, self.w_qkv, self.b_qkv, qkv)
            if fused is None:
                position.apply(qkv, batch, self.heads, self.kv_heads, self.head_dim)
            if not reads_only:
                kernels.rope_kvwrite(qkv, batch.positions, inv_freq, rotary_dim, cache.k, cache.v, batch.entry_of_token,
                                     table, self.heads, self.kv_heads, self.head_dim, angles)
            elif rotary_dim:
                kernels.rope_kvwrite(qkv, batch.positions, inv_freq, rotary_dim, None, None, batch.entry_of_token,
                                     None, self.heads, self.kv_heads, self.head_dim, angles)
        attn = self.runtime.empty((tokens, self.q_width))
        paged_attention(qkv, cache.k, cache.v, attn, batch, table, self.heads, self.kv_heads, self.head_dim,
                        self.scale, self.window)
        if handoff is not None:
            # the output product also prepares the norm that follows (its gained copy of the residual, its squares)
            # where its kernel can; 0 groups say that it could not
            handoff.groups = linear_follow(attn, self.w_o, self.b_o, residual, handoff.gain, handoff.scaled, handoff.sumsq)
        else:
            linear(attn, self.w_o, self.b_o, residual, accumulate=True)


register_mixer("attention", Attention)
