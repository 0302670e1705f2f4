"""Attention dispatch: which kernel attends over the paged cache for a step's tokens."""
from __future__ import annotations

import torch

from . import kernels

_bf16_attention = None


def set_bf16_attention(fn) -> None:
    """Install the matrix-core implementation; ``fn(...) -> bool`` (False: not taken, fall through)."""
    global _bf16_attention
    _bf16_attention = fn


def paged_attention(qkv, k_cache, v_cache, out, batch, table, heads, kv_heads, head_dim, scale, window) -> None:
    if _bf16_attention is not None and qkv.dtype == torch.bfloat16:
        if _bf16_attention(qkv, k_cache, v_cache, out, batch, table, heads, kv_heads, head_dim, scale, window):
            return
    kernels.attn_generic(qkv, k_cache, v_cache, out, batch.positions, batch.entry_of_token, table, heads, kv_heads,
                         head_dim, scale, window)
