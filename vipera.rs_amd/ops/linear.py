"""Matrix product dispatch: which kernel runs ``out (+)= a @ w.T + bias``.

All-bfloat16 operands go to the matrix-core kernels once those are loaded; every other
combination (the 32-bit run, or a matrix kept in 32-bit inside a bfloat16 run) goes to the
32-bit FMA kernel.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import kernels

_bf16_gemm = None


def set_bf16_gemm(fn) -> None:
    """Install the matrix-core implementation ``fn(a, w, bias, out, accumulate) -> bool`` (False: not taken)."""
    global _bf16_gemm
    _bf16_gemm = fn


def linear(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
           accumulate: bool = False) -> torch.Tensor:
    if _bf16_gemm is not None and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        if _bf16_gemm(a, w, bias, out, accumulate):
            return out
    kernels.gemm_generic(a, w, bias, out, accumulate)
    return out
