"""Matrix product dispatch: which kernel runs ``out (+)= a @ w.T + bias``.

All-bfloat16 operands whose rows are 16-byte aligned go to the matrix-core kernels; every other
combination (the 32-bit run, or a matrix kept in 32-bit inside a bfloat16 run) goes to the
32-bit FMA kernel.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import kernels

def linear(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
           accumulate: bool = False) -> torch.Tensor:
    if a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and kernels.gemm_bf16_supported(a, w, out):
        kernels.gemm_bf16(a, w, bias, out, accumulate)
    else:
        kernels.gemm_generic(a, w, bias, out, accumulate)
    return out
