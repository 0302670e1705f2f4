"""What every part needs to run: the device, the run's dtype, and scratch allocation."""
from __future__ import annotations

from typing import Sequence

import torch

from .errors import InternalError, UnsupportedError

_DTYPE_NAMES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise UnsupportedError(f"dtype {name} is not implemented; use bfloat16 or float32")
        return name
    if name not in _DTYPE_NAMES:
        raise UnsupportedError(f"dtype \"{name}\" is not implemented; use bfloat16 or float32")
    return _DTYPE_NAMES[name]


class Runtime:
    """Device and dtype of a run.

    ``dtype`` is the storage type of activations between kernels, of matrices and of the cache:
    ``bfloat16`` (what serving uses) or ``float32`` (every product and sum in true 32-bit).  The
    residual stream, norms' sums, softmax and rotation angles are 32-bit in both.
    """

    def __init__(self, device="cuda:0", dtype="bfloat16"):
        self.dtype = parse_dtype(dtype)
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise UnsupportedError("the engine runs on a GPU only; there is no CPU path")
        if not torch.cuda.is_available():
            raise InternalError("no GPU is visible to this process (torch.cuda.is_available() is false)")
        torch.cuda.set_device(self.device)

    def empty(self, shape: Sequence[int], dtype: torch.dtype = None) -> torch.Tensor:
        return torch.empty(tuple(shape), dtype=dtype or self.dtype, device=self.device)

    def zeros(self, shape: Sequence[int], dtype: torch.dtype = None) -> torch.Tensor:
        return torch.zeros(tuple(shape), dtype=dtype or self.dtype, device=self.device)
