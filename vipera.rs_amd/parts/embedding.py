"""Token embedding and the output projection.

Reference: the embedding is a row read with no scaling (crates/vipera-backend-cpu/src/model.rs:607-616);
the head is ``logits = Wout h`` on the normed rows that are wanted, and when the model has no output
matrix the embedding table serves as one (model.rs:425, 1201-1237).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..config.base import PartSpec
from ..ops import kernels
from ..ops.linear import linear
from ..weights.checkpoint import MATRIX, TensorSpec
from .base import Part, register_embedding, register_head


class Embedding(Part):
    reads_device_tokens = True  # forward() takes (source, sampled): ids may be read from the device

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        self.vocab = int(spec.params["vocab"])
        self.width = int(spec.params["width"])
        self.table: Optional[torch.Tensor] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        return [TensorSpec(f"{prefix}{spec.params['name']}.weight",
                           (int(spec.params["vocab"]), int(spec.params["width"])), MATRIX)]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors[f"{self.prefix}{self.spec.params['name']}.weight"]

    def embed(self, batch) -> torch.Tensor:
        """The 32-bit residual ``[tokens, width]`` a step starts from.  An embedding sees the whole batch, so one
        that adds something by position (``batch.positions``) needs nothing else."""
        if batch.sampled_tokens is not None and batch.token_source is not None:  # ids the sampler left on the device
            return self.forward(batch.tokens, batch.num_tokens, batch.token_source, batch.sampled_tokens)
        return self.forward(batch.tokens, batch.num_tokens)

    def forward(self, tokens: torch.Tensor, count: int, source: Optional[torch.Tensor] = None,
                sampled: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Rows of the table for ``tokens``; where ``source`` is not negative the id is read from
        ``sampled`` on the device instead (see ``kernels.embed_gather``)."""
        out = self.runtime.empty((count, self.width), torch.float32)
        kernels.embed_gather(self.table, tokens, out, source, sampled)
        return out


class LMHead(Part):
    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        self.vocab = int(spec.params["vocab"])
        self.width = int(spec.params["width"])
        self.tied_to = spec.params.get("tied_to")
        self.weight: Optional[torch.Tensor] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        # With tied embeddings the output matrix is optional: a folder that holds one has it used, as the reference
        # uses `output.weight` whenever the file has it and the embedding table only otherwise (model.rs:424-425).
        return [TensorSpec(f"{prefix}{spec.params['name']}.weight",
                           (int(spec.params["vocab"]), int(spec.params["width"])), MATRIX,
                           optional=bool(spec.params.get("tied_to")))]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        own = f"{self.prefix}{self.spec.params['name']}.weight"
        if self.tied_to and own not in tensors:
            self.weight = tensors[f"{self.tied_to}.weight"]  # tied: the same buffer, no copy
        else:
            self.weight = tensors[own]

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        logits = self.runtime.empty((h.shape[0], self.vocab), torch.float32)
        linear(h, self.weight, None, logits)
        return logits


register_embedding("embedding", Embedding)
register_head("lm_head", LMHead)
