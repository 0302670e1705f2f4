"""The step function: run a batch of (request, its next tokens) through the model from the cache.

``ModelRunner`` owns the model, the cache manager and the cache's device memory.  ``step`` takes
entries whose pages are already reserved, runs only the tokens it is given as one batch, and
returns the logits at the wanted places.  It corresponds to the reference's ``ForwardPass`` seam
(crates/vipera-runtime/src/pipeline.rs:192-230), with ``logits``, ``logits_range`` and
``logits_batch`` folded into one call.
"""
from __future__ import annotations

import os
from typing import List, Optional, Sequence

import torch

from ..cache import CacheManager, CacheStorage, plan_groups
from ..config.base import ModelConfig
from ..config.registry import load_config
from ..errors import InvalidArgumentError
from ..models import build_model
from ..runtime import Runtime
from ..weights import Checkpoint, load_tensors
from .batch import StepBatch, StepEntry, build_batch


SAMPLED_CAPACITY = 1024  # rows of logits one step may be sampled for with device-side feedback


class ModelRunner:
    """``block_size`` and ``num_blocks``: positions per page and pages in the pool, one number for every cache group
    or a list with one per group (in the order of ``cache.group_keys(model.cache_needs())``)."""

    def __init__(self, model, runtime: Runtime, block_size, num_blocks, num_slots: int,
                 use_graphs: bool = False, max_context: int = 0):
        if not model.loaded:
            raise InvalidArgumentError("the model has no weights yet; load them before building a runner")
        self.model = model
        self.runtime = runtime
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.needs = model.cache_needs()
        groups = plan_groups(self.needs, block_size, num_blocks)
        self.cache = CacheManager(groups, num_slots)
        self.storage = CacheStorage(self.needs, groups, num_slots, runtime)
        self.vocab_size = model.vocab_size
        self.steps = 0
        # where a sampler may leave the ids it draws, for a next step that is launched before they reach the
        # host (StepEntry.source); at a fixed address, because captured steps read it
        self.sampled_tokens = None
        if getattr(model.embedding, "reads_device_tokens", False):
            self.sampled_tokens = torch.zeros(SAMPLED_CAPACITY, dtype=torch.int32, device=runtime.device)
        self.graphs = None
        if use_graphs:
            from .graphs import DecodeGraphs
            longest = min((g.block_size * g.num_blocks for g in groups if g.window == 0), default=0)
            self.graphs = DecodeGraphs(self, max_context or longest or max((g.block_size * g.num_blocks for g in groups), default=1))

    # --- construction helpers -----------------------------------------------------------------
    @staticmethod
    def load_model(folder: str, config: ModelConfig, runtime: Runtime, progress=None, keep_float32: bool = False):
        """The model of ``config`` with the weights of ``folder`` on the runtime's device.  A model with a size that
        no kernel takes is refused when it is built, before the folder's tensors are opened.  ``keep_float32``:
        matrices that the folder stores in 32-bit stay so in a bfloat16 run (see ``weights.kept_dtype``)."""
        model = build_model(config, runtime)
        checkpoint = Checkpoint(folder)
        try:
            tensors = load_tensors(checkpoint, model.tensor_specs(), runtime.dtype, runtime.device, progress,
                                   keep_float32)
        finally:
            checkpoint.close()
        model.load(tensors)
        return model

    @classmethod
    def from_folder(cls, folder: str, dtype="bfloat16", device="cuda:0", block_size: int = 16,
                    num_blocks: int = 256, num_slots: int = 8, progress=None, use_graphs: bool = False,
                    max_context: int = 0, keep_float32: bool = False) -> "ModelRunner":
        runtime = Runtime(device, dtype)
        model = cls.load_model(folder, load_config(folder), runtime, progress, keep_float32)
        return cls(model, runtime, block_size, num_blocks, num_slots, use_graphs, max_context)

    # --- the step ---------------------------------------------------------------------------------
    def prepare(self, entries: Sequence[StepEntry]) -> StepBatch:
        batch = build_batch(entries, self.cache, self.vocab_size, self.runtime.device)
        batch.sampled_tokens = self.sampled_tokens
        return batch

    def run(self, batch: StepBatch) -> Optional[torch.Tensor]:
        self.steps += 1
        return self.model.forward(batch, self.storage)

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Logits ``[wanted, vocab]`` (32-bit, on the device) in the order of the entries and their ``want``.

        With captured steps the tensor may be a view of a graph's own output buffer, which the next step of the
        same size overwrites: it holds this step's logits until the next call of ``step``, in stream order.  A
        caller that keeps logits longer copies them."""
        if self.graphs is not None and self.graphs.wants(entries):
            self.steps += 1
            return self.graphs.step(entries)
        return self.run(self.prepare(entries))
