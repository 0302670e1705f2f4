"""Captured decode steps: a step of single tokens replayed as one HIP graph.

A decode step launches a few hundred small kernels; launched one by one from Python the host is
slower than the GPU.  A graph of the step is captured once per (padded batch size, context bucket)
and replayed with new metadata copied into its standing buffers.  The kernels, their order and their
arithmetic are those of the eager step.  Nothing that clears memory is recorded into a graph.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence, Tuple

import numpy as np
import torch

from .batch import PackedStep, StepEntry, batch_from_buffer, pack_entries

BATCH_BUCKETS = (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 192, 256)


def _bucket(value: int, buckets: Sequence[int]) -> Optional[int]:
    for b in buckets:
        if value <= b:
            return b
    return None


class _Captured:
    def __init__(self, graph, buffer, staging, batch, logits):
        self.graph, self.buffer, self.staging, self.batch, self.logits = graph, buffer, staging, batch, logits


class DecodeGraphs:
    """Graphs of the runner's model for steps in which every entry holds one token."""

    def __init__(self, runner, max_context: int):
        self.runner = runner
        self.max_context = max_context
        self.graphs: Dict[Tuple[int, int], _Captured] = {}
        self.pool = None
        self.replays = 0

    def _context_bucket(self, kv_len: int) -> int:
        bucket = 256
        while bucket < kv_len:
            bucket *= 2
        return bucket

    def wants(self, entries: Sequence[StepEntry]) -> bool:
        return (all(len(e.tokens) == 1 for e in entries) and _bucket(len(entries), BATCH_BUCKETS) is not None)

    def _pack(self, entries, batch_bucket: int, context_bucket: int) -> PackedStep:
        cache = self.runner.cache
        width = max((context_bucket + g.block_size - 1) // g.block_size for g in cache.groups) if cache.groups else 1
        packed = pack_entries(entries, cache, self.runner.vocab_size, min_table_width=width,
                              pad_entries=batch_bucket - len(entries), pad_page=self.runner.num_blocks)
        # every row's logits are computed; the caller picks the wanted ones
        packed.sections[7] = np.arange(batch_bucket, dtype=np.int32)
        packed.num_logit_rows = batch_bucket
        packed.max_decode_kv_len = context_bucket
        packed.max_kv_len = context_bucket
        return packed

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Logits ``[wanted, vocab]`` like the eager step; ``want`` of an entry is ``[]`` or ``[0]``."""
        runner = self.runner
        batch_bucket = _bucket(len(entries), BATCH_BUCKETS)
        longest = max(e.start + 1 for e in entries)
        context_bucket = self._context_bucket(longest)
        packed = self._pack(entries, batch_bucket, context_bucket)
        flat = packed.flat()
        key = (batch_bucket, context_bucket)
        captured = self.graphs.get(key)
        if captured is None:
            device = runner.runtime.device
            staging = torch.empty(flat.size, dtype=torch.int32).pin_memory()
            buffer = torch.empty(flat.size, dtype=torch.int32, device=device)
            staging.numpy()[:] = flat
            buffer.copy_(staging, non_blocking=True)
            batch = batch_from_buffer(packed, buffer)
            # an eager run first: it loads every kernel module the step needs, outside of the capture
            runner.model.forward(batch, runner.storage)
            torch.cuda.synchronize(device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool=self.pool):
                logits = runner.model.forward(batch, runner.storage)
            if self.pool is None:
                self.pool = graph.pool()
            captured = _Captured(graph, buffer, staging, batch, logits)
            self.graphs[key] = captured
        else:
            captured.staging.numpy()[:] = flat
            captured.buffer.copy_(captured.staging, non_blocking=True)
        captured.graph.replay()
        self.replays += 1
        rows = [k for k, e in enumerate(entries) if len(e.want)]
        if len(rows) == batch_bucket:
            return captured.logits
        index = torch.tensor(rows, dtype=torch.long, device=captured.logits.device)
        return captured.logits.index_select(0, index)
