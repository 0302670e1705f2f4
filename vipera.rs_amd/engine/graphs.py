"""Captured decode steps: a step of single tokens replayed as one HIP graph.

A decode step launches a few hundred small kernels; launched one by one from Python the host is
slower than the GPU.  A graph of the step is captured once per (padded batch size, context bucket,
fill class) and replayed with new metadata copied into its standing buffers.  The kernels, their order and
their arithmetic are those of the eager step.  Nothing that clears memory is recorded into a graph.

The fill class says which share of batch size x context bucket the entries' positions take up: the launches
of a step may depend on it (the attention over single tokens cuts the positions into shorter chunks where
most entries are short), and a graph holds the launches of its capture.  Classes whose launches come out the
same share one graph.

A graph is warmed up and captured on a step of padding entries only (token 0 at position 0 on the scratch
page and the scratch state row), so that a real step runs exactly once, as the graph's first replay: a
mixer that keeps state advances it once.
"""
from __future__ import annotations

import gc
from typing import Dict, Optional, Sequence, Tuple

import numpy as np
import torch

from ..ops import kernels
from .batch import PackedStep, StepEntry, batch_from_buffer, pack_entries

# Padded batch sizes of the captured steps. A padding entry sees no positions, but its row of activations is read by
# every workgroup of the products that stream weights in wave order (up to 8 tokens), so 5 and 6 requests have a
# size of their own below 8 (the 7B shape: 5 requests as 8 took 3.60 ms a step, as 6 they take 3.48; 4 take 3.37),
# and 9 to 12 one below 16 (9 requests 3.93 to 3.84 ms). Past 64 the sizes are 16 apart, then 32: a step of 96 tokens
# costs what 96 cost in every product (72 requests as 96 took 8.02 ms, as 80 they take 7.69).
BATCH_BUCKETS = (1, 2, 4, 6, 8, 12, 16, 24, 32, 48, 64, 80, 96, 112, 128, 160, 192, 224, 256)

# The shares of batch bucket x context bucket that a captured step's entries are taken to fill; a step replays the
# graph of the nearest one (in ratio).
FILL_CLASSES = (1.0, 0.5, 0.25)


def fill_class(total_kv_len: int, batch_bucket: int, context_bucket: int) -> int:
    share = total_kv_len / float(batch_bucket * context_bucket)
    return 0 if share > 0.7 else 1 if share > 0.35 else 2


def _bucket(value: int, buckets: Sequence[int]) -> Optional[int]:
    for b in buckets:
        if value <= b:
            return b
    return None


class _Captured:
    def __init__(self, graph, buffer, staging, batch, logits, plans):
        self.graph, self.buffer, self.staging, self.batch, self.logits = graph, buffer, staging, batch, logits
        self.plans = plans  # the launch decisions that the capture's step noted
        self.turn = 0  # which of the two staging buffers the last step used
        self.fetched = [None, None]  # per staging buffer: the event after the GPU's last read of it


class DecodeGraphs:
    """Graphs of the runner's model for steps in which every entry holds one token."""

    def __init__(self, runner, max_context: int):
        self.runner = runner
        self.max_context = max_context
        self.graphs: Dict[Tuple[int, int, int], _Captured] = {}
        self.pool = None
        self.replays = 0

    def _context_bucket(self, kv_len: int) -> int:
        bucket = 256
        while bucket < kv_len:
            bucket *= 2
        return bucket

    def wants(self, entries: Sequence[StepEntry]) -> bool:
        return (all(len(e.tokens) == 1 for e in entries) and _bucket(len(entries), BATCH_BUCKETS) is not None)

    def _pack(self, entries, batch_bucket: int, context_bucket: int, fill: int) -> PackedStep:
        cache = self.runner.cache
        width = max((context_bucket + g.block_size - 1) // g.block_size for g in cache.groups) if cache.groups else 1
        packed = pack_entries(entries, cache, self.runner.vocab_size, min_table_width=width,
                              pad_entries=batch_bucket - len(entries),
                              pad_slot=self.runner.storage.scratch_slot)
        # every row's logits are computed; the caller picks the wanted ones
        packed.sections[7] = np.arange(batch_bucket, dtype=np.int32)
        packed.num_logit_rows = batch_bucket
        packed.max_decode_kv_len = context_bucket
        packed.max_kv_len = context_bucket
        packed.sum_decode_kv_len = max(batch_bucket, int(FILL_CLASSES[fill] * batch_bucket * context_bucket))
        return packed

    def _capture(self, batch_bucket: int, context_bucket: int, fill: int, words: int) -> _Captured:
        """Warm up and capture the step of ``batch_bucket`` entries over ``context_bucket`` positions, filled as
        class ``fill`` says (on padding entries only), and keep it; ``words``: the length of such a step's
        packed metadata.  If the step's launches are those of another fill class's graph, that one is shared."""
        runner = self.runner
        device = runner.runtime.device
        padding = self._pack([], batch_bucket, context_bucket, fill)
        buffer = torch.from_numpy(padding.flat()).to(device)
        batch = batch_from_buffer(padding, buffer)
        batch.sampled_tokens = runner.sampled_tokens
        # an eager run first: it loads every kernel module the step needs, outside of the capture
        runner.model.forward(batch, runner.storage)
        torch.cuda.synchronize(device)
        plans = tuple(batch.launch_plans)
        for other in range(len(FILL_CLASSES)):
            same = self.graphs.get((batch_bucket, context_bucket, other))
            if same is not None and same.plans == plans:
                self.graphs[(batch_bucket, context_bucket, fill)] = same
                return same
        # two pinned staging buffers, used in turn: with steps launched ahead of their results, the copy of
        # the step before may still be waiting in the stream when the next step is packed
        staging = [torch.empty(words, dtype=torch.int32).pin_memory() for _ in range(2)]
        graph = torch.cuda.CUDAGraph()
        # No garbage collection while the stream is capturing: a collected object that holds pinned or
        # device memory, an event or another graph (an engine that is no longer used, say) would be
        # freed through calls that are not allowed during a capture, and the process would abort.
        # What is garbage now is collected before the capture starts.
        gc.collect()
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph, pool=self.pool):
                logits = runner.model.forward(batch, runner.storage)
        finally:
            if collecting:
                gc.enable()
        if self.pool is None:
            self.pool = graph.pool()
        captured = _Captured(graph, buffer, staging, batch, logits, plans)
        self.graphs[(batch_bucket, context_bucket, fill)] = captured
        return captured

    def capture_ahead(self, max_batch: int, max_context: int) -> int:
        """Capture the steps of every batch bucket up to ``max_batch`` entries and every context bucket up to
        ``max_context`` positions that are not captured yet, in every fill class, so that no step of a running
        engine has to (a capture drains the stream and takes tens of milliseconds). Returns how many were captured
        (fill classes that share a graph count once)."""
        top_batch = _bucket(max(1, min(max_batch, BATCH_BUCKETS[-1])), BATCH_BUCKETS)
        top_context = self._context_bucket(max(1, min(max_context, self.max_context)))
        def distinct() -> int:
            return len({id(captured) for captured in self.graphs.values()})

        before = distinct()
        for batch_bucket in BATCH_BUCKETS:
            if batch_bucket > top_batch:
                break
            context_bucket = 256
            while context_bucket <= top_context:
                for fill in range(len(FILL_CLASSES)):
                    if (batch_bucket, context_bucket, fill) not in self.graphs:
                        words = self._pack([], batch_bucket, context_bucket, fill).flat().size
                        self._capture(batch_bucket, context_bucket, fill, words)
                context_bucket *= 2
        return distinct() - before

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Logits ``[wanted, vocab]`` like the eager step; ``want`` of an entry is ``[]`` or ``[0]``."""
        runner = self.runner
        batch_bucket = _bucket(len(entries), BATCH_BUCKETS)
        longest = max(e.start + 1 for e in entries)
        context_bucket = self._context_bucket(longest)
        fill = fill_class(sum(e.start + 1 for e in entries), batch_bucket, context_bucket)
        packed = self._pack(entries, batch_bucket, context_bucket, fill)
        flat = packed.flat()
        captured = self.graphs.get((batch_bucket, context_bucket, fill))
        if captured is None:
            captured = self._capture(batch_bucket, context_bucket, fill, flat.size)
        captured.turn ^= 1
        staging = captured.staging[captured.turn]
        if captured.fetched[captured.turn] is not None:
            # a caller that never waits for results (steps in which no logits are wanted) could be more than two
            # steps ahead of the GPU: the buffer is not written before its last reader has run
            captured.fetched[captured.turn].synchronize()
        staging.numpy()[:] = flat
        # a kernel fetches the step's words from the pinned buffer: a copy command of this size goes to the copy
        # engine, whose hand-over leaves the GPU idle between two steps
        if not kernels.fetch_words(staging, captured.buffer):
            captured.buffer.copy_(staging, non_blocking=True)
        read = torch.cuda.Event()
        read.record()
        captured.fetched[captured.turn] = read
        captured.graph.replay()
        self.replays += 1
        rows = [k for k, e in enumerate(entries) if len(e.want)]
        if len(rows) == batch_bucket:
            return captured.logits
        if rows == list(range(len(rows))):
            # the usual case, every entry wants its logits and the padding comes last: a view of the first rows
            # (an index tensor made from a list is a blocking copy, which would end the launching ahead)
            return captured.logits[:len(rows)]
        index = torch.tensor(rows, dtype=torch.long, device=captured.logits.device)
        return captured.logits.index_select(0, index)
