"""Trace replay: feed given token ids through the engine's step function, as a trace dictates.

The trace is the schedule: each step lists requests with their next tokens and the places whose
logits are wanted; requests named in ``end`` give back their pages after the step.  No sampling,
no scheduler.  The model, the step function, the cache manager and the kernels are the ones that
generation uses.
"""
from __future__ import annotations

from typing import Callable, Dict, List, Optional

import numpy as np

from ..errors import InvalidArgumentError
from .batch import StepEntry
from .runner import ModelRunner


class Replayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, block_size: int = 16,
                 device: str = "cuda:0", log: Optional[Callable[[str], None]] = None, keep_float32: bool = False):
        if max_tokens < 1:
            raise InvalidArgumentError(f"--max-tokens must be at least 1, got {max_tokens}")
        if block_size < 1:
            raise InvalidArgumentError(f"--block-size must be at least 1, got {block_size}")
        # live requests hold at most max_tokens, each count rounded up to a multiple of 64; with pages
        # no larger than 64 positions that many tokens' worth of pages always suffices
        rounded = (max_tokens + 63) // 64 * 64
        page = block_size
        num_blocks = (rounded + page - 1) // page
        if page > 64 or 64 % page:
            num_blocks = (max_tokens + page - 1) // page + 4  # each of four live requests may waste a page
        if log:
            log(f"[trace_run] loading {model_dir} as {dtype}; {num_blocks} pages of {page} positions per cache group")
        self.runner = ModelRunner.from_folder(model_dir, dtype=dtype, device=device, block_size=page,
                                              num_blocks=num_blocks, num_slots=16, keep_float32=keep_float32)
        self.ids: Dict[str, int] = {}
        self.lengths: Dict[int, int] = {}
        self.next_id = 0
        if log:
            log("[trace_run] ready")

    def step(self, entries: List[dict], end: List[str]) -> Optional[np.ndarray]:
        cache = self.runner.cache
        step_entries: List[StepEntry] = []
        for entry in entries:
            name = str(entry["id"])
            tokens = [int(t) for t in entry["tokens"]]
            want = [int(w) for w in entry.get("want", [])]
            if name not in self.ids:
                self.ids[name] = self.next_id
                self.lengths[self.next_id] = 0
                self.next_id += 1
            request = self.ids[name]
            start = self.lengths[request]
            cache.reserve(request, start, start + len(tokens))
            step_entries.append(StepEntry(request, start, tokens, want))
        logits = None
        if step_entries:
            out = self.runner.step(step_entries)
            if out is not None:
                logits = out.float().cpu().numpy()
            for entry in step_entries:
                self.lengths[entry.request] = entry.start + len(entry.tokens)
                cache.advance(entry.request, self.lengths[entry.request])
        for name in end:
            name = str(name)
            if name in self.ids:
                request = self.ids.pop(name)
                if cache.knows(request):
                    cache.release(request)
                self.lengths.pop(request, None)
        return logits
