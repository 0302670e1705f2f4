"""Sampling options and the batched sampler that runs them on the device.

Names, meanings, defaults and validation of the options follow the reference's ``SamplerConfig``
(crates/vipera-sampler/src/lib.rs:36-115); a temperature of 0 selects greedy decoding and skips
every other filter (lib.rs:273-280).  The engine's default temperature is 0, as the reference's
engine and command line set it (crates/vipera-runtime/src/engine.rs:50-53, bins/vipera/src/main.rs:557-560).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..errors import InvalidArgumentError
from ..ops import kernels
from .rng import Rng

MAX_LOGIT_BIAS = 16
RECENT_WINDOW = 128  # tokens the penalties look back over (bins/vipera/src/main.rs:685)


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_k: int = 40
    top_p: float = 0.95
    min_p: float = 0.05
    repetition_penalty: float = 1.0
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    logit_bias: Tuple[Tuple[int, float], ...] = ()
    seed: int = 0

    def validate(self) -> None:
        """Reject values that cannot describe a distribution (lib.rs:73-115)."""
        def finite(v):
            return isinstance(v, (int, float)) and math.isfinite(v)

        if not finite(self.temperature) or self.temperature < 0.0:
            raise InvalidArgumentError("temperature must be a finite number at or above 0")
        if not isinstance(self.top_k, int) or self.top_k < 0:
            raise InvalidArgumentError("top_k must be an integer at or above 0")
        if not finite(self.top_p) or self.top_p <= 0.0 or self.top_p > 1.0:
            raise InvalidArgumentError("top_p must be greater than 0 and at most 1")
        if not finite(self.min_p) or self.min_p < 0.0 or self.min_p >= 1.0:
            raise InvalidArgumentError("min_p must be at least 0 and below 1")
        if not finite(self.repetition_penalty) or self.repetition_penalty <= 0.0:
            raise InvalidArgumentError("repetition_penalty must be a finite number above 0")
        for name in ("presence_penalty", "frequency_penalty"):
            value = getattr(self, name)
            if not finite(value) or not -2.0 <= value <= 2.0:
                raise InvalidArgumentError(f"{name} must be a finite number from -2 to 2")
        if len(self.logit_bias) > MAX_LOGIT_BIAS:
            raise InvalidArgumentError(f"logit_bias holds at most {MAX_LOGIT_BIAS} entries")
        for _, value in self.logit_bias:
            if not finite(value) or not -100.0 <= value <= 100.0:
                raise InvalidArgumentError("logit_bias values must be finite numbers from -100 to 100")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0

    @property
    def penalizes(self) -> bool:
        return (self.repetition_penalty != 1.0 or self.presence_penalty != 0.0 or self.frequency_penalty != 0.0)


@dataclass
class RowRequest:
    """What one row of logits is sampled with: options, the request's state slot (where its generator lives),
    the position the drawn token will take, its recent tokens, and ``seed_state``: the generator state to put
    into the slot first (the request's first row in this slot), or None to go on from what the slot holds."""

    params: SamplingParams
    slot: int = 0
    position: int = 0
    recent: Sequence[int] = ()
    seed_state: Optional[int] = None


def seeded_state(seed: int, draws: int = 0) -> int:
    """The generator state of a request with ``seed`` that has drawn ``draws`` times."""
    return Rng(seed).skip(draws).state


class PendingSample:
    """Tokens that have been drawn on the device and are on their way to the host."""

    def __init__(self, count: int, host: torch.Tensor, event):
        self.count, self.host, self.event = count, host, event


class BatchSampler:
    """Samples one token per row of ``[rows, vocab]`` logits on the device.

    Per-row options go up in one small copy; the drawn ids come back in one.  A request's generator lives in
    its row of ``slot_table`` (int64 ``[slots, 2]`` on the device: generator state, position of the next token)
    and the kernel advances it: each random row consumes exactly one uniform of its request's generator per
    token, so a request's stream does not depend on its company in the batch or on the order of arrival (the
    invariant of crates/vipera-runtime/src/engine.rs:665-670), and a step that is launched before the tokens
    of the step before have reached the host needs nothing from the host to draw.

    ``launch`` enqueues the work and returns at once, ``collect`` waits for the ids; ``out`` (optional,
    int32 on the device) is where the ids are left for a next step that reads them there.  Without a
    ``slot_table`` the sampler keeps one of ``slots`` rows of its own.
    """

    def __init__(self, device, out: Optional[torch.Tensor] = None, slot_table: Optional[torch.Tensor] = None,
                 slots: int = 64):
        self.device = torch.device(device)
        self.out = out
        self.slot_table = slot_table if slot_table is not None else torch.zeros((slots, 2), dtype=torch.int64,
                                                                                 device=self.device)
        # pinned host words of the per-row options and of the ids, two of each used in turn (a launch may
        # follow before the copies of the one before have run), and the options' place on the device
        self._options = [None, None]
        self._ids = [None, None]
        self._device_words = None
        self._turn = 0
        self._done = [None, None]

    def sample(self, logits: torch.Tensor, rows: Sequence[RowRequest]) -> List[int]:
        return self.collect(self.launch(logits, rows))

    def launch(self, logits: torch.Tensor, rows: Sequence[RowRequest]) -> PendingSample:
        count, vocab = logits.shape
        if count != len(rows):
            raise InvalidArgumentError(f"{count} rows of logits for {len(rows)} requests")
        if logits.dtype != torch.float32 or not logits.is_contiguous():
            raise InvalidArgumentError("logits must be contiguous float32")
        self._penalize(logits, rows, vocab)
        self._turn ^= 1
        turn = self._turn
        if self._done[turn] is not None:
            self._done[turn].synchronize()   # the launch that last used this pair of pinned buffers has run
        slots = self.slot_table.shape[0]
        for r in rows:
            if not 0 <= r.slot < slots:
                raise InvalidArgumentError(f"state slot {r.slot} is outside the table of {slots}")
        # one pinned staging buffer, one copy: seven 4-byte columns (of an even length, so that the 8-byte
        # column behind them is aligned), then the generator states for rows that seed their slot
        n = count + (count & 1)
        words = 10 * n
        if self._options[turn] is None or self._options[turn].numel() < words:
            self._options[turn] = torch.empty(max(words, 10 * 64), dtype=torch.int32).pin_memory()
            self._ids[turn] = torch.empty(max(count, 64), dtype=torch.int32).pin_memory()
        if self._device_words is None or self._device_words.numel() < words:
            self._device_words = torch.empty(max(words, 10 * 64), dtype=torch.int32, device=self.device)
        host = self._options[turn].numpy()
        host[0:count].view(np.float32)[:] = [r.params.temperature for r in rows]
        host[n:n + count] = [r.params.top_k for r in rows]
        host[2 * n:2 * n + count].view(np.float32)[:] = [r.params.top_p for r in rows]
        host[3 * n:3 * n + count].view(np.float32)[:] = [r.params.min_p for r in rows]
        host[4 * n:4 * n + count] = [r.slot for r in rows]
        host[5 * n:5 * n + count] = [r.position for r in rows]
        host[6 * n:6 * n + count] = [0 if r.seed_state is None else 1 for r in rows]
        host[8 * n:8 * n + 2 * count].view(np.uint64)[:] = [r.seed_state or 0 for r in rows]
        dev = self._device_words
        dev[:words].copy_(self._options[turn][:words], non_blocking=True)
        if self.out is not None:
            if count > self.out.numel():
                raise InvalidArgumentError(f"{count} rows to sample, the id buffer holds {self.out.numel()}")
            out = self.out[:count]
        else:
            out = torch.empty(count, dtype=torch.int32, device=self.device)
        kernels.sample(logits, dev[0:count].view(torch.float32), dev[n:n + count],
                       dev[2 * n:2 * n + count].view(torch.float32), dev[3 * n:3 * n + count].view(torch.float32),
                       None, out, slot=dev[4 * n:4 * n + count], position=dev[5 * n:5 * n + count],
                       reseed=dev[6 * n:6 * n + count], seed_state=dev[8 * n:8 * n + 2 * count].view(torch.int64),
                       slot_table=self.slot_table)
        ids = self._ids[turn]
        ids[:count].copy_(out, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        self._done[turn] = event
        return PendingSample(count, ids, event)

    def collect(self, pending: PendingSample) -> List[int]:
        pending.event.synchronize()
        return pending.host[:pending.count].tolist()

    def _penalize(self, logits: torch.Tensor, rows: Sequence[RowRequest], vocab: int) -> None:
        pen_rows: List[int] = []
        pen_tokens: List[int] = []
        pen_counts: List[int] = []
        bias_rows: List[int] = []
        bias_tokens: List[int] = []
        bias_values: List[float] = []
        for index, row in enumerate(rows):
            if row.params.penalizes and row.recent:
                counts = {}
                for token in list(row.recent)[-RECENT_WINDOW:]:
                    counts[token] = counts.get(token, 0) + 1
                for token, n in counts.items():
                    pen_rows.append(index)
                    pen_tokens.append(token)
                    pen_counts.append(n)
            seen = set()
            for token, value in sorted(row.params.logit_bias, key=lambda item: item[0]):
                if token not in seen and 0 <= token < vocab:  # the first entry of a token id stands
                    seen.add(token)
                    bias_rows.append(index)
                    bias_tokens.append(token)
                    bias_values.append(value)
        ints = lambda a: torch.tensor(a, dtype=torch.int32, device=self.device)  # noqa: E731
        floats = lambda a: torch.tensor(a, dtype=torch.float32, device=self.device)  # noqa: E731
        if pen_rows:
            kernels.penalize(logits, ints(pen_rows), ints(pen_tokens), ints(pen_counts),
                             floats([r.params.repetition_penalty for r in rows]),
                             floats([r.params.presence_penalty for r in rows]),
                             floats([r.params.frequency_penalty for r in rows]))
        if bias_rows:
            kernels.logit_bias(logits, ints(bias_rows), ints(bias_tokens), floats(bias_values))
