"""The scheduler above the step function (decisions in the C++ host library).

It admits requests, cuts prompts into portions under a token budget, hands every decoding
request its one token, ends requests and gives back what they hold, and preempts the most
recently admitted running request when a decode token finds no page, or when every running prompt
waits for one.  See
``csrc/host/scheduler.h`` for the policy and what it takes from the reference's
``Engine`` (crates/vipera-runtime/src/engine.rs).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Sequence

from ..cache.manager import CacheManager, _host
from ..errors import InfeasibleError, InternalError, InvalidArgumentError

NOT_FINISHED, FINISH_STOP, FINISH_LENGTH = 0, 1, 2
FINISH_NAMES = {FINISH_STOP: "stop", FINISH_LENGTH: "length"}


@dataclass
class PlannedEntry:
    request: int
    start: int
    tokens: List[int]
    wants_logits: bool


@dataclass
class StepPlan:
    entries: List[PlannedEntry]
    preempted: List[int]

    @property
    def num_tokens(self) -> int:
        return sum(len(e.tokens) for e in self.entries)


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int, max_num_batched_tokens: int, chunk_size: int,
                 max_model_len: int, eager_admission: bool = False):
        if max_num_seqs < 1 or max_num_batched_tokens < 1 or chunk_size < 1 or max_model_len < 2:
            raise InvalidArgumentError(
                "scheduler limits must be positive: "
                f"max_num_seqs={max_num_seqs}, max_num_batched_tokens={max_num_batched_tokens}, "
                f"chunk_size={chunk_size}, max_model_len={max_model_len}")
        self.cache = cache
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        self.chunk_size = chunk_size
        self.max_model_len = max_model_len
        self._lib = _host()
        self._handle = self._lib.vk_sched_create(cache._handle, max_num_seqs, max_num_batched_tokens, chunk_size,
                                                 max_model_len, 1 if eager_admission else 0)
        if not self._handle:
            raise InternalError("the native scheduler could not be created")

    def __del__(self):
        handle, self._handle = getattr(self, "_handle", None), None
        if handle:
            self._lib.vk_sched_destroy(handle)

    def add(self, request: int, prompt: Sequence[int], max_new_tokens: int) -> None:
        """Queue a request; refuses what can never run (texts after engine.rs:396-424)."""
        arr = (ctypes.c_int * max(len(prompt), 1))(*prompt)
        code = self._lib.vk_sched_add(self._handle, request, arr, len(prompt), max_new_tokens)
        if code == 0:
            return
        if code == 1:
            raise InvalidArgumentError("a request needs at least one prompt token")
        if code == 2:
            raise InvalidArgumentError(f"max_new_tokens must be at least 1, got {max_new_tokens}")
        if code == 3:
            raise InfeasibleError(
                f"a request of {len(prompt)} prompt tokens and {max_new_tokens} new tokens needs more pages than "
                "the cache has; shorten the context or give the cache more pages")
        if code == 4:
            raise InfeasibleError(
                f"a prompt of {len(prompt)} tokens leaves no room to generate within the context of "
                f"{self.max_model_len}")
        raise InvalidArgumentError(f"request id {request} is already in use")

    def plan(self) -> StepPlan:
        num_tokens, num_preempted = ctypes.c_int(0), ctypes.c_int(0)
        n = self._lib.vk_sched_plan(self._handle, ctypes.byref(num_tokens), ctypes.byref(num_preempted))
        ids = (ctypes.c_ulonglong * max(n, 1))()
        starts = (ctypes.c_int * max(n, 1))()
        counts = (ctypes.c_int * max(n, 1))()
        wants = (ctypes.c_int * max(n, 1))()
        tokens = (ctypes.c_int * max(num_tokens.value, 1))()
        preempted = (ctypes.c_ulonglong * max(num_preempted.value, 1))()
        self._lib.vk_sched_plan_read(self._handle, ids, starts, counts, wants, tokens, preempted)
        entries, at = [], 0
        for k in range(n):
            entries.append(PlannedEntry(int(ids[k]), starts[k], list(tokens[at:at + counts[k]]), bool(wants[k])))
            at += counts[k]
        return StepPlan(entries, [int(preempted[k]) for k in range(num_preempted.value)])

    def advance(self, request: int) -> None:
        self._lib.vk_sched_advance(self._handle, request)

    def append(self, request: int, token: int, is_end_of_sequence: bool) -> int:
        return self._lib.vk_sched_append(self._handle, request, token, 1 if is_end_of_sequence else 0)

    def replace_token(self, request: int, back: int, token: int) -> bool:
        """Overwrite the generated token ``back`` places before the request's last one (a placeholder that
        was appended before the sampled token reached the host)."""
        return self._lib.vk_sched_replace_token(self._handle, request, back, token) == 0

    def cancel(self, request: int) -> bool:
        return self._lib.vk_sched_cancel(self._handle, request) == 0

    def has_work(self) -> bool:
        return bool(self._lib.vk_sched_has_work(self._handle))

    @property
    def num_waiting(self) -> int:
        return self._lib.vk_sched_num_waiting(self._handle)

    @property
    def num_running(self) -> int:
        return self._lib.vk_sched_num_running(self._handle)

    @property
    def preemptions(self) -> int:
        return self._lib.vk_sched_preemptions(self._handle)

    def length_of(self, request: int) -> int:
        return self._lib.vk_sched_length_of(self._handle, request)
