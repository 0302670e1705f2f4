"""The Python entry point: requests in, tokens out.

``Engine`` puts the parts together: a model with its weights, the cache manager and its device
memory, the step function, the scheduler above it and the sampler.  Its methods mirror the
reference's ``Engine`` (crates/vipera-runtime/src/engine.rs:329-1232): ``add_request`` is ``admit`` +
``enqueue``, ``step`` makes one scheduling decision and one forward pass and samples, ``generate``
runs until the given requests are done.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch

from ..errors import InfeasibleError, InvalidArgumentError, ViperaError
from ..runtime import Runtime
from ..sampling import RECENT_WINDOW, BatchSampler, RowRequest, SamplingParams, seeded_state
from .batch import StepEntry
from .runner import ModelRunner
from .scheduler import FINISH_NAMES, FINISH_STOP, NOT_FINISHED, Scheduler


@dataclass
class Generation:
    """A finished request (engine.rs:308-327)."""

    request: int
    prompt_tokens: int
    tokens: List[int]            # generated ids, the end-of-sequence token included when one ended it
    finish: str                  # "stop" | "length" | "cancelled" | "error"
    processed_tokens: int = 0    # tokens run through the model, recomputation after preemption included
    preemptions: int = 0
    error: Optional[str] = None


@dataclass
class StepToken:
    request: int
    token: int


@dataclass
class StepReport:
    """What one step did (engine.rs:283-304), plus the requests it preempted."""

    tokens: List[StepToken] = field(default_factory=list)
    finished: List[Generation] = field(default_factory=list)
    failed: List[Tuple[int, str]] = field(default_factory=list)
    preempted: List[int] = field(default_factory=list)
    num_batched_tokens: int = 0


@dataclass
class _Live:
    prompt: List[int]
    generated: List[int]
    params: SamplingParams
    eos: frozenset
    draws: int = 0            # uniforms its generator has given out
    seeded: bool = False      # whether the slot it holds now has its generator's state
    processed: int = 0
    preemptions: int = 0
    on_token: Optional[Callable[[int], None]] = None


@dataclass
class _InFlight:
    """A launched step whose sampled tokens are still on their way: per row the request, and why the
    scheduler ended it when the placeholder was appended (NOT_FINISHED if it did not)."""

    pending: object                      # sampling.PendingSample
    requests: List[int]
    reasons: List[int]
    row_of: Dict[int, int]               # request -> its row of the sampler's output


def _recent_tokens(live) -> List[int]:
    """The last RECENT_WINDOW tokens of a request (prompt then generated): all that the penalties look at."""
    generated = live.generated[-RECENT_WINDOW:]
    missing = RECENT_WINDOW - len(generated)
    return (live.prompt[-missing:] if missing > 0 else []) + generated


class Engine:
    """Continuous-batching generation on one GPU.

    ``model``: a folder with ``config.json`` and ``model.safetensors``.  ``dtype``: ``"bfloat16"``
    or ``"float32"``.  The cache has ``num_blocks`` pages of ``block_size`` positions per group of
    layers (each one number for every group, or a list with one per group in the order in which the model's
    layers first need each group); when ``num_blocks`` is absent it is sized for ``max_num_seqs`` requests of
    ``max_model_len`` tokens, bounded by free device memory.  ``use_graphs`` (default on) replays
    steps of single tokens as captured HIP graphs.

    ``pipelined``: a step is launched before the tokens of the step before have reached the host (they
    are read on the device, where the sampler left them), and ``step()`` reports the tokens of the step
    *before* the one it launches; the GPU then never waits for the host between steps.  What is generated
    is the same.  A request that ends on an end-of-sequence token has one token more computed, which is
    dropped.  While a live request uses penalties (they look at the last tokens on the host), steps run
    one after the other as without the option.

    ``keep_float32``: matrices that the folder stores in 32-bit stay in 32-bit in a bfloat16 run instead of being
    converted to bfloat16 when they are loaded; their products then run through the 32-bit kernel.

    ``eager_admission``: start a waiting request as soon as its first portion finds pages, instead of only
    when all its tokens fit beside what the running requests still need (see ``csrc/host/scheduler.h``).
    """

    def __init__(self, model: str, dtype: str = "bfloat16", device: str = "cuda:0", block_size: int = 16,
                 num_blocks: Optional[int] = None, max_num_seqs: int = 8, max_num_batched_tokens: int = 2048,
                 chunk_size: int = 512, max_model_len: Optional[int] = None,
                 eos_token_ids: Optional[Sequence[int]] = None, runner: Optional[ModelRunner] = None,
                 use_graphs: Optional[bool] = None, pipelined: bool = False, eager_admission: bool = False,
                 keep_float32: bool = False):
        if runner is None:
            runtime = Runtime(device, dtype)
            from ..config.registry import load_config
            config = load_config(model)
            limit = int(max_model_len or config.context_limit)
            if limit > config.context_limit:
                raise InvalidArgumentError(
                    f"requested context {limit} exceeds the model's maximum of {config.context_limit}")
            if num_blocks is None:
                sizes = [block_size] if isinstance(block_size, int) else list(block_size)
                counts = [max_num_seqs * ((limit + size - 1) // size) for size in sizes]
                num_blocks = counts[0] if isinstance(block_size, int) else counts
            if use_graphs is None:
                use_graphs = True
            runner = self._load(model, config, runtime, block_size, num_blocks, max_num_seqs, use_graphs, limit,
                                keep_float32)
        else:  # a runner that is already set up (its model, cache and graphs are used as they are)
            config = runner.model.config
            limit = int(max_model_len or config.context_limit)
        self.runner = runner
        self.config = config
        self.max_model_len = limit
        self.scheduler = Scheduler(runner.cache, max_num_seqs, max_num_batched_tokens, chunk_size, limit,
                                   eager_admission)
        self.sampler = BatchSampler(runner.runtime.device, out=runner.sampled_tokens,
                                    slot_table=runner.storage.slot_table)
        self.pipelined = bool(pipelined) and runner.sampled_tokens is not None
        self._inflight: Optional[_InFlight] = None   # the launched step whose tokens have not been collected
        default_eos = getattr(config, "eos_token_ids", ()) or ()
        self.eos_token_ids = frozenset(eos_token_ids if eos_token_ids is not None else default_eos)
        self._live: Dict[int, _Live] = {}
        self._next_id = 0
        self.generations = 0
        self.failed = 0
        self.step_count = 0
        # host microseconds by stage, as the reference's per-turn log keeps them (crates/vipera-runtime/src/
        # pipeline.rs:251-270): deciding the step, reserving and giving back pages (counted by the cache manager
        # itself, inside the scheduler's calls and outside them), packing and launching the model, sampling
        self.micros = {"schedule": 0, "allocate": 0, "compute": 0, "sample": 0}
        self._allocate_seen = runner.cache.allocate_micros()
        self.max_num_seqs = int(max_num_seqs)

    def warm_up(self, max_batch: Optional[int] = None, max_context: Optional[int] = None) -> int:
        """Capture the decode steps of every batch size up to ``max_batch`` requests (default: ``max_num_seqs``)
        and every context length up to ``max_context`` (default: the engine's limit) before the first request
        needs them; without it a step is captured when its size first occurs, which stalls that step for tens
        of milliseconds.  Returns the number of steps captured (0 for an engine without captured steps)."""
        graphs = getattr(self.runner, "graphs", None)
        if graphs is None:
            return 0
        return graphs.capture_ahead(int(max_batch or self.max_num_seqs), int(max_context or self.max_model_len))

    @staticmethod
    def _load(folder, config, runtime, block_size, num_blocks, num_slots, use_graphs, max_context,
              keep_float32=False) -> ModelRunner:
        from ..cache import cache_bytes, group_position_bytes, plan_groups

        model = ModelRunner.load_model(folder, config, runtime, keep_float32=keep_float32)
        free, _ = torch.cuda.mem_get_info(runtime.device)
        num_slots = max(num_slots, 1)
        element = 4 if runtime.dtype == torch.float32 else 2
        needs = model.cache_needs()
        _, per_slot = cache_bytes(needs, element)
        room = 0.9 * free - per_slot * (num_slots + 1)       # fixed-size state first: one row per slot and a scratch row
        if room < 0:
            raise InfeasibleError(
                f"no room for {num_slots} state slots of {per_slot} bytes in {free} free bytes of device memory")
        groups = plan_groups(needs, block_size, num_blocks)
        per_page = [spec.block_size * per_position
                    for spec, per_position in zip(groups, group_position_bytes(needs, element))]
        wanted = sum(spec.num_blocks * page for spec, page in zip(groups, per_page))
        if wanted > room:   # every pool shrinks by the same share
            counts = [int(spec.num_blocks * room / wanted) for spec in groups]
            if min(counts) < 1:
                raise InfeasibleError(
                    f"no room for a single cache page of {max(per_page)} bytes per group in {free} free bytes of "
                    "device memory")
            num_blocks = counts if not isinstance(num_blocks, int) else min(counts)
        return ModelRunner(model, runtime, block_size, num_blocks, num_slots, use_graphs, max_context)

    # --- requests ---------------------------------------------------------------------------------
    def add_request(self, prompt: Sequence[int], max_new_tokens: int = 32,
                    sampling: Optional[SamplingParams] = None, eos_token_ids: Optional[Sequence[int]] = None,
                    on_token: Optional[Callable[[int], None]] = None) -> int:
        """Queue a request and return its id. Refuses what can never run, before any work."""
        params = sampling or SamplingParams()
        params.validate()
        prompt = [int(t) for t in prompt]
        for token in prompt:
            if not 0 <= token < self.runner.vocab_size:
                raise InvalidArgumentError(f"token {token} is outside the vocabulary of {self.runner.vocab_size}")
        request = self._next_id
        self.scheduler.add(request, prompt, int(max_new_tokens))
        self._next_id += 1
        eos = frozenset(eos_token_ids) if eos_token_ids is not None else self.eos_token_ids
        self._live[request] = _Live(prompt, [], params, eos, on_token=on_token)
        return request

    def cancel(self, request: int) -> Optional[Generation]:
        """Remove a request at a step boundary; its pages are free afterwards."""
        live = self._live.pop(request, None)
        if live is None:
            return None
        self.scheduler.cancel(request)
        return Generation(request, len(live.prompt), live.generated, "cancelled", live.processed, live.preemptions)

    def _row(self, entry, recent=()) -> RowRequest:
        """How the last token of ``entry`` is sampled: from the generator in the request's slot, which is seeded
        when the request draws for the first time in that slot (at its start, or wound forward by the draws it
        had made when it comes back after a preemption)."""
        live = self._live[entry.request]
        seed_state = None if live.seeded else seeded_state(live.params.seed, live.draws)
        return RowRequest(live.params, self.runner.cache.slot(entry.request), entry.start + len(entry.tokens), recent,
                          seed_state)

    def _launch_sampling(self, logits, wanting, rows, report: StepReport):
        """Launch the sampling of ``rows`` (one per entry of ``wanting``).  Only once the launch has gone through is
        it booked on the host that these requests' slots hold their generators and that each drawing row has used
        one uniform: a launch that raises leaves the host's counts where the device's generators are, and fails the
        requests it was for.  Returns the pending sample, or None after a failure."""
        try:
            pending = self.sampler.launch(logits, rows)
        except ViperaError as err:
            for e in wanting:
                self._fail(e.request, str(err), report)
            return None
        for e in wanting:
            live = self._live[e.request]
            live.seeded = True
            if not live.params.greedy:
                live.draws += 1
        return pending

    def _note_preempted(self, plan, report: StepReport) -> None:
        for request in plan.preempted:
            if request in self._live:
                self._live[request].preemptions += 1
                self._live[request].seeded = False      # its slot is given back; the next one starts unseeded
        report.preempted = list(plan.preempted)

    def has_work(self) -> bool:
        return self.scheduler.has_work() or self._inflight is not None

    # --- one step -----------------------------------------------------------------------------------
    def step(self) -> StepReport:
        if self.pipelined and not any(live.params.penalizes for live in self._live.values()):
            return self._step_ahead()
        report = StepReport()
        if self._inflight is not None:  # leaving the pipelined way: first take in what is on its way
            self._collect(report)
        return self._step_in_turn(report)

    def _step_ahead(self) -> StepReport:
        """Launch the next step, then take in the tokens of the step launched before it."""
        report = StepReport()
        self._book("", 0.0)     # pages moved since the last step (requests added or cancelled) are booked first
        started = time.perf_counter()
        plan = self.scheduler.plan()
        self._note_preempted(plan, report)
        scheduled = time.perf_counter()
        self._book("schedule", scheduled - started)
        previous, launched = self._inflight, None
        if plan.entries:
            entries = []
            for e in plan.entries:
                # the last token of a request whose sample is still on its way is a placeholder on the host:
                # the step reads it from the sampler's output on the device
                source = -1
                if previous is not None and len(e.tokens) == 1 and e.request in previous.row_of \
                        and e.start + 1 == self.scheduler.length_of(e.request):
                    source = previous.row_of[e.request]
                entries.append(StepEntry(e.request, e.start, e.tokens, [len(e.tokens) - 1] if e.wants_logits else [],
                                         source))
            report.num_batched_tokens = plan.num_tokens
            self.step_count += 1
            try:
                logits = self.runner.step(entries)
            except ViperaError as err:
                if previous is not None:
                    self._collect(report)
                for e in plan.entries:
                    self._fail(e.request, str(err), report)
                return report
            for e in plan.entries:
                self.scheduler.advance(e.request)
                self._live[e.request].processed += len(e.tokens)
            wanting = [e for e in plan.entries if e.wants_logits]
            pending = self._launch_sampling(logits, wanting, [self._row(e) for e in wanting], report) if wanting else None
            if pending is not None:
                # the scheduler goes on as if the token were known: a placeholder stands for it until it arrives
                reasons = [self.scheduler.append(e.request, 0, False) for e in wanting]
                launched = _InFlight(pending, [e.request for e in wanting], reasons,
                                     {e.request: row for row, e in enumerate(wanting)})
        computed = time.perf_counter()
        self._book("compute", computed - scheduled)
        self._inflight = previous
        if previous is not None:
            self._collect(report, newer=launched)
        self._inflight = launched
        self._book("sample", time.perf_counter() - computed)
        return report

    def _collect(self, report: StepReport, newer: Optional[_InFlight] = None) -> None:
        """Take in the tokens of the step in flight. ``newer``: a step launched after it, in which the same
        requests may already hold one more placeholder."""
        flight, self._inflight = self._inflight, None
        tokens = self.sampler.collect(flight.pending)
        for request, reason, token in zip(flight.requests, flight.reasons, tokens):
            live = self._live.get(request)
            if live is None:  # ended, failed or cancelled since the launch: what was computed for it is dropped
                continue
            if token < 0:
                self._fail(request, "the logits hold no finite value", report)
                continue
            live.generated.append(token)
            is_eos = token in live.eos
            report.tokens.append(StepToken(request, token))
            if is_eos:
                reason = FINISH_STOP
                self.scheduler.cancel(request)   # a no-op if the scheduler ended it at its token budget already
            else:
                back = 1 if newer is not None and request in newer.row_of else 0
                self.scheduler.replace_token(request, back, token)
                if live.on_token is not None:
                    live.on_token(token)
            if reason != NOT_FINISHED:
                self._live.pop(request)
                self.generations += 1
                report.finished.append(Generation(request, len(live.prompt), live.generated, FINISH_NAMES[reason],
                                                  live.processed, live.preemptions))

    def _book(self, stage: str, seconds: float) -> None:
        """Book ``seconds`` of host time: what the cache manager spent on pages since the last booking is
        ``allocate`` (it happens inside the scheduler's decisions, after a step, and when a request ends), the rest
        goes to ``stage``."""
        now = self.runner.cache.allocate_micros()
        pages, self._allocate_seen = now - self._allocate_seen, now
        self.micros["allocate"] += pages
        if stage:
            self.micros[stage] += max(0, int(seconds * 1e6) - pages)

    def _step_in_turn(self, report: StepReport) -> StepReport:
        self._book("", 0.0)
        started = time.perf_counter()
        plan = self.scheduler.plan()
        self._note_preempted(plan, report)
        scheduled = time.perf_counter()
        self._book("schedule", scheduled - started)
        if not plan.entries:
            return report
        entries = [StepEntry(e.request, e.start, e.tokens, [len(e.tokens) - 1] if e.wants_logits else [])
                   for e in plan.entries]
        report.num_batched_tokens = plan.num_tokens
        self.step_count += 1
        try:
            logits = self.runner.step(entries)
        except ViperaError as err:  # every request of the batch fails and gives back what it holds
            for e in plan.entries:
                self._fail(e.request, str(err), report)
            return report
        for e in plan.entries:
            self.scheduler.advance(e.request)
            self._live[e.request].processed += len(e.tokens)
        wanting = [e for e in plan.entries if e.wants_logits]
        computed = time.perf_counter()
        self._book("compute", computed - scheduled)
        if wanting:
            rows = []
            for e in wanting:
                live = self._live[e.request]
                rows.append(self._row(e, _recent_tokens(live) if live.params.penalizes else ()))
            pending = self._launch_sampling(logits, wanting, rows, report)
            tokens = self.sampler.collect(pending) if pending is not None else []
            for e, token in zip(wanting, tokens):
                if token < 0:
                    self._fail(e.request, "the logits hold no finite value", report)
                    continue
                live = self._live[e.request]
                live.generated.append(token)
                is_eos = token in live.eos
                reason = self.scheduler.append(e.request, token, is_eos)
                report.tokens.append(StepToken(e.request, token))
                if not is_eos and live.on_token is not None:
                    live.on_token(token)
                if reason != NOT_FINISHED:
                    self._live.pop(e.request)
                    self.generations += 1
                    report.finished.append(Generation(e.request, len(live.prompt), live.generated,
                                                      FINISH_NAMES[reason], live.processed, live.preemptions))
        self._book("sample", time.perf_counter() - computed)
        return report

    def _fail(self, request: int, message: str, report: StepReport) -> None:
        live = self._live.pop(request, None)
        self.scheduler.cancel(request)
        self.failed += 1
        report.failed.append((request, message))
        if live is not None:
            report.finished.append(Generation(request, len(live.prompt), live.generated, "error", live.processed,
                                              live.preemptions, message))

    # --- whole generations --------------------------------------------------------------------------
    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 32,
                 sampling=None, eos_token_ids: Optional[Sequence[int]] = None) -> List[Generation]:
        """Run ``prompts`` to the end; ``sampling`` is one :class:`SamplingParams` or one per prompt."""
        if sampling is None or isinstance(sampling, SamplingParams):
            sampling = [sampling] * len(prompts)
        if len(sampling) != len(prompts):
            raise InvalidArgumentError(f"{len(sampling)} sampling settings for {len(prompts)} prompts")
        ids = [self.add_request(p, max_new_tokens, s, eos_token_ids) for p, s in zip(prompts, sampling)]
        done: Dict[int, Generation] = {}
        idle = 0
        while len(done) < len(ids):
            report = self.step()
            for generation in report.finished:
                done[generation.request] = generation
            idle = idle + 1 if report.num_batched_tokens == 0 else 0
            if idle > 2:
                raise InfeasibleError("the scheduler can run none of the waiting requests")
        return [done[i] for i in ids]

    def stats(self) -> dict:
        """Counters in the manner of the reference's ``RuntimeStats`` (engine.rs:95-110)."""
        cache = self.runner.cache
        return {
            "requests": len(self._live),
            "waiting": self.scheduler.num_waiting,
            "running": self.scheduler.num_running,
            "kv_used_blocks": [cache.used_blocks(g) for g in range(len(cache.groups))],
            "kv_free_blocks": [cache.free_blocks(g) for g in range(len(cache.groups))],
            "kv_bytes": self.runner.storage.bytes,
            "generations": self.generations,
            "failed": self.failed,
            "preemptions": self.scheduler.preemptions,
            "steps": self.step_count,
            "micros": dict(self.micros),
        }
