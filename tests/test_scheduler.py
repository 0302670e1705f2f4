"""The scheduler's decisions, without a model: a toy step stands in for the forward pass.

The toy favours token ``(last token + its position) % vocab``, like the reference's ``ToyForward``
(crates/vipera-runtime/src/engine.rs:1270-1331), so a request's continuation depends on exactly the
tokens and positions the scheduler feeds; any wrong portion shows as a wrong token.
"""
import random

import pytest

import vipera_rs_amd  # noqa: F401
from vipera_rs_amd.cache import CacheGroupSpec, CacheManager
from vipera_rs_amd.engine.scheduler import FINISH_LENGTH, FINISH_STOP, NOT_FINISHED, Scheduler
from vipera_rs_amd.errors import InfeasibleError, InvalidArgumentError

VOCAB = 97


def solo(prompt, max_new, eos=None):
    tokens, out = list(prompt), []
    for _ in range(max_new):
        token = (tokens[-1] + len(tokens) - 1) % VOCAB
        out.append(token)
        tokens.append(token)
        if token == eos:
            break
    return out


class Harness:
    def __init__(self, blocks=64, block_size=4, seqs=4, budget=32, chunk=8, max_len=256, window_blocks=None,
                 eager=False):
        groups = [CacheGroupSpec(block_size, blocks)]
        if window_blocks:
            groups.append(CacheGroupSpec(block_size, window_blocks, window=10))
        self.cache = CacheManager(groups, seqs)
        self.sched = Scheduler(self.cache, seqs, budget, chunk, max_len, eager_admission=eager)
        self.budget, self.chunk, self.seqs = budget, chunk, seqs
        self.fed = {}        # request -> tokens fed so far in its current run
        self.out = {}        # request -> generated tokens
        self.done = {}       # request -> finish code
        self.eos = {}
        self.history = []    # per step: list of (request, start, count)

    def add(self, rid, prompt, max_new, eos=None):
        self.sched.add(rid, prompt, max_new)
        self.out[rid] = []
        self.eos[rid] = eos

    def step(self):
        plan = self.sched.plan()
        for rid in plan.preempted:
            self.fed[rid] = []
        assert plan.num_tokens <= self.budget
        assert len(plan.entries) <= self.seqs
        record = []
        for e in plan.entries:
            assert 1 <= len(e.tokens) <= self.chunk
            fed = self.fed.setdefault(e.request, [])
            assert e.start == len(fed), "a portion must continue where the last one ended"
            for g in range(len(self.cache.groups)):   # every position of the portion is backed by a page
                table = self.cache.table(e.request, g)
                spec = self.cache.groups[g]
                lo = max(0, e.start + 1 - spec.window) if spec.window else 0
                for pos in range(lo, e.start + len(e.tokens)):
                    assert table[pos // spec.block_size] >= 0
            fed.extend(e.tokens)
            record.append((e.request, e.start, len(e.tokens)))
        self.history.append(record)
        for e in plan.entries:
            self.sched.advance(e.request)
        for e in plan.entries:
            if e.wants_logits:
                fed = self.fed[e.request]
                token = (fed[-1] + len(fed) - 1) % VOCAB
                self.out[e.request].append(token)
                reason = self.sched.append(e.request, token, token == self.eos[e.request])
                if reason != NOT_FINISHED:
                    self.done[e.request] = reason
        assert self.cache.check() == ""
        return plan

    def drain(self, limit=10_000):
        steps = 0
        while self.sched.has_work():
            plan = self.step()
            assert plan.entries, "a plan is empty although requests wait or run"
            steps += 1
            assert steps < limit, "the scheduler makes no progress"
        return steps


def prompt_of(n, seed):
    rng = random.Random(seed)
    return [rng.randrange(VOCAB) for _ in range(n)]


def test_a_batch_gives_every_request_its_solo_tokens():
    h = Harness()
    prompts = {r: prompt_of(n, r) for r, n in enumerate((5, 8, 13, 1))}
    for r, p in prompts.items():
        h.add(r, p, 9)
    h.drain()
    assert all(h.out[r] == solo(p, 9) for r, p in prompts.items())
    assert all(code == FINISH_LENGTH for code in h.done.values())
    assert h.cache.live_requests() == 0 and h.cache.free_blocks(0) == 64


def test_prompts_are_cut_under_the_token_budget_and_decodes_come_first():
    h = Harness(budget=10, chunk=6)
    h.add(0, prompt_of(3, 0), 30)
    h.step()                                    # request 0 is prefilled and decodes from now on
    h.add(1, prompt_of(40, 1), 4)
    for _ in range(6):
        plan = h.step()
        assert plan.entries[0].request == 0 and len(plan.entries[0].tokens) == 1   # decode is never starved
        assert len(plan.entries[1].tokens) == 6                                     # one portion under the chunk size
    h.drain()
    assert h.out[0] == solo(prompt_of(3, 0), 30) and h.out[1] == solo(prompt_of(40, 1), 4)
    assert max(sum(c for _, _, c in step) for step in h.history) <= 10


def test_the_budget_is_shared_by_several_prompts():
    h = Harness(budget=10, chunk=8)
    h.add(0, prompt_of(20, 0), 2)
    h.add(1, prompt_of(20, 1), 2)
    plan = h.step()
    assert [(e.request, len(e.tokens)) for e in plan.entries] == [(0, 8), (1, 2)]
    h.drain()
    assert h.out[1] == solo(prompt_of(20, 1), 2)


def test_admission_is_oldest_first_and_bounded():
    h = Harness(seqs=2)
    for r in range(4):
        h.add(r, prompt_of(4, r), 3)
    plan = h.step()
    assert [e.request for e in plan.entries] == [0, 1] and h.sched.num_waiting == 2
    order = []
    while h.sched.has_work():
        for e in h.step().entries:
            if e.request not in order:
                order.append(e.request)
    assert order == [0, 1, 2, 3] or order[:2] == [0, 1] and order[2:] == [2, 3]


def test_a_late_arrival_joins_the_running_batch():
    h = Harness()
    h.add(0, prompt_of(6, 0), 12)
    for _ in range(3):
        h.step()
    h.add(1, prompt_of(5, 1), 5)
    plan = h.step()
    assert sorted(e.request for e in plan.entries) == [0, 1]
    h.drain()
    assert h.out[0] == solo(prompt_of(6, 0), 12) and h.out[1] == solo(prompt_of(5, 1), 5)


def test_finishing_by_end_token_length_and_full_context():
    p = prompt_of(7, 3)
    free_run = solo(p, 10)
    h = Harness(max_len=256)
    h.add(0, p, 10, eos=free_run[4])
    h.drain()
    stop_at = free_run.index(free_run[4])
    assert h.out[0] == free_run[:stop_at + 1] and h.done[0] == FINISH_STOP     # the end token is kept
    h = Harness(max_len=12)
    h.add(0, p, 100)
    h.drain()
    assert len(p) + len(h.out[0]) == 12 and h.done[0] == FINISH_LENGTH          # the context is full
    assert h.cache.live_requests() == 0


def test_what_can_never_run_is_refused_before_any_work():
    h = Harness(blocks=4, block_size=4, max_len=64)
    with pytest.raises(InfeasibleError, match="more pages"):
        h.sched.add(0, prompt_of(30, 0), 4)        # 8 pages needed, 4 exist (engine.rs:396-424)
    with pytest.raises(InvalidArgumentError, match="at least one prompt token"):
        h.sched.add(1, [], 4)
    with pytest.raises(InvalidArgumentError, match="max_new_tokens"):
        h.sched.add(2, [1], 0)
    with pytest.raises(InfeasibleError, match="no room"):
        h.sched.add(3, prompt_of(64, 0), 4)
    h.sched.add(4, [1, 2], 3)
    with pytest.raises(InvalidArgumentError, match="already in use"):
        h.sched.add(4, [1, 2], 3)
    assert h.sched.num_waiting == 1 and h.cache.live_requests() == 0


def test_cancel_frees_pages_at_a_step_boundary():
    h = Harness()
    h.add(0, prompt_of(9, 0), 20)
    h.add(1, prompt_of(9, 1), 3)
    h.step()
    used = h.cache.used_blocks(0)
    assert h.sched.cancel(0) and h.cache.used_blocks(0) < used and not h.cache.knows(0)
    assert not h.sched.cancel(0)
    h.drain()
    assert h.out[1] == solo(prompt_of(9, 1), 3) and h.cache.used_blocks(0) == 0


def test_when_pages_run_out_the_newest_request_gives_way_and_is_recomputed():
    # three requests that grow to 9 pages together, 7 pages in the pool
    h = Harness(blocks=7, block_size=4, seqs=3, budget=32, chunk=8)
    prompts = {r: prompt_of(n, 10 + r) for r, n in enumerate((6, 5, 7))}
    for r, p in prompts.items():
        h.add(r, p, 6)
    preempted = []
    while h.sched.has_work():
        preempted += h.step().preempted
        assert len(h.history) < 500
    assert preempted and set(preempted) <= {1, 2} and preempted[0] == 2          # the most recently admitted goes first
    assert 0 not in preempted                                                    # the oldest always makes progress
    assert all(h.out[r] == solo(p, 6) for r, p in prompts.items())              # recomputation changes no token
    assert h.sched.preemptions == len(preempted)
    assert h.cache.free_blocks(0) == 7 and h.cache.live_requests() == 0
    # a preempted request restarts at position 0 and is fed everything it had, generated tokens included
    restarts = [step for step in h.history if any(r == preempted[0] and s == 0 for r, s, _ in step)]
    assert len(restarts) >= 2


def test_a_prompt_waits_for_pages_without_pushing_anyone_out():
    h = Harness(blocks=6, block_size=4, seqs=2, budget=32, chunk=8)
    h.add(0, prompt_of(16, 0), 3)      # two portions of 8: two pages each
    h.add(1, prompt_of(8, 1), 2)       # one portion of 8, then one decoded token on a third page
    first = h.step()
    assert [(e.request, len(e.tokens)) for e in first.entries] == [(0, 8), (1, 8)]
    second = h.step()                  # request 1 decodes (page 5 of 6); request 0's next portion needs two pages
    assert [(e.request, len(e.tokens)) for e in second.entries] == [(1, 1)] and second.preempted == []
    assert 1 in h.done                 # request 1 is finished and has given its pages back
    third = h.step()
    assert [(e.request, e.start, len(e.tokens)) for e in third.entries] == [(0, 8, 8)]
    h.drain()
    assert h.sched.preemptions == 0
    assert h.out[0] == solo(prompt_of(16, 0), 3) and h.out[1] == solo(prompt_of(8, 1), 2)


@pytest.mark.parametrize("seed", range(4))
def test_random_arrivals_on_a_small_cache_with_a_windowed_group(seed):
    rng = random.Random(seed)
    h = Harness(blocks=rng.randrange(10, 16), block_size=4, seqs=3, budget=rng.randrange(6, 20), chunk=rng.randrange(2, 9),
                window_blocks=rng.randrange(8, 12))
    expected, next_id = {}, 0
    for step in range(400):
        if rng.random() < 0.15 and next_id < 12:
            p, n = prompt_of(rng.randrange(1, 22), 100 * seed + next_id), rng.randrange(1, 12)
            h.add(next_id, p, n)
            expected[next_id] = solo(p, n)
            next_id += 1
        if h.sched.has_work():
            h.step()
    h.drain()
    assert h.out == expected
    assert h.cache.live_requests() == 0 and h.cache.check() == ""
    assert all(h.cache.used_blocks(g) == 0 for g in range(2))


def test_two_long_prompts_on_a_pool_that_holds_one_both_finish():
    # 10 pages of 16 positions; each 120-token prompt needs 8. Started side by side they would both stall
    # at 5 pages with nothing free: the second is admitted only once the first one's pages leave room.
    h = Harness(blocks=10, block_size=16, seqs=4, budget=32, chunk=16, max_len=256)
    prompts = {0: prompt_of(120, 0), 1: prompt_of(120, 1)}
    for r, p in prompts.items():
        h.add(r, p, 5)
    first = h.step()
    assert [(e.request, len(e.tokens)) for e in first.entries] == [(0, 16)]     # no room for request 1 beside it
    h.drain()
    assert all(h.out[r] == solo(p, 5) for r, p in prompts.items())
    assert h.sched.preemptions == 0
    assert h.cache.free_blocks(0) == 10 and h.cache.live_requests() == 0


def test_started_side_by_side_the_newer_of_two_stalled_prompts_gives_way():
    # the same pool and prompts with eager admission: both are started, both stall at 5 pages of 8 with nothing
    # free and no decoding request to push anyone out; the newer one gives way, the older one always moves
    h = Harness(blocks=10, block_size=16, seqs=4, budget=32, chunk=16, max_len=256, eager=True)
    prompts = {0: prompt_of(120, 0), 1: prompt_of(120, 1)}
    for r, p in prompts.items():
        h.add(r, p, 5)
    preempted = []
    while h.sched.has_work():
        plan = h.step()
        assert plan.entries, "a plan is empty although requests wait or run"
        assert not h.cache.knows(0) or plan.entries[0].request == 0      # the oldest moves in every step
        preempted += plan.preempted
        assert len(h.history) < 500
    assert preempted and set(preempted) == {1}
    assert all(h.out[r] == solo(p, 5) for r, p in prompts.items())
    assert h.cache.free_blocks(0) == 10 and h.cache.live_requests() == 0


def test_when_every_running_prompt_waits_for_a_page_the_newest_gives_way():
    # both requests run (their prompts fitted side by side when they were admitted) and have grown by decoding;
    # after a preemption both recompute, meet in the middle of their tokens with no page left, and the newer one
    # gives way instead of both waiting for ever
    h = Harness(blocks=6, block_size=4, seqs=3, budget=32, chunk=4, max_len=64)
    h.add(0, prompt_of(4, 0), 14)
    h.add(1, prompt_of(4, 1), 14)
    h.add(2, prompt_of(4, 2), 14)
    preempted = []
    while h.sched.has_work():
        plan = h.step()
        assert plan.entries
        preempted += plan.preempted
        assert len(h.history) < 2000
    assert preempted and 0 not in preempted
    assert all(h.out[r] == solo(prompt_of(4, r), 14) for r in range(3))
    assert h.cache.free_blocks(0) == 6 and h.cache.live_requests() == 0


def test_a_stall_of_running_prompts_is_broken_from_the_back():
    # admission is by the tokens known at the time; here two requests are put into the running list by hand
    # in a state that admission would not have produced (both mid-prompt, no page free)
    h = Harness(blocks=4, block_size=4, seqs=2, budget=8, chunk=4, max_len=64)
    h.add(0, prompt_of(12, 0), 2)
    plan = h.step()                       # request 0 holds one page
    assert [(e.request, len(e.tokens)) for e in plan.entries] == [(0, 4)]
    h.add(1, prompt_of(4, 1), 9)          # fits beside what request 0 still needs (two more pages) exactly
    plan = h.step()
    assert [(e.request, len(e.tokens)) for e in plan.entries] == [(0, 4), (1, 4)]
    plan = h.step()                       # request 1 decodes on the last free page, request 0's portion waits
    assert [(e.request, len(e.tokens)) for e in plan.entries] == [(1, 1)] and plan.preempted == []
    for _ in range(3):                    # request 1 decodes within its page
        plan = h.step()
        assert [(e.request, len(e.tokens)) for e in plan.entries] == [(1, 1)]
    plan = h.step()                       # request 1 needs a page too: it is the newest, so it gives way itself,
    assert plan.preempted == [1]          # and request 0 goes on in the same step
    assert [(e.request, e.start, len(e.tokens)) for e in plan.entries] == [(0, 8, 4)]
    h.drain()
    assert h.out[0] == solo(prompt_of(12, 0), 2) and h.out[1] == solo(prompt_of(4, 1), 9)


@pytest.mark.parametrize("eager", (False, True))
@pytest.mark.parametrize("seed", range(8))
def test_random_arrivals_of_long_prompts_on_pools_that_hold_one_or_two(seed, eager):
    rng = random.Random(1000 + seed)
    block_size = rng.choice((4, 8, 16))
    blocks = rng.randrange(6, 12)
    capacity = blocks * block_size
    h = Harness(blocks=blocks, block_size=block_size, seqs=4, budget=rng.randrange(8, 40), chunk=rng.randrange(3, 20),
                max_len=capacity + 8, eager=eager)
    expected, next_id = {}, 0
    for step in range(600):
        if rng.random() < 0.2 and next_id < 14:
            n = rng.randrange(1, 12)
            length = rng.randrange(capacity // 3, capacity - n)      # most pairs do not fit side by side
            p = prompt_of(length, 7000 * seed + next_id)
            h.add(next_id, p, n)
            expected[next_id] = solo(p, n)
            next_id += 1
        if h.sched.has_work():
            assert h.step().entries, "a plan is empty although requests wait or run"
    h.drain()
    assert h.out == expected
    assert h.cache.live_requests() == 0 and h.cache.check() == "" and h.cache.used_blocks(0) == 0
