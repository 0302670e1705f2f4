"""The sampling kernels against the plain sampler.

Vectors from the reference's own tests: greedy ties go to the lowest id and non-finite logits are
skipped (crates/vipera-conformance/src/lib.rs:461-484); logits ``[ln 3, 0]`` at temperature 1 draw the
two tokens 0.75 / 0.25 of the time within 0.05 over 4,000 draws (crates/vipera-sampler/src/lib.rs:945-955);
``top_k = 1`` is the argmax.  The kept set after the cuts is compared with a sort-based plain
implementation; the draw is checked through its distribution, since the engine walks the kept tokens
in id order and the reference in order of probability.
"""
import math

import numpy as np
import pytest
import torch

from plain import sampler_plain

pytestmark = pytest.mark.gpu


def _sample(logits, temperature, top_k, top_p, min_p, uniform):
    from vipera_rs_amd.ops import kernels
    dev = "cuda:0"
    rows = logits.shape[0]
    t = lambda v, d: torch.tensor(np.broadcast_to(np.asarray(v), (rows,)).copy(), dtype=d, device=dev)  # noqa: E731
    out = torch.empty(rows, dtype=torch.int32, device=dev)
    kernels.sample(torch.tensor(logits, dtype=torch.float32, device=dev).contiguous(), t(temperature, torch.float32),
                   t(top_k, torch.int32), t(top_p, torch.float32), t(min_p, torch.float32),
                   t(uniform, torch.float64), out)
    return out.cpu().numpy()


def test_greedy_ties_and_non_finite():
    rows = np.array([
        [1.0, 3.0, 3.0, 2.0, -1.0],
        [float("nan"), float("inf"), 0.5, 0.5, float("-inf")],
        [-5.0, -2.0, -2.0, -7.0, -2.0],
        [float("nan")] * 5,
    ], dtype=np.float32)
    got = _sample(rows, 0.0, 40, 0.95, 0.05, 0.0)
    assert list(got[:3]) == [sampler_plain.greedy(r) for r in rows[:3]] == [1, 2, 1]
    assert got[3] == -1


@pytest.mark.parametrize("vocab", [300, 1000, 152064])
def test_greedy_matches_argmax_on_random_rows(vocab):
    rng = np.random.default_rng(vocab)
    rows = rng.normal(size=(5, vocab)).astype(np.float32)
    rows[0, 17] = rows[0].max() + 1
    rows[1, vocab - 1] = rows[1].max() + 1
    rows[2, 0] = rows[2, vocab - 1] = rows[2].max() + 1  # a tie between the ends
    got = _sample(rows, 0.0, 0, 1.0, 0.0, 0.0)
    assert list(got) == [int(np.argmax(r)) for r in rows]


def test_reference_frequencies_075_025():
    draws = 4000
    rng = sampler_plain.Rng(7)
    u = np.array([rng.next_f64() for _ in range(draws)])
    rows = np.tile(np.array([math.log(3.0), 0.0], dtype=np.float32), (draws, 1))
    got = _sample(rows, 1.0, 0, 1.0, 0.0, u)
    share = float(np.mean(got == 0))
    assert abs(share - 0.75) < 0.05, share


def test_top_k_one_is_argmax():
    rng = np.random.default_rng(3)
    rows = rng.normal(size=(64, 500)).astype(np.float32)
    got = _sample(rows, 0.8, 1, 1.0, 0.0, rng.random(64))
    assert list(got) == [int(np.argmax(r)) for r in rows]


def test_top_k_ties_keep_the_lowest_ids():
    row = np.array([1.0, 1.0, 1.0, 1.0, 0.0, 2.0], dtype=np.float32)
    u = np.linspace(0.0, 0.999, 512)
    got = _sample(np.tile(row, (512, 1)), 1.0, 3, 1.0, 0.0, u)
    assert set(got.tolist()) == {5, 0, 1}


@pytest.mark.parametrize("vocab,temperature,top_k,top_p,min_p", [
    (300, 0.8, 40, 0.95, 0.05),
    (300, 1.3, 0, 0.9, 0.0),
    (1000, 0.7, 0, 1.0, 0.1),
    (1000, 1.0, 25, 1.0, 0.0),
    (5000, 0.5, 0, 0.5, 0.0),
    (152064, 0.8, 40, 0.95, 0.05),
    (152064, 1.0, 0, 0.8, 0.0),
])
def test_kept_set_and_distribution(vocab, temperature, top_k, top_p, min_p):
    rng = np.random.default_rng(vocab + top_k)
    row = (rng.normal(size=vocab) * 2.5).astype(np.float32)
    row[rng.integers(0, vocab, 5)] = float("-inf")
    kept = sampler_plain.kept_set(row, temperature, top_k, top_p, min_p)
    ids = {i for i, _ in kept}
    mass = sum(float(w) for _, w in kept)
    draws = 8192
    u = (np.arange(draws) + 0.5) / draws
    got = _sample(np.tile(row, (draws, 1)), temperature, top_k, top_p, min_p, u)
    assert set(got.tolist()) <= ids, f"drawn outside the kept set: {sorted(set(got.tolist()) - ids)[:5]}"
    # an evenly spaced u must hit every kept token whose share is well above the spacing
    for token, weight in kept:
        if float(weight) / mass > 4.0 / draws:
            assert token in set(got.tolist()), f"kept token {token} never drawn"
    # and the shares follow the weights
    for token, weight in kept[:5]:
        share = float(np.mean(got == token))
        assert abs(share - float(weight) / mass) < 2.0 / draws + 1e-3
    # the walk is in id order: a larger u never selects a smaller id
    assert np.all(np.diff(got) >= 0)


def test_penalties_match_the_plain_formula():
    from vipera_rs_amd.sampling import BatchSampler, RowRequest, SamplingParams
    rng = np.random.default_rng(11)
    vocab = 400
    base = rng.normal(size=(3, vocab)).astype(np.float32)
    recent = [[5, 5, 9, 200, 5], [], [399, 0, 0]]
    params = [
        SamplingParams(temperature=0.0, repetition_penalty=1.3, presence_penalty=0.5, frequency_penalty=0.25,
                       logit_bias=((9, 4.0), (7, -100.0))),
        SamplingParams(temperature=0.0, repetition_penalty=1.5),
        SamplingParams(temperature=0.0, repetition_penalty=0.8, logit_bias=((1, 2.0), (1, 50.0))),
    ]
    for r in range(3):  # make the penalized tokens matter
        for token in recent[r]:
            base[r, token] = abs(base[r, token]) + 3.0
    logits = torch.tensor(base, device="cuda:0").contiguous()
    sampler = BatchSampler("cuda:0")
    got = sampler.sample(logits, [RowRequest(p, slot, 0, rec, 1) for slot, (p, rec) in enumerate(zip(params, recent))])
    after = logits.cpu().numpy()
    for r in range(3):
        want = sampler_plain.penalize(base[r], recent[r], params[r].repetition_penalty, params[r].presence_penalty,
                                      params[r].frequency_penalty, params[r].logit_bias)
        np.testing.assert_allclose(after[r], want, rtol=1e-6, atol=1e-6)
        assert got[r] == sampler_plain.greedy(want)


def test_the_stream_of_a_request_does_not_depend_on_its_company():
    """A request's generator lives in its state slot on the device and the kernel advances it; the host's
    generator (the reference's xorshift64* behind SplitMix64) is only the oracle here."""
    from vipera_rs_amd.sampling import BatchSampler, RowRequest, SamplingParams, seeded_state
    rng = np.random.default_rng(5)
    vocab = 300
    rows = rng.normal(size=(4, vocab)).astype(np.float32) * 2
    params = [SamplingParams(temperature=0.8, seed=s) for s in (1, 2, 3, 4)]
    # the oracle: the plain sampler's kept set walked in id order with the plain generator's uniforms
    want = []
    for r in range(4):
        gen = sampler_plain.Rng(params[r].seed)
        kept = sorted(sampler_plain.kept_set(rows[r], 0.8, params[r].top_k, params[r].top_p, params[r].min_p))
        tokens = []
        for _ in range(6):
            u = gen.next_f64()
            ids = [i for i, _ in kept]
            shares = np.cumsum([float(w) for _, w in kept])
            tokens.append((u, ids, shares / shares[-1]))
        want.append(tokens)
    sampler = BatchSampler("cuda:0", slots=8)
    alone = []
    for r in range(4):
        alone.append([sampler.sample(torch.tensor(rows[r:r + 1], device="cuda:0"),
                                     [RowRequest(params[r], 5, k, (), seeded_state(params[r].seed) if k == 0 else None)])[0]
                      for k in range(6)])
        assert sampler.slot_table[5, 1].item() == 5                                   # the position is recorded
        assert sampler.slot_table[5, 0].item() % 2 ** 64 == seeded_state(params[r].seed, 6)   # the host's, wound on
    for r in range(4):     # each draw falls where the plain generator's uniform points, up to rounding of the shares
        for token, (u, ids, cumulative) in zip(alone[r], want[r]):
            at = ids.index(token)
            lo = cumulative[at - 1] if at else 0.0
            assert lo - 1e-4 <= u <= cumulative[at] + 1e-4, (r, token, u)
    together = [[] for _ in range(4)]
    slot_of = {0: 3, 1: 0, 2: 7, 3: 1}
    for k in range(6):
        order = [2, 0, 3, 1] if k % 2 else [1, 3, 0, 2]
        out = sampler.sample(torch.tensor(rows[order], device="cuda:0").contiguous(),
                             [RowRequest(params[r], slot_of[r], k, (), seeded_state(params[r].seed) if k == 0 else None)
                              for r in order])
        for r, token in zip(order, out):
            together[r].append(token)
    assert together == alone
    # a request that comes back into another slot after 3 draws goes on where it was
    again = [sampler.sample(torch.tensor(rows[2:3], device="cuda:0"),
                            [RowRequest(params[2], 6, k, (), seeded_state(params[2].seed, 3) if k == 3 else None)])[0]
             for k in range(3, 6)]
    assert again == alone[2][3:]
    # a greedy row leaves its generator alone
    before = sampler.slot_table[6, 0].item()
    sampler.sample(torch.tensor(rows[0:1], device="cuda:0"), [RowRequest(SamplingParams(), 6, 9)])
    assert sampler.slot_table[6, 0].item() == before and sampler.slot_table[6, 1].item() == 9
