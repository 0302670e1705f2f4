"""Generation through the entry point: greedy tokens against the plain implementation, sampling that
does not depend on a request's company, preemption when pages run out, cancelling, long decoding."""
import numpy as np
import pytest
import torch

from helpers import CONFIG_A, CONFIG_B, CONFIG_D, assert_tokens_follow_plain, make_folder, random_tokens
from plain import qwen2_plain

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {
        "A": make_folder(tmp_path_factory.mktemp("engine_A"), CONFIG_A, 0, torch.float32),
        "B": make_folder(tmp_path_factory.mktemp("engine_B"), CONFIG_B, 1, torch.float32),
        "D": make_folder(tmp_path_factory.mktemp("engine_D"), CONFIG_D, 3, torch.float32),
        "B16": make_folder(tmp_path_factory.mktemp("engine_B16"), CONFIG_B, 1, torch.bfloat16),
    }


def _engine(folder, **kw):
    from vipera_rs_amd import Engine
    kw.setdefault("dtype", "float32")
    return Engine(folder, **kw)


def test_greedy_generation_equals_the_plain_implementation(folders):
    # workload of the first tiny configuration: prompts of 5, 8 and 13 tokens, 8 new tokens each
    cfg, weights = qwen2_plain.load_folder(folders["A"])
    prompts = [random_tokens(CONFIG_A["vocab_size"], n, 40 + n) for n in (5, 8, 13)]
    want = [qwen2_plain.greedy_generate(cfg, weights, p, 8) for p in prompts]
    engine = _engine(folders["A"], block_size=16, num_blocks=12, max_num_seqs=4)
    got = engine.generate(prompts, max_new_tokens=8)
    assert [g.tokens for g in got] == want
    assert all(g.finish == "length" and g.prompt_tokens == len(p) for g, p in zip(got, prompts))
    assert engine.runner.cache.check() == "" and engine.runner.cache.live_requests() == 0
    # the last sampled token is never fed back (engine.rs:1509-1514)
    assert [g.processed_tokens for g in got] == [len(p) + 7 for p in prompts]


@pytest.mark.parametrize("name", ["B", "D"])
def test_greedy_generation_with_an_untied_head(folders, name):
    # tied embeddings make a random model repeat its last token; the second configuration does not (D: the same
    # with windowed layers, prompts and continuations past the window of 21)
    cfg, weights = qwen2_plain.load_folder(folders[name])
    prompts = [random_tokens(CONFIG_B["vocab_size"], n, 60 + n) for n in (3, 30, 11)]
    want = [qwen2_plain.greedy_generate(cfg, weights, p, 24) for p in prompts]
    assert all(len(set(w)) > 3 for w in want), "the continuation should not be one repeated token"
    engine = _engine(folders[name], block_size=8, num_blocks=24, max_num_seqs=3, chunk_size=7)
    assert [g.tokens for g in engine.generate(prompts, max_new_tokens=24)] == want


@pytest.mark.parametrize("graphs", [False, True])
def test_bfloat16_generation_follows_the_plain_implementation(folders, graphs):
    """bfloat16 through the entry point, prompts in portions beside decoding requests: every generated token is
    the plain implementation's best one (on the same bfloat16 weights) wherever that one's lead is clear."""
    cfg, weights = qwen2_plain.load_folder(folders["B16"])
    prompts = [random_tokens(CONFIG_B["vocab_size"], n, 80 + n) for n in (2, 37, 9, 21, 50)]
    engine = _engine(folders["B16"], dtype="bfloat16", block_size=8, num_blocks=48, max_num_seqs=3, chunk_size=6,
                     max_num_batched_tokens=11, use_graphs=graphs)
    got = engine.generate(prompts, max_new_tokens=40)
    checked = 0
    for p, g in zip(prompts, got):
        assert len(g.tokens) == 40 and len(set(g.tokens)) > 1
        logits = qwen2_plain.forward(cfg, weights, p + g.tokens[:-1])
        # a lead of 4 % of the largest logit; bfloat16 logits have been seen 0.7 % off
        checked += assert_tokens_follow_plain(logits, len(p), g.tokens, 1e-2, f"prompt of {len(p)}")
    assert checked > 75, "too few tokens had a clear lead to say anything"
    assert engine.runner.cache.check() == "" and engine.runner.cache.live_requests() == 0


def test_end_of_sequence_stops_and_is_kept_in_the_tokens(folders):
    cfg, weights = qwen2_plain.load_folder(folders["A"])
    prompt = random_tokens(CONFIG_A["vocab_size"], 9, 3)
    free_run = qwen2_plain.greedy_generate(cfg, weights, prompt, 6)
    eos = free_run[3]
    stop_at = free_run.index(eos)
    engine = _engine(folders["A"], num_blocks=8)
    streamed = []
    rid = engine.add_request(prompt, 6, eos_token_ids=[eos], on_token=streamed.append)
    done = None
    while done is None:
        for g in engine.step().finished:
            done = g
    assert done.request == rid and done.finish == "stop"
    assert done.tokens == free_run[:stop_at + 1]
    assert streamed == free_run[:stop_at]  # the end token is not streamed (engine.rs:571-575)


def test_seeded_sampling_is_independent_of_company_and_arrival(folders):
    # workload of the second tiny configuration: prompts of 1, 7, 19 and 33 tokens in portions of 6
    # mixed with decoding, temperature 0.8 with a seed, 10 new tokens each
    from vipera_rs_amd import SamplingParams
    prompts = [random_tokens(CONFIG_B["vocab_size"], n, 70 + n) for n in (1, 7, 19, 33)]
    params = [SamplingParams(temperature=0.8, seed=11 + k) for k in range(4)]
    alone = []
    for p, s in zip(prompts, params):
        engine = _engine(folders["B"], block_size=8, num_blocks=16, max_num_seqs=1, chunk_size=6)
        alone.append(engine.generate([p], 10, s)[0].tokens)
    engine = _engine(folders["B"], block_size=8, num_blocks=40, max_num_seqs=4, chunk_size=6,
                     max_num_batched_tokens=16)
    together = [g.tokens for g in engine.generate(prompts, 10, params)]
    assert together == alone
    engine = _engine(folders["B"], block_size=8, num_blocks=40, max_num_seqs=4, chunk_size=6,
                     max_num_batched_tokens=16)
    order = [3, 1, 0, 2]
    shuffled = engine.generate([prompts[i] for i in order], 10, [params[i] for i in order])
    assert [g.tokens for g in shuffled] == [alone[i] for i in order]
    assert all(len(t) == 10 for t in alone)


def test_preemption_when_pages_run_out_keeps_every_request_right(folders):
    prompts = [random_tokens(CONFIG_A["vocab_size"], n, 90 + n) for n in (30, 28, 25, 31)]
    solo = []
    for p in prompts:
        solo.append(_engine(folders["A"], num_blocks=8, max_num_seqs=1).generate([p], 40)[0].tokens)
    # 4 requests growing to ~70 tokens need ~20 pages of 16; 10 pages force preemption
    engine = _engine(folders["A"], block_size=16, num_blocks=10, max_num_seqs=4, chunk_size=16)
    got = engine.generate(prompts, 40)
    assert [g.tokens for g in got] == solo
    assert engine.stats()["preemptions"] > 0 and sum(g.preemptions for g in got) == engine.stats()["preemptions"]
    assert engine.runner.cache.check() == "" and engine.runner.cache.live_requests() == 0
    assert engine.runner.cache.free_blocks(0) == 10


@pytest.mark.parametrize("pipelined", [False, True])
def test_a_preempted_request_goes_on_with_its_own_stream_of_draws(folders, pipelined):
    """A request's generator lives in its state slot; a preempted request loses the slot and, when it comes back,
    its new slot is seeded with the generator wound forward by the draws it has made."""
    from vipera_rs_amd import SamplingParams
    prompts = [random_tokens(CONFIG_B["vocab_size"], n, 90 + n) for n in (30, 28, 25, 31)]
    params = [SamplingParams(temperature=0.9, seed=21 + k) for k in range(4)]
    solo = [_engine(folders["B"], block_size=16, num_blocks=8, max_num_seqs=1).generate([p], 40, s)[0].tokens
            for p, s in zip(prompts, params)]
    engine = _engine(folders["B"], block_size=16, num_blocks=10, max_num_seqs=4, chunk_size=16, pipelined=pipelined)
    got = engine.generate(prompts, 40, params)
    assert engine.stats()["preemptions"] > 0
    assert [g.tokens for g in got] == solo
    assert engine.runner.cache.check() == "" and engine.runner.cache.live_requests() == 0


def test_a_request_that_can_never_fit_is_refused_at_admission(folders):
    from vipera_rs_amd.errors import InfeasibleError, InvalidArgumentError
    engine = _engine(folders["A"], block_size=16, num_blocks=2, max_num_seqs=2)
    with pytest.raises(InfeasibleError):
        engine.add_request(random_tokens(256, 40, 1), 8)
    with pytest.raises(InvalidArgumentError):
        engine.add_request([], 8)
    with pytest.raises(InvalidArgumentError):
        engine.add_request([1, 2], 0)
    with pytest.raises(InvalidArgumentError):
        engine.add_request([1, 256], 4)
    assert not engine.has_work()


def test_cancel_frees_pages_at_a_step_boundary(folders):
    engine = _engine(folders["A"], block_size=16, num_blocks=8, max_num_seqs=2)
    a = engine.add_request(random_tokens(256, 20, 1), 30)
    b = engine.add_request(random_tokens(256, 20, 2), 5)
    engine.step()
    assert engine.runner.cache.used_blocks(0) == 4
    cancelled = engine.cancel(a)
    assert cancelled.finish == "cancelled" and engine.runner.cache.used_blocks(0) == 2
    done = []
    while engine.has_work():
        done += engine.step().finished
    assert [g.request for g in done] == [b] and engine.runner.cache.used_blocks(0) == 0
    assert engine.runner.cache.check() == ""


def test_long_decoding_follows_the_plain_implementation(folders):
    cfg, weights = qwen2_plain.load_folder(folders["B"])
    prompt = random_tokens(CONFIG_B["vocab_size"], 6, 5)
    engine = _engine(folders["B"], block_size=8, num_blocks=40, max_num_seqs=1)
    tokens = engine.generate([prompt], 240)[0].tokens
    assert len(tokens) == 240
    logits = qwen2_plain.forward(cfg, weights, prompt + tokens[:-1])
    assert assert_tokens_follow_plain(logits, len(prompt), tokens, 2.5e-5, "long decoding") > 200


def test_captured_decode_steps_equal_eager_steps_on_every_replay(folders):
    """A graph is replayed many times, with eager prompt steps and synchronizations in between; each
    replay must give the logits of the same step run eagerly."""
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    vocab = CONFIG_B["vocab_size"]
    runners = [ModelRunner.from_folder(folders["B"], dtype="bfloat16", block_size=8, num_blocks=64, num_slots=8)
               for _ in range(2)]
    from vipera_rs_amd.engine.graphs import DecodeGraphs
    runners[1].graphs = DecodeGraphs(runners[1], 512)
    prompts = {r: random_tokens(vocab, n, 300 + r) for r, n in enumerate((9, 30, 17))}
    lengths = {r: 0 for r in prompts}
    feed = {r: random_tokens(vocab, 40, 400 + r) for r in prompts}
    for runner in runners:
        for r, tokens in prompts.items():
            runner.cache.reserve(r, 0, len(tokens))
        runner.step([StepEntry(r, 0, tokens, [len(tokens) - 1]) for r, tokens in prompts.items()])
    for r, tokens in prompts.items():
        lengths[r] = len(tokens)
    for step in range(24):
        live = [r for r in prompts if not (step % 7 == 3 and r == 1)]  # one request sits out now and then
        outs = []
        for runner in runners:
            entries = []
            for r in live:
                runner.cache.reserve(r, lengths[r], lengths[r] + 1)
                entries.append(StepEntry(r, lengths[r], [feed[r][step]], [0]))
            outs.append(runner.step(entries).float().cpu())
            torch.cuda.synchronize()
        assert torch.equal(outs[0], outs[1]), f"replay {step} differs from the eager step"
        for r in live:
            lengths[r] += 1
        if step == 10:  # a new request arrives: an eager prompt step between replays, then a wider graph
            prompts[3] = random_tokens(vocab, 21, 303)
            feed[3] = random_tokens(vocab, 40, 403)
            for runner in runners:
                runner.cache.reserve(3, 0, 21)
                runner.step([StepEntry(3, 0, prompts[3], [20])])
            lengths[3] = 21
    assert runners[1].graphs.replays == 24 and len(runners[1].graphs.graphs) >= 2


def test_a_captured_step_of_many_requests_rotates_by_the_positions_of_each_replay(folders):
    """From 128 tokens on a step computes its sines and cosines once into a table: a captured step has to
    compute it in every replay, from that replay's positions."""
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.graphs import DecodeGraphs
    from vipera_rs_amd.engine.runner import ModelRunner
    vocab, live = CONFIG_B["vocab_size"], 130
    runners = [ModelRunner.from_folder(folders["B16"], dtype="bfloat16", block_size=8, num_blocks=live * 4,
                                       num_slots=live) for _ in range(2)]
    runners[1].graphs = DecodeGraphs(runners[1], 256)
    prompts = {r: random_tokens(vocab, 3 + r % 11, 900 + r) for r in range(live)}
    for runner in runners:
        for r, tokens in prompts.items():
            runner.cache.reserve(r, 0, len(tokens))
        runner.step([StepEntry(r, 0, tokens, []) for r, tokens in prompts.items()])
    lengths = {r: len(tokens) for r, tokens in prompts.items()}
    for step in range(6):
        outs = []
        for runner in runners:
            entries = []
            for r in prompts:
                runner.cache.reserve(r, lengths[r], lengths[r] + 1)
                entries.append(StepEntry(r, lengths[r], [(7 * r + 13 * step) % vocab], [0]))
            outs.append(runner.step(entries).float().cpu())
            torch.cuda.synchronize()
        assert torch.equal(outs[0], outs[1]), f"replay {step} differs from the eager step"
        for r in prompts:
            lengths[r] += 1
    assert runners[1].graphs.replays == 6 and [key[:2] for key in runners[1].graphs.graphs] == [(160, 256)]


def test_captured_steps_of_every_fill_class_follow_the_eager_steps(tmp_path):
    """64 requests under one context bucket of 1,024: first one long among short ones (a small share of the bucket
    is filled: the graph's attention cuts the positions into shorter chunks), then all long (the full class).  Each
    class has a graph of its own where the launches differ, and every replay follows the eager step, whose chunks
    are chosen from the true lengths."""
    from helpers import rel_err
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.graphs import DecodeGraphs
    from vipera_rs_amd.engine.runner import ModelRunner
    config = dict(CONFIG_A, max_position_embeddings=1024)
    folder = make_folder(tmp_path, config, 8, torch.bfloat16)
    vocab, live = config["vocab_size"], 64
    runners = [ModelRunner.from_folder(folder, dtype="bfloat16", block_size=16, num_blocks=live * 60, num_slots=live)
               for _ in range(2)]
    runners[1].graphs = DecodeGraphs(runners[1], 1024)
    lengths = {r: 0 for r in range(live)}

    def extend(request, count):
        tokens = random_tokens(vocab, count, 1000 * request + lengths[request])
        for runner in runners:
            runner.cache.reserve(request, lengths[request], lengths[request] + count)
            runner.step([StepEntry(request, lengths[request], tokens, [])])
        lengths[request] += count

    def decode(step):
        outs = []
        for runner in runners:
            entries = []
            for r in range(live):
                runner.cache.reserve(r, lengths[r], lengths[r] + 1)
                entries.append(StepEntry(r, lengths[r], [(5 * r + 11 * step) % vocab], [0]))
            outs.append(runner.step(entries).float().cpu().numpy())
            torch.cuda.synchronize()
        for r in range(live):
            lengths[r] += 1
            assert rel_err(outs[1][r], outs[0][r]) < 1e-2, f"step {step}, request {r} of {lengths[r]} positions"

    extend(0, 900)
    for r in range(1, live):
        extend(r, 20 + r % 41)
    for step in range(3):
        decode(step)
    assert {key[2] for key in runners[1].graphs.graphs} == {2}
    for r in range(1, live):
        extend(r, 800 - lengths[r] + r % 7)
    for step in range(3, 6):
        decode(step)
    graphs = runners[1].graphs
    assert graphs.replays == 6 and set(graphs.graphs) == {(64, 1024, 2), (64, 1024, 0)}
    assert graphs.graphs[(64, 1024, 2)].plans != graphs.graphs[(64, 1024, 0)].plans
    assert graphs.graphs[(64, 1024, 2)].plans[0][:2] == (128, 8) and graphs.graphs[(64, 1024, 0)].plans[0][:2] == (256, 4)
    # a class whose launches are another's shares that one's graph
    made = graphs.capture_ahead(1, 256)
    assert made == 1 and len({id(g) for key, g in graphs.graphs.items() if key[:2] == (1, 256)}) == 1


# --- steps launched ahead of their tokens ---------------------------------------------------------------------------
def test_steps_launched_ahead_generate_the_same_tokens(folders):
    """``pipelined=True``: greedy and seeded generation, portions mixed with decoding, with and without
    captured steps, give exactly the tokens of the engine that runs one step after the other."""
    from vipera_rs_amd import SamplingParams
    prompts = [random_tokens(CONFIG_B["vocab_size"], n, 70 + n) for n in (1, 7, 19, 33)]
    for params in (None, [SamplingParams(temperature=0.8, seed=11 + k) for k in range(4)]):
        kw = dict(block_size=8, num_blocks=40, max_num_seqs=4, chunk_size=6, max_num_batched_tokens=16)
        want = [g.tokens for g in _engine(folders["B"], **kw).generate(prompts, 14, params)]
        for graphs in (True, False):
            engine = _engine(folders["B"], pipelined=True, use_graphs=graphs, **kw)
            got = engine.generate(prompts, 14, params)
            assert [g.tokens for g in got] == want, (params is None, graphs)
            assert all(g.finish == "length" for g in got)
            assert engine.runner.cache.check() == "" and engine.runner.cache.live_requests() == 0
            assert not engine.has_work()


def test_steps_launched_ahead_stop_at_end_of_sequence_and_drop_the_extra_token(folders):
    cfg, weights = qwen2_plain.load_folder(folders["A"])
    prompts = [random_tokens(CONFIG_A["vocab_size"], n, 3 + n) for n in (9, 12)]
    free = [qwen2_plain.greedy_generate(cfg, weights, p, 9) for p in prompts]
    eos = free[0][3]
    engine = _engine(folders["A"], num_blocks=12, pipelined=True)
    streamed = {0: [], 1: []}
    ids = [engine.add_request(p, 9, eos_token_ids=[eos], on_token=streamed[k].append) for k, p in enumerate(prompts)]
    done = {}
    while engine.has_work():
        for g in engine.step().finished:
            done[g.request] = g
    for k, rid in enumerate(ids):
        stop_at = free[k].index(eos) if eos in free[k] else None
        want = free[k] if stop_at is None else free[k][:stop_at + 1]
        assert done[rid].tokens == want and done[rid].finish == ("length" if stop_at is None else "stop")
        assert streamed[k] == (want if stop_at is None else want[:-1])
    assert engine.runner.cache.check() == "" and engine.runner.cache.live_requests() == 0


def test_steps_launched_ahead_survive_preemption_and_penalties(folders):
    from vipera_rs_amd import SamplingParams
    prompts = [random_tokens(CONFIG_A["vocab_size"], n, 90 + n) for n in (30, 28, 25, 31)]
    kw = dict(block_size=16, num_blocks=10, max_num_seqs=4, chunk_size=16)
    want = [g.tokens for g in _engine(folders["A"], **kw).generate(prompts, 40)]
    engine = _engine(folders["A"], pipelined=True, **kw)
    got = engine.generate(prompts, 40)
    assert [g.tokens for g in got] == want and engine.stats()["preemptions"] > 0
    assert engine.runner.cache.check() == "" and engine.runner.cache.free_blocks(0) == 10
    # a request with penalties makes the engine run its steps in turn while it lives; the others are unchanged
    params = [SamplingParams(temperature=0.7, seed=5, repetition_penalty=1.3), None, SamplingParams(temperature=0.9, seed=6)]
    kw = dict(block_size=16, num_blocks=24, max_num_seqs=3)
    want = [g.tokens for g in _engine(folders["A"], **kw).generate(prompts[:3], 12, params)]
    got = _engine(folders["A"], pipelined=True, **kw).generate(prompts[:3], 12, params)
    assert [g.tokens for g in got] == want


def test_cancel_while_a_step_is_on_its_way(folders):
    prompts = [random_tokens(CONFIG_A["vocab_size"], n, 20 + n) for n in (6, 7)]
    want = _engine(folders["A"], num_blocks=12).generate([prompts[1]], 10)[0].tokens
    engine = _engine(folders["A"], num_blocks=12, pipelined=True)
    first, second = [engine.add_request(p, 10) for p in prompts]
    for _ in range(4):
        engine.step()
    assert engine.cancel(first).finish == "cancelled"
    done = {}
    while engine.has_work():
        for g in engine.step().finished:
            done[g.request] = g
    assert list(done) == [second] and done[second].tokens == want
    assert engine.runner.cache.check() == "" and engine.runner.cache.live_requests() == 0


@pytest.mark.gpu
def test_decode_steps_captured_ahead_are_the_ones_that_generation_replays():
    """warm_up captures every batch and context bucket once; generation afterwards captures nothing more and gives
    the tokens of an engine that captures as it goes."""
    import tempfile
    from helpers import CONFIG_A, make_folder, random_tokens
    from vipera_rs_amd import Engine
    with tempfile.TemporaryDirectory() as tmp:
        make_folder(tmp, CONFIG_A, 5, torch.float32)
        prompts = [random_tokens(CONFIG_A["vocab_size"], n, 70 + n) for n in (9, 30, 17)]
        lazy = Engine(tmp, dtype="float32", max_num_seqs=4, max_model_len=300).generate(prompts, 24)
        engine = Engine(tmp, dtype="float32", max_num_seqs=4, max_model_len=300)
        made = engine.warm_up()
        assert made == 3 * 2                       # batch buckets 1, 2, 4 x context buckets 256, 512
        assert engine.warm_up() == 0               # nothing left to capture
        graphs = engine.runner.graphs
        before = set(graphs.graphs)
        ahead = engine.generate(prompts, 24)
        assert set(graphs.graphs) == before and graphs.replays > 0
        assert [g.tokens for g in ahead] == [g.tokens for g in lazy]


def test_captured_steps_without_any_wait_between_them_keep_their_own_metadata():
    """Thirty captured decode steps launched back to back, no result read in between (nothing wanted until the
    last): every step must run with its own positions and pages, although the host is far ahead of the GPU."""
    import tempfile
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    with tempfile.TemporaryDirectory() as tmp:
        make_folder(tmp, CONFIG_B, 3, torch.float32)
        tokens = random_tokens(CONFIG_B["vocab_size"], 50, 9)
        cfg, weights = qwen2_plain.load_folder(tmp)
        want = qwen2_plain.forward(cfg, weights, tokens)[-1]
        runner = ModelRunner.from_folder(tmp, dtype="float32", block_size=16, num_blocks=8, num_slots=2, use_graphs=True,
                                         max_context=128)
        runner.cache.reserve(1, 0, len(tokens))
        runner.step([StepEntry(1, 0, tokens[:20], [])])
        logits = None
        for p in range(20, len(tokens)):
            logits = runner.step([StepEntry(1, p, [tokens[p]], [0] if p == len(tokens) - 1 else [])])
        got = logits[0].double().cpu().numpy()
        assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()
        assert runner.graphs.replays == 30


# --- sampling through the engine, held to an oracle outside it ------------------------------------------------------
def _id_order_draw(logits, params, u):
    """The draw the engine makes, from the plain sampler's parts: the kept set of the reference's cuts
    (crates/vipera-sampler/src/lib.rs:172-232), walked in id order with ``target = u * mass`` until
    ``target < running`` (lib.rs:234-242 with the engine's order of walking).  Returns the token and how far,
    as a share of the mass, the target lies from the nearest edge between two kept tokens."""
    from plain import sampler_plain as S
    kept = sorted(S.kept_set(logits.astype(np.float32), params.temperature, params.top_k, params.top_p, params.min_p))
    mass = sum(float(w) for _, w in kept)
    target, running, token, edges = u * mass, 0.0, None, []
    for candidate, weight in kept:
        running += float(weight)
        edges.append(running)
        if token is None and target < running:
            token = candidate
    token = kept[-1][0] if token is None else token
    margin = min(abs(target - edge) for edge in edges[:-1]) / mass if len(edges) > 1 else 1.0
    return token, margin


@pytest.mark.parametrize("cuts", ["none", "default"])
@pytest.mark.parametrize("pipelined", [False, True])
def test_seeded_sampling_through_the_engine_equals_the_plain_sampler(folders, cuts, pipelined):
    """The second tiny configuration's workload (prompts of 1, 7, 19 and 33 tokens in portions of 6 beside decoding
    requests, temperature 0.8, a seed per request, 10 new tokens): every token the engine draws is the one that
    the plain forward pass, the plain sampler's kept set and the plain generator's next uniform select, token by
    token.  A draw that walked the ids the wrong way, used a uniform one draw late, or took another request's
    generator would pass every comparison of the engine with itself; it does not pass this one."""
    from plain import sampler_plain as S
    from vipera_rs_amd import SamplingParams
    cfg, weights = qwen2_plain.load_folder(folders["B"])
    prompts = [random_tokens(CONFIG_B["vocab_size"], n, 70 + n) for n in (1, 7, 19, 33)]
    extra = dict(top_k=0, top_p=1.0, min_p=0.0) if cuts == "none" else {}
    params = [SamplingParams(temperature=0.8, seed=11 + k, **extra) for k in range(4)]
    engine = _engine(folders["B"], block_size=8, num_blocks=40, max_num_seqs=4, chunk_size=6, max_num_batched_tokens=16,
                     pipelined=pipelined)
    got = engine.generate(prompts, 10, params)
    clear = 0
    for prompt, p, generation in zip(prompts, params, got):
        assert len(generation.tokens) == 10
        logits = qwen2_plain.forward(cfg, weights, prompt + generation.tokens[:-1])
        rng = S.Rng(p.seed)
        for k, token in enumerate(generation.tokens):
            want, margin = _id_order_draw(logits[len(prompt) - 1 + k], p, rng.next_f64())
            if margin > 1e-4:     # the target is clear of an edge between two tokens: no rounding can move the draw
                assert token == want, f"prompt of {len(prompt)}, seed {p.seed}: token {k} is {token}, the plain draw {want}"
                clear += 1
    assert clear >= 36, f"only {clear} of 40 draws were clear of an edge"


def test_the_generator_step_in_the_sampling_kernel():
    """xorshift64* worked by hand from state 1 (x ^= x >> 12; x ^= x << 25; x ^= x >> 27; output
    x * 0x2545F4914F6CDD1D): the next state is 2^25 + 1 and the output 5180492295206395165, so the uniform is
    (output >> 11) / 2^53 = 0.28083...; with masses 0.25 / 0.75 the id-order walk takes token 1, with 0.3 / 0.7
    token 0."""
    from vipera_rs_amd.ops import kernels
    dev = "cuda:0"
    u = (5180492295206395165 >> 11) / float(1 << 53)
    assert 0.25 < u < 0.3
    for masses, want in (((0.25, 0.75), 1), ((0.3, 0.7), 0)):
        logits = torch.tensor([[np.log(masses[0]), np.log(masses[1])]], dtype=torch.float32, device=dev)
        table = torch.zeros((3, 2), dtype=torch.int64, device=dev)
        out = torch.full((1,), -7, dtype=torch.int32, device=dev)
        one = lambda v, d: torch.tensor([v], dtype=d, device=dev)  # noqa: E731
        kernels.sample(logits, one(1.0, torch.float32), one(0, torch.int32), one(1.0, torch.float32),
                       one(0.0, torch.float32), None, out, slot=one(2, torch.int32), position=one(41, torch.int32),
                       reseed=one(1, torch.int32), seed_state=one(1, torch.int64), slot_table=table)
        assert out.item() == want
        assert table.cpu().tolist() == [[0, 0], [0, 0], [33554433, 41]]   # the slot keeps the state after the step
        # the next draw goes on from the slot's state: the host's generator from the same state agrees
        kernels.sample(logits, one(1.0, torch.float32), one(0, torch.int32), one(1.0, torch.float32),
                       one(0.0, torch.float32), None, out, slot=one(2, torch.int32), position=one(42, torch.int32),
                       reseed=one(0, torch.int32), seed_state=one(0, torch.int64), slot_table=table)
        from vipera_rs_amd.sampling import Rng
        host = Rng(0)
        host.state = 33554433
        u2 = host.next_f64()
        assert out.item() == (0 if u2 < masses[0] else 1) and table[2, 0].item() == host.state


def test_a_sampler_launch_that_fails_leaves_the_other_requests_streams_alone(folders):
    """The host books a request's draws only when the launch has gone through.  Here the launch raises once, in a
    step in which two requests draw while a third is still in its prompt: the two fail, the third finishes with
    exactly its solo tokens, and nothing is left held."""
    from vipera_rs_amd import SamplingParams
    from vipera_rs_amd.errors import InvalidArgumentError
    prompts = [random_tokens(CONFIG_B["vocab_size"], n, 70 + n) for n in (3, 5, 40)]
    params = [SamplingParams(temperature=0.8, seed=31 + k) for k in range(3)]
    solo = _engine(folders["B"], block_size=8, num_blocks=16, max_num_seqs=1, chunk_size=6).generate(
        [prompts[2]], 10, params[2])[0].tokens
    engine = _engine(folders["B"], block_size=8, num_blocks=40, max_num_seqs=3, chunk_size=6, max_num_batched_tokens=16)
    launch, calls = engine.sampler.launch, []

    def flaky(logits, rows):
        calls.append(len(rows))
        if len(calls) == 3:
            raise InvalidArgumentError("state slot 99 is outside the table")
        return launch(logits, rows)

    engine.sampler.launch = flaky
    got = engine.generate(prompts, 10, params)
    assert calls[2] == 2 and [g.finish for g in got] == ["error", "error", "length"]
    assert "state slot 99" in got[0].error
    assert got[2].tokens == solo
    assert engine.runner.cache.check() == "" and engine.runner.cache.live_requests() == 0


# --- preemption in the configurations and dtypes that had none ----------------------------------------------------
def test_preemption_with_windowed_layers(folders):
    """The fourth configuration (two cache groups: all positions, and a window of 21) with so few pages that
    requests are preempted and recomputed: every request's tokens are its solo run's."""
    prompts = [random_tokens(CONFIG_B["vocab_size"], n, 90 + n) for n in (30, 28, 25, 31)]
    solo = [_engine(folders["D"], block_size=8, num_blocks=12, max_num_seqs=1).generate([p], 40)[0].tokens
            for p in prompts]
    engine = _engine(folders["D"], block_size=8, num_blocks=18, max_num_seqs=4, chunk_size=16)
    got = engine.generate(prompts, 40)
    assert engine.stats()["preemptions"] > 0
    assert [g.tokens for g in got] == solo
    cache = engine.runner.cache
    assert cache.check() == "" and cache.live_requests() == 0 and len(cache.groups) == 2
    assert [cache.free_blocks(g) for g in range(2)] == [18, 18]


@pytest.mark.parametrize("pipelined", [False, True])
def test_bfloat16_generation_under_preemption_follows_the_plain_implementation(folders, pipelined):
    """bfloat16 with so few pages that requests are preempted: a recomputed request must go on as the plain
    implementation does wherever that one's best token leads clearly."""
    cfg, weights = qwen2_plain.load_folder(folders["B16"])
    prompts = [random_tokens(CONFIG_B["vocab_size"], n, 90 + n) for n in (30, 28, 25, 31)]
    engine = _engine(folders["B16"], dtype="bfloat16", block_size=16, num_blocks=10, max_num_seqs=4, chunk_size=16,
                     pipelined=pipelined)
    got = engine.generate(prompts, 40)
    assert engine.stats()["preemptions"] > 0
    checked = 0
    for p, g in zip(prompts, got):
        assert len(g.tokens) == 40
        logits = qwen2_plain.forward(cfg, weights, p + g.tokens[:-1])
        checked += assert_tokens_follow_plain(logits, len(p), g.tokens, 1e-2, f"prompt of {len(p)}")
    assert checked > 60, "too few tokens had a clear lead to say anything"
    assert engine.runner.cache.check() == "" and engine.runner.cache.live_requests() == 0


def test_a_request_on_pages_that_a_request_with_nan_activations_gave_back(folders):
    """A request whose pages hold NaN ends (here: is cancelled after its keys and values were overwritten with NaN, as
    overflowed activations leave them) and the next request takes exactly those pages; a portion of 5 leaves most of
    its last page unwritten.  Its tokens are those of a run on a fresh pool."""
    prompt = random_tokens(CONFIG_B["vocab_size"], 21, 77)
    for dtype, name in (("float32", "B"), ("bfloat16", "B16")):
        want = _engine(folders[name], dtype=dtype, block_size=16, num_blocks=6, max_num_seqs=1).generate([prompt], 12)[0].tokens
        engine = _engine(folders[name], dtype=dtype, block_size=16, num_blocks=6, max_num_seqs=1, chunk_size=5)
        first = engine.add_request(random_tokens(CONFIG_B["vocab_size"], 60, 78), 30)
        for _ in range(20):
            engine.step()
        assert engine.runner.cache.used_blocks(0) >= 4
        for paged in engine.runner.storage.kv:
            paged.k.fill_(float("nan"))
            paged.v.fill_(float("nan"))
        assert engine.cancel(first).finish == "cancelled" and engine.runner.cache.used_blocks(0) == 0
        got = engine.generate([prompt], 12)[0]
        assert got.finish == "length" and got.tokens == want, dtype
