"""The engine against the plain implementation under every way of cutting the work.

Each request's logits at every position must equal the plain implementation's (whole sequence, no
cache), whether the request runs alone and whole, mostly in one step with its last 32 tokens one
by one, in portions of changing size down to two tokens, or mixed with other requests with so few
pages that they are used again.  In 32-bit the bound is 1e-4 of the largest logit; bfloat16 is
held to 3e-2 and must pick the same best token wherever the plain implementation's lead is clear.
"""
import numpy as np
import pytest
import torch

from helpers import (CONFIGS, make_folder, peak_tokens, random_tokens, rel_err, replay, trace_chunks,
                     trace_decode_tail, trace_mixed, trace_whole)
from plain import qwen2_plain

pytestmark = pytest.mark.gpu

TOL = {"float32": 1e-4, "bfloat16": 3e-2}
LENGTHS = [70, 33, 5, 49, 91, 18, 64]


@pytest.fixture(scope="module", params=["A", "B", "C", "D"])
def case(request, tmp_path_factory):
    name = request.param
    config, seed = CONFIGS[name]
    out = {"name": name, "config": config}
    for dtype, tdtype in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        folder = make_folder(tmp_path_factory.mktemp(f"model_{name}_{dtype}"), config, seed, tdtype)
        cfg, weights = qwen2_plain.load_folder(folder)
        requests = {f"r{k}": random_tokens(config["vocab_size"], n, 100 * seed + k) for k, n in enumerate(LENGTHS)}
        want = {rid: qwen2_plain.forward(cfg, weights, toks) for rid, toks in requests.items()}
        out[dtype] = {"folder": folder, "requests": requests, "want": want}
    return out


def _replayer(folder, dtype, max_tokens, block_size):
    from vipera_rs_amd.engine.replay import Replayer
    return Replayer(folder, dtype, max_tokens, block_size)


def _compare(got, want, requests, dtype, label):
    worst = 0.0
    for rid, rows in got.items():
        assert sorted(rows) == list(range(len(requests[rid]))), f"{label}: request {rid} misses positions"
        for pos, row in rows.items():
            err = rel_err(row, want[rid][pos])
            if not err <= TOL[dtype]:   # NaN fails too
                raise AssertionError(f"{label}: request {rid} position {pos}: error {err:.3e} above {TOL[dtype]:.0e}")
            worst = max(worst, err)
            ref = want[rid][pos]
            order = np.argsort(ref)
            lead = ref[order[-1]] - ref[order[-2]]
            if lead > 4 * TOL[dtype] * np.max(np.abs(ref)):
                assert int(np.argmax(row)) == int(order[-1]), f"{label}: request {rid} position {pos}: best token differs"
    print(f"{label}: worst relative error {worst:.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("block_size", [16, 8])
def test_whole(case, dtype, block_size):
    data = case[dtype]
    steps = trace_whole(data["requests"])
    rep = _replayer(data["folder"], dtype, peak_tokens(steps), block_size)
    _compare(replay(rep, steps), data["want"], data["requests"], dtype, f"whole {case['name']} {dtype} bs{block_size}")
    assert rep.runner.cache.check() == "" and rep.runner.cache.live_requests() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_tail(case, dtype):
    data = case[dtype]
    for rid in ("r0", "r4", "r1"):
        steps = trace_decode_tail(rid, data["requests"][rid], 32)
        rep = _replayer(data["folder"], dtype, peak_tokens(steps), 16)
        _compare(replay(rep, steps), data["want"], data["requests"], dtype, f"tail {case['name']} {dtype} {rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(7, 2, 13, 3, 2), (2,), (16, 1, 15, 17, 2)])
def test_chunks(case, dtype, sizes):
    data = case[dtype]
    for rid in ("r0", "r4"):
        steps = trace_chunks(rid, data["requests"][rid], sizes)
        rep = _replayer(data["folder"], dtype, peak_tokens(steps), 16)
        _compare(replay(rep, steps), data["want"], data["requests"], dtype, f"chunks{sizes} {case['name']} {dtype} {rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("block_size", [16, 64])
def test_mixed_with_page_reuse(case, dtype, block_size):
    data = case[dtype]
    steps = trace_mixed(data["requests"], seed=7)
    peak = peak_tokens(steps)
    total = sum((len(t) + 63) // 64 * 64 for t in data["requests"].values())
    assert peak < total, "the trace must need fewer pages than all requests together, so pages are reused"
    rep = _replayer(data["folder"], dtype, peak, block_size)
    _compare(replay(rep, steps), data["want"], data["requests"], dtype, f"mixed {case['name']} {dtype} bs{block_size}")
    assert rep.runner.cache.check() == "" and rep.runner.cache.live_requests() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("block_size", [16, 64])
def test_mixed_on_a_pool_that_holds_nan(case, dtype, block_size):
    """Every page starts out holding NaN, as the pages do that a request with overflowed activations gave back.  A
    request reads only what it wrote itself: no slot past its last position, no page it does not hold (behind a
    window: given back and taken by another request) may reach its result, not even with a weight of zero."""
    data = case[dtype]
    steps = trace_mixed(data["requests"], seed=11)
    rep = _replayer(data["folder"], dtype, peak_tokens(steps), block_size)
    for paged in rep.runner.storage.kv:
        if paged is not None:
            paged.k.fill_(float("nan"))
            paged.v.fill_(float("nan"))
    _compare(replay(rep, steps), data["want"], data["requests"], dtype,
             f"mixed on NaN pages {case['name']} {dtype} bs{block_size}")



# --- what a folder stores and what a run keeps -------------------------------------------------------------------------
def _restored(tmp_path, source, convert):
    """A copy of the model folder ``source`` with every tensor passed through ``convert(spec, tensor)``."""
    import os
    from vipera_rs_amd.config import load_config
    from vipera_rs_amd.models import declare_model
    from vipera_rs_amd.weights import Checkpoint, write_safetensors
    config = load_config(source)
    specs = {s.name: s for s in declare_model(config)}
    ck = Checkpoint(source)
    tensors = [(name, convert(specs[name], ck.read(name).clone())) for name in ck.names()]
    ck.close()
    config.save(str(tmp_path))
    write_safetensors(os.path.join(str(tmp_path), "model.safetensors"), tensors)
    return str(tmp_path)


def test_a_folder_stored_in_32_bit_runs_in_bfloat16_as_the_same_weights_stored_in_bfloat16(tmp_path):
    """The loader converts a matrix to the run's dtype once, by rounding to nearest even, whatever the folder stores: a
    bfloat16 run of a 32-bit folder gives bit for bit the logits of a folder that holds the same matrices already
    rounded (its vectors, which both runs keep in 32-bit, left as they are), under a mixed trace.  It therefore runs
    on the matrix-core kernels; a 16-bit float folder likewise."""
    config, seed = CONFIGS["B"]
    source = make_folder(tmp_path / "f32", config, seed, torch.float32)
    rounded = _restored(tmp_path / "bf16", source,
                        lambda spec, t: t.to(torch.bfloat16) if spec.role == "matrix" else t)
    halves = _restored(tmp_path / "f16", source, lambda spec, t: t.to(torch.float16))
    halves_rounded = _restored(tmp_path / "f16_bf16", halves,
                               lambda spec, t: t.to(torch.bfloat16) if spec.role == "matrix" else t.float())
    requests = {f"r{k}": random_tokens(config["vocab_size"], n, 500 + k) for k, n in enumerate(LENGTHS)}
    steps = trace_mixed(requests, seed=3)
    runs = {}
    for name, folder in (("f32", source), ("bf16", rounded), ("f16", halves), ("f16_bf16", halves_rounded)):
        rep = _replayer(folder, "bfloat16", peak_tokens(steps), 16)
        weights = [layer.mixer.w_qkv for layer in rep.runner.model.layers] + [rep.runner.model.head.weight]
        assert all(w.dtype == torch.bfloat16 for w in weights), name
        runs[name] = replay(rep, steps)
    for a, b in (("f32", "bf16"), ("f16", "f16_bf16")):
        for rid, rows in runs[a].items():
            for pos, row in rows.items():
                assert np.array_equal(row, runs[b][rid][pos]), f"{a} against {b}: request {rid} position {pos}"
    cfg, weights = qwen2_plain.load_folder(rounded)
    want = {rid: qwen2_plain.forward(cfg, weights, toks) for rid, toks in requests.items()}
    _compare(runs["f32"], want, requests, "bfloat16", "32-bit folder run as bfloat16")


def test_32_bit_matrices_kept_on_request_in_a_bfloat16_run(tmp_path):
    """``keep_float32``: matrices stored in 32-bit stay so and their products go through the 32-bit kernel on
    bfloat16 activations; held to the plain implementation on the unrounded weights like any bfloat16 run."""
    from vipera_rs_amd.engine.replay import Replayer
    config, seed = CONFIGS["B"]
    source = make_folder(tmp_path / "f32", config, seed, torch.float32)
    requests = {f"r{k}": random_tokens(config["vocab_size"], n, 600 + k) for k, n in enumerate(LENGTHS[:4])}
    steps = trace_mixed(requests, seed=5)
    rep = Replayer(source, "bfloat16", peak_tokens(steps), 16, keep_float32=True)
    assert rep.runner.model.layers[0].mixer.w_qkv.dtype == torch.float32
    assert rep.runner.model.layers[0].ffn.w_down.dtype == torch.float32
    cfg, weights = qwen2_plain.load_folder(source)
    want = {rid: qwen2_plain.forward(cfg, weights, toks) for rid, toks in requests.items()}
    _compare(replay(rep, steps), want, requests, "bfloat16", "32-bit matrices kept in a bfloat16 run")


def test_a_tied_model_uses_an_output_matrix_that_its_folder_holds(tmp_path):
    """crates/vipera-backend-cpu/src/model.rs:424-425: the output matrix is the file's when it has one and the
    embedding table only otherwise, whatever the configuration says about tying."""
    import os
    from vipera_rs_amd.weights import Checkpoint, write_safetensors
    config, seed = CONFIGS["A"]          # tied embeddings
    folder = make_folder(tmp_path / "tied", config, seed, torch.float32)
    ck = Checkpoint(folder)
    tensors = {name: ck.read(name).clone() for name in ck.names()}
    ck.close()
    g = torch.Generator().manual_seed(1)
    tensors["lm_head.weight"] = torch.randn(tensors["model.embed_tokens.weight"].shape, generator=g) * 0.05
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors.items())
    cfg, weights = qwen2_plain.load_folder(folder)
    tokens = random_tokens(config["vocab_size"], 40, 9)
    want = {"r": qwen2_plain.forward(cfg, weights, tokens)}
    tied = dict(weights)
    del tied["lm_head.weight"]
    assert rel_err(qwen2_plain.forward(cfg, tied, tokens), want["r"]) > 0.1     # the two heads do differ
    for dtype in ("float32", "bfloat16"):
        rep = _replayer(folder, dtype, 64, 16)
        assert rep.runner.model.head.weight.data_ptr() != rep.runner.model.embedding.table.data_ptr()
        _compare(replay(rep, trace_chunks("r", tokens, (13, 2, 1))), want, {"r": tokens}, dtype, f"own head, {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cache_groups_with_pages_and_pools_of_their_own(tmp_path, dtype):
    """The fourth configuration has two cache groups (all positions; a window of 21).  Here each has its own page
    size and pool: pages of 16 for the first, pages of 8 and a pool that holds little more than the windows of four
    requests for the second.  A mixed trace through the runner equals the plain implementation."""
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    config, seed = CONFIGS["D"]
    folder = make_folder(tmp_path / "m", config, seed, torch.float32 if dtype == "float32" else torch.bfloat16)
    cfg, weights = qwen2_plain.load_folder(folder)
    requests = {f"r{k}": random_tokens(config["vocab_size"], n, 700 + k) for k, n in enumerate(LENGTHS)}
    want = {rid: qwen2_plain.forward(cfg, weights, toks) for rid, toks in requests.items()}
    steps = trace_mixed(requests, seed=13)
    runner = ModelRunner.from_folder(folder, dtype=dtype, block_size=[16, 8], num_blocks=[peak_tokens(steps) // 16, 24],
                                     num_slots=4)
    groups = runner.cache.groups
    assert [(g.block_size, g.window) for g in groups] == [(16, 0), (8, 21)] and groups[1].num_blocks == 24
    assert runner.storage.kv[0].k.shape[2] == 16 and runner.storage.kv[1].k.shape[2] == 8
    ids, at, got = {}, {}, {}
    for step in steps:
        entries = []
        for entry in step["entries"]:
            request = ids.setdefault(entry["id"], len(ids))
            start = at.get(request, 0)
            runner.cache.reserve(request, start, start + len(entry["tokens"]))
            entries.append(StepEntry(request, start, entry["tokens"], entry["want"]))
        logits = runner.step(entries).float().cpu().numpy()
        row = 0
        for entry, e in zip(step["entries"], entries):
            for w in entry["want"]:
                got.setdefault(entry["id"], {})[e.start + w] = logits[row]
                row += 1
            at[e.request] = e.start + len(e.tokens)
            runner.cache.advance(e.request, at[e.request])
        for name in step["end"]:
            runner.cache.release(ids[name])
    _compare(got, want, requests, dtype, f"two groups with their own pages, {dtype}")
    assert runner.cache.check() == "" and runner.cache.live_requests() == 0
