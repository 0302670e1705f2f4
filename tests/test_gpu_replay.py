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
            if err > TOL[dtype]:
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
