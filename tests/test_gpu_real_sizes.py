"""The layer sizes of Qwen2.5-7B (hidden 3584, 28 heads over 4 key heads of width 128, feed-forward
18944, rotary base 1e6, q/k/v bias) with one layer and a small vocabulary, so that the plain
implementation stays affordable: whole prompts, portions and single tokens against it in 32-bit and
bfloat16, and a vocabulary of 152064 for the output projection and the samplers alone."""
import numpy as np
import pytest
import torch

from helpers import make_folder, random_tokens, rel_err
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu

CONFIG_7B_LAYER = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 1, "hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4,
    "intermediate_size": 18944, "vocab_size": 1000, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "max_position_embeddings": 32768, "hidden_act": "silu",
    "use_sliding_window": False, "sliding_window": 131072, "max_window_layers": 28,
}


@pytest.fixture(scope="module")
def real(tmp_path_factory):
    out = {}
    tokens = random_tokens(1000, 150, 21)
    for dtype, tdtype in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        folder = make_folder(tmp_path_factory.mktemp(f"real_{dtype}"), CONFIG_7B_LAYER, 3, tdtype)
        cfg, w = P.load_folder(folder)
        out[dtype] = (folder, P.forward(cfg, w, tokens))
    out["tokens"] = tokens
    return out


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-4), ("bfloat16", 3e-2)])
def test_real_layer_sizes_under_every_cut(real, dtype, tol):
    folder, want = real[dtype]
    _under_every_cut(folder, want, real["tokens"], dtype, tol)


# hidden 896 is no multiple of 256 and has heads of width 64; rows of 2,048 values lie 4 KB apart, which the
# weight-streaming kernels answer with a different first chunk for every workgroup
# hidden 5,120: weights of 26 to 71 M elements, whose products split K over workgroups from few tokens on (q/k/v from
# eleven, the output projection from seven, the down projection from the first)
OTHER_WIDTHS = {
    "0.5b": dict(hidden_size=896, num_attention_heads=14, num_key_value_heads=2, intermediate_size=4864),
    "3b": dict(hidden_size=2048, num_attention_heads=16, num_key_value_heads=2, intermediate_size=11008),
    "14b": dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, intermediate_size=13824),
    # the attention of the 72B shape (q/k/v of 10,240 x 8,192 splits K from four tokens on, in two ranges that the
    # rows alone would not ask for; the output projection from the first) with a small feed-forward
    "72b attention": dict(hidden_size=8192, num_attention_heads=64, num_key_value_heads=8, intermediate_size=1024),
}


@pytest.mark.parametrize("name", sorted(OTHER_WIDTHS))
def test_the_layer_sizes_of_other_models_under_every_cut(tmp_path, name):
    config = dict(CONFIG_7B_LAYER, **OTHER_WIDTHS[name])
    tokens = random_tokens(1000, 150, 31)
    folder = make_folder(tmp_path / name, config, 5, torch.bfloat16)
    cfg, w = P.load_folder(folder)
    _under_every_cut(folder, P.forward(cfg, w, tokens), tokens, "bfloat16", 3e-2)


def _under_every_cut(folder, want, tokens, dtype, tol):
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    runner = ModelRunner.from_folder(folder, dtype=dtype, block_size=16, num_blocks=40, num_slots=4)
    # whole
    runner.cache.reserve(0, 0, len(tokens))
    whole = runner.step([StepEntry(0, 0, tokens, list(range(len(tokens))))]).cpu().numpy()
    assert rel_err(whole, want) < tol
    runner.cache.release(0)
    # portions of changing size beside another request's portions (steps of 87, 20, 19, 47, 28 and 11 tokens), alone
    # (8, 12 and 4 tokens), then the last tokens one by one
    other = random_tokens(1000, 90, 22)
    rows, at, oat = [], 0, 0
    sizes = [70, 3, 2, 30, 11, 6, 8, 12, 4]
    assert len(tokens) - sum(sizes) >= 4
    for size in sizes + [1] * (len(tokens) - sum(sizes)):
        entries = []
        runner.cache.reserve(1, at, at + size)
        entries.append(StepEntry(1, at, tokens[at:at + size], list(range(size))))
        if oat < len(other):
            osize = min(17, len(other) - oat)
            runner.cache.reserve(2, oat, oat + osize)
            entries.append(StepEntry(2, oat, other[oat:oat + osize], []))
            oat += osize
        rows.append(runner.step(entries).cpu().numpy())
        at += size
    assert rel_err(np.concatenate(rows), want) < tol
    assert runner.cache.check() == ""


def test_two_layers_at_the_7b_widths_in_32_bit_over_a_thousand_positions(tmp_path):
    """Two layers of the benchmark's widths in true 32-bit arithmetic against the plain implementation's
    float64: a prompt of 1,024 tokens in one step, then portions, then single tokens, 1,100 positions in all."""
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    folder = make_folder(tmp_path / "two", dict(CONFIG_7B_LAYER, num_hidden_layers=2), 4, torch.float32)
    cfg, w = P.load_folder(folder)
    tokens = random_tokens(1000, 1100, 23)
    want = P.forward(cfg, w, tokens, attend=P.attention_by_head)
    del w
    runner = ModelRunner.from_folder(folder, dtype="float32", block_size=16, num_blocks=72, num_slots=2)
    rows, at = [], 0
    for size in [1024, 40, 2, 17] + [1] * 17:
        runner.cache.reserve(0, at, at + size)
        rows.append(runner.step([StepEntry(0, at, tokens[at:at + size], list(range(size)))]).cpu().numpy())
        at += size
    assert at == len(tokens)
    got = np.concatenate(rows)
    assert rel_err(got, want) < 1e-4
    worst = max(rel_err(got[t], want[t]) for t in range(len(tokens)))       # row by row as well
    assert worst < 1e-4, worst


CONFIG_BENCH_HEADS = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 256, "num_attention_heads": 28, "num_key_value_heads": 4, "head_dim": 128,
    "intermediate_size": 512, "vocab_size": 300, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "max_position_embeddings": 8192, "hidden_act": "silu",
}


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-4), ("bfloat16", 3e-2)])
def test_thousands_of_positions_at_the_benchmark_head_shape(tmp_path, dtype, tol):
    """28 query heads over 4 key heads of width 128 (a narrow model otherwise, so that the plain implementation
    stays affordable): a prompt of 2,030 tokens whole, then captured decode steps that cross 2,048 positions,
    where the context bucket of the captured step and the number of chunks of the decode attention change,
    beside a second, short request; then the same tokens as a second request in portions of 512."""
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    stored = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = make_folder(tmp_path / "heads", CONFIG_BENCH_HEADS, 9, stored)
    cfg, w = P.load_folder(folder)
    tokens = random_tokens(300, 2075, 41)
    short = random_tokens(300, 80, 42)
    want = P.forward(cfg, w, tokens, attend=P.attention_by_head)
    want_short = P.forward(cfg, w, short, attend=P.attention_by_head)
    runner = ModelRunner.from_folder(folder, dtype=dtype, block_size=16, num_blocks=2 * 131 + 8, num_slots=4,
                                     use_graphs=True, max_context=8192)
    head = 2030
    wanted = list(range(0, head, 97)) + list(range(head - 5, head))
    runner.cache.reserve(0, 0, head)
    runner.cache.reserve(1, 0, 35)
    logits = runner.step([StepEntry(0, 0, tokens[:head], wanted), StepEntry(1, 0, short[:35], [34])]).cpu().numpy()
    assert rel_err(logits[:-1], want[wanted]) < tol and rel_err(logits[-1], want_short[34]) < tol
    for k in range(len(tokens) - head):           # single tokens of both requests, replayed as captured steps
        at, at_short = head + k, 35 + k
        runner.cache.reserve(0, at, at + 1)
        runner.cache.reserve(1, at_short, at_short + 1)
        logits = runner.step([StepEntry(1, at_short, [short[at_short]], [0]), StepEntry(0, at, [tokens[at]], [0])])
        logits = logits.cpu().numpy()
        assert rel_err(logits[1], want[at]) < tol, f"position {at}"
        assert rel_err(logits[0], want_short[at_short]) < tol, f"position {at_short} of the short request"
    assert {key[1] for key in runner.graphs.graphs} == {2048, 4096}
    runner.cache.release(0)
    runner.cache.release(1)
    at = 0
    while at < len(tokens):                       # pages that the first request gave back
        size = min(512, len(tokens) - at)
        runner.cache.reserve(2, at, at + size)
        rows = list(range(0, size, 61)) + [size - 1]
        logits = runner.step([StepEntry(2, at, tokens[at:at + size], rows)]).cpu().numpy()
        assert rel_err(logits, want[[at + r for r in rows]]) < tol, f"portion from {at}"
        at += size
    assert runner.cache.check() == ""


CONFIG_SPLIT_NORMS = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 3, "hidden_size": 1024, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 128,
    "intermediate_size": 4096, "vocab_size": 300, "rope_theta": 10000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": True, "max_position_embeddings": 4096, "hidden_act": "silu",
}


def test_norms_split_between_the_products_around_them(tmp_path, monkeypatch):
    """Sizes at which a step of up to 16 tokens runs its norms inside the neighbouring products (the second norm of
    a layer between output and gate/up product, the first between the layer before's down product, with K split
    over workgroups or not, and the fused q/k/v product): single tokens, steps of 2 to 16 tokens and whole prompts
    against the plain implementation, and the norm kernel runs only where no product precedes it."""
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    from vipera_rs_amd.ops import kernels
    folder = make_folder(tmp_path / "split", CONFIG_SPLIT_NORMS, 5, torch.bfloat16)
    cfg, w = P.load_folder(folder)
    tokens = random_tokens(300, 170, 31)
    want = P.forward(cfg, w, tokens)
    runner = ModelRunner.from_folder(folder, dtype="bfloat16", block_size=16, num_blocks=24, num_slots=4)
    calls = []
    real_rmsnorm = kernels.rmsnorm
    monkeypatch.setattr(kernels, "rmsnorm", lambda *a, **k: (calls.append(1), real_rmsnorm(*a, **k))[1])
    rows, at = [], 0
    # up to 16 tokens both norms of a layer run inside products; from 17 to 64 the first one does (the kernel that
    # adds the K ranges of the q/k/v product divides by it), beyond that none
    for size in [70, 40, 17, 16, 9, 5, 4, 2] + [1] * 7:
        runner.cache.reserve(0, at, at + size)
        calls.clear()
        rows.append(runner.step([StepEntry(0, at, tokens[at:at + size], list(range(size)))]).cpu().numpy())
        assert len(calls) == (2 * 3 + 1 if size > 64 else 3 + 2 if size > 16 else 2), (size, len(calls))
        at += size
    assert at == len(tokens)
    assert rel_err(np.concatenate(rows), want) < 3e-2


def test_the_full_vocabulary_head_and_greedy_choice():
    """152064 columns are no power of two: the output projection and the argmax at that width."""
    from vipera_rs_amd.ops import kernels
    from vipera_rs_amd.ops.linear import linear
    g = torch.Generator().manual_seed(4)
    h = torch.randn(5, 3584, generator=g).to(torch.bfloat16).to("cuda:0")
    w = (torch.randn(152064, 3584, generator=g) * 0.02).to(torch.bfloat16).to("cuda:0")
    logits = torch.empty(5, 152064, dtype=torch.float32, device="cuda:0")
    linear(h, w, None, logits)
    want = h.double() @ w.double().T
    assert float((logits.double() - want).abs().max() / want.abs().max()) < 1e-5
    rows = logits.shape[0]
    out = torch.empty(rows, dtype=torch.int32, device="cuda:0")
    zeros = lambda d: torch.zeros(rows, dtype=d, device="cuda:0")  # noqa: E731
    kernels.sample(logits, zeros(torch.float32), zeros(torch.int32), torch.ones(rows, device="cuda:0"),
                   zeros(torch.float32), zeros(torch.float64), out)
    assert out.cpu().tolist() == want.argmax(dim=1).cpu().tolist()
