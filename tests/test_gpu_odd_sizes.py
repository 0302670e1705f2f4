"""Sizes that are no powers of two and fit no fast path: every kernel either takes them or the engine
falls back to the kernels that do; the logits still equal the plain implementation under portions
and single tokens.  Sizes outside what any kernel takes are refused with an error that says so."""
import numpy as np
import pytest
import torch

from helpers import make_folder, random_tokens, rel_err
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu


def _config(hidden, heads, kv_heads, head_dim, inter, vocab, layers=2, window=0, tied=False, theta=10000.0, eps=1e-6):
    cfg = {"architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": layers, "hidden_size": hidden,
           "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": head_dim,
           "intermediate_size": inter, "vocab_size": vocab, "rope_theta": theta, "rms_norm_eps": eps,
           "tie_word_embeddings": tied, "max_position_embeddings": 2048, "hidden_act": "silu"}
    if window:
        cfg.update(use_sliding_window=True, sliding_window=window, max_window_layers=1)
    return cfg


ODD = {
    "hd20_k100": _config(100, 5, 5, 20, 70, 77),                         # nothing divides by 8: 32-bit-FMA products, 32-bit attention
    "hd16_group20": _config(320, 20, 1, 16, 344, 513, tied=True),       # 20 query heads on one key head: two column blocks
    "hd80_group5": _config(160, 10, 2, 80, 408, 1001, window=37),       # head width 80 pads to 96; a window of 37
    "hd112": _config(224, 2, 2, 112, 120, 130, layers=1, theta=5e5, eps=1e-5),
    "hd256": _config(256, 3, 1, 256, 264, 259, layers=1),
    "hd48_inter_not_16": _config(96, 2, 1, 48, 200, 300, layers=3),     # feed-forward width 200: no interleaving
}


@pytest.mark.parametrize("name", list(ODD))
@pytest.mark.parametrize("dtype,tol", [("float32", 1e-4), ("bfloat16", 3e-2)])
@pytest.mark.parametrize("block_size", [16, 24])
def test_odd_sizes_against_plain(tmp_path, name, dtype, tol, block_size):
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    cfg = ODD[name]
    folder = make_folder(tmp_path / "m", cfg, 5, torch.float32 if dtype == "float32" else torch.bfloat16)
    c, w = P.load_folder(folder)
    tokens = random_tokens(cfg["vocab_size"], 83, 6)
    want = P.forward(c, w, tokens)
    runner = ModelRunner.from_folder(folder, dtype=dtype, block_size=block_size, num_blocks=16, num_slots=2)
    rows, at = [], 0
    for size in [50, 2, 9] + [1] * 22:
        runner.cache.reserve(0, at, at + size)
        rows.append(runner.step([StepEntry(0, at, tokens[at:at + size], list(range(size)))]).cpu().numpy())
        at += size
        runner.cache.advance(0, at)
    assert at == len(tokens)
    assert rel_err(np.concatenate(rows), want) < tol


def test_sizes_no_kernel_takes_are_refused_with_a_clear_error(tmp_path):
    """When the model is opened, not at its first step: from the runner's and the engine's constructors."""
    from vipera_rs_amd import Engine
    from vipera_rs_amd.engine.runner import ModelRunner
    from vipera_rs_amd.errors import UnsupportedError
    folder = make_folder(tmp_path / "wide", _config(64, 1, 1, 272, 32, 40, layers=1), 1)
    for dtype in ("float32", "bfloat16"):
        with pytest.raises(UnsupportedError, match="head_dim 272"):
            ModelRunner.from_folder(folder, dtype=dtype, block_size=16, num_blocks=4, num_slots=1)
        with pytest.raises(UnsupportedError, match="head_dim 272"):
            Engine(folder, dtype=dtype, block_size=16, num_blocks=4, max_num_seqs=1)
