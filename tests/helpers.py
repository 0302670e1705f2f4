"""Tiny configurations and trace helpers shared by the tests."""
from __future__ import annotations

import os
import random
from typing import Dict, List, Sequence

import numpy as np
import torch

# Two tiny configurations that differ in every size and option (A and B), a third whose head width is not
# hidden / heads (C), and B with windowed layers (D).  B's `max_position_embeddings` of 256 is above every
# trace length the tests use on it (at most 246 positions).
CONFIG_A = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "intermediate_size": 128, "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True, "max_position_embeddings": 512, "hidden_act": "silu",
    "use_sliding_window": False, "sliding_window": 4096, "max_window_layers": 2,
}
CONFIG_B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
    "head_dim": 32, "intermediate_size": 200, "vocab_size": 300, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 256,
    "hidden_act": "silu", "use_sliding_window": False, "sliding_window": 21, "max_window_layers": 1,
}
CONFIG_C = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 1, "hidden_size": 80, "num_attention_heads": 6, "num_key_value_heads": 3,
    "head_dim": 48, "intermediate_size": 176, "vocab_size": 331, "rope_theta": 50000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "max_position_embeddings": 512,
    "hidden_act": "silu",
}
# Layers from `max_window_layers` on see the last `sliding_window` positions.  The reference has no such layer
# rule (its window is a run-time option over all layers, crates/vipera-core/src/window.rs:38-55) and pins only
# the visible range [p + 1 - w, p] (crates/vipera-backend-cpu/src/model.rs:2509): which layers are windowed is
# this engine's reading of the config keys, parity unpinned, and D is reported apart from A, B and C.
CONFIG_D = dict(CONFIG_B, use_sliding_window=True, sliding_window=21, max_window_layers=1,
                max_position_embeddings=1024)
CONFIGS = {"A": (CONFIG_A, 0), "B": (CONFIG_B, 1), "C": (CONFIG_C, 2), "D": (CONFIG_D, 3)}


def make_folder(path: str, config: dict, seed: int, dtype=torch.float32) -> str:
    """Write a model folder with the engine's random-weights mode."""
    import vipera_rs_amd  # noqa: F401
    from vipera_rs_amd.config import config_from_dict
    from vipera_rs_amd.models import declare_model
    from vipera_rs_amd.weights import write_random_model

    cfg = config_from_dict(config)
    return write_random_model(str(path), cfg, declare_model(cfg), seed, dtype)


def random_tokens(vocab: int, count: int, seed: int) -> List[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(count)]


def rel_err(got: np.ndarray, want: np.ndarray) -> float:
    """Largest difference relative to the largest wanted magnitude."""
    return float(np.max(np.abs(got.astype(np.float64) - want)) / max(np.max(np.abs(want)), 1e-30))


def assert_tokens_follow_plain(logits: np.ndarray, prompt_len: int, tokens: Sequence[int], tol: float,
                               label: str = "") -> int:
    """``tokens`` were generated greedily after a prompt of ``prompt_len``; ``logits`` are the plain
    implementation's over prompt + tokens[:-1].  Every token must be the plain implementation's best one
    wherever its lead over the runner-up is clear of ``tol``; returns how many were clear."""
    checked = 0
    for k, token in enumerate(tokens):
        row = logits[prompt_len - 1 + k]
        order = np.argsort(row)
        if row[order[-1]] - row[order[-2]] > 4 * tol * np.max(np.abs(row)):
            assert int(token) == int(order[-1]), f"{label}: generated token {k} is not the plain implementation's"
            checked += 1
    return checked


# --- traces ---------------------------------------------------------------------------------------
def trace_whole(requests: Dict[str, Sequence[int]]):
    """Each request alone and whole, all places wanted, one after the other."""
    steps = []
    for step, (name, tokens) in enumerate(requests.items()):
        steps.append({"step": step, "entries": [{"id": name, "tokens": list(tokens),
                                                  "want": list(range(len(tokens)))}], "end": [name]})
    return steps


def trace_decode_tail(name: str, tokens: Sequence[int], tail: int = 32):
    """Most of the request in one step, the last ``tail`` tokens one by one."""
    head = max(1, len(tokens) - tail)
    steps = [{"step": 0, "entries": [{"id": name, "tokens": list(tokens[:head]), "want": list(range(head))}],
              "end": []}]
    for k, position in enumerate(range(head, len(tokens))):
        steps.append({"step": k + 1, "entries": [{"id": name, "tokens": [tokens[position]], "want": [0]}],
                      "end": [name] if position == len(tokens) - 1 else []})
    if head == len(tokens):
        steps[0]["end"] = [name]
    return steps


def trace_chunks(name: str, tokens: Sequence[int], sizes: Sequence[int]):
    """Portions of changing size (cycled), every place wanted."""
    steps, at, k = [], 0, 0
    while at < len(tokens):
        size = min(sizes[k % len(sizes)], len(tokens) - at)
        last = at + size == len(tokens)
        steps.append({"step": k, "entries": [{"id": name, "tokens": list(tokens[at:at + size]),
                                               "want": list(range(size))}], "end": [name] if last else []})
        at += size
        k += 1
    return steps


def trace_mixed(requests: Dict[str, Sequence[int]], seed: int, max_live: int = 4, sizes=(7, 2, 13, 3, 1, 5, 1, 1)):
    """Up to ``max_live`` requests at a time; each step gives every live request a portion (often a
    single token), sometimes leaves one out; finished requests end and new ones start, so pages are
    used again."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live: Dict[str, int] = {}
    steps, step = [], 0
    while waiting or live:
        while waiting and len(live) < max_live:
            name, _ = waiting.pop(0)
            live[name] = 0
        entries, end = [], []
        names = list(live)
        for name in names:
            if len(names) > 1 and rng.random() < 0.2:
                continue  # left out of this step, goes on later
            tokens = requests[name]
            at = live[name]
            size = min(rng.choice(sizes), len(tokens) - at)
            entries.append({"id": name, "tokens": list(tokens[at:at + size]), "want": list(range(size))})
            live[name] = at + size
            if live[name] == len(tokens):
                end.append(name)
        if not entries:
            continue
        rng.shuffle(entries)
        steps.append({"step": step, "entries": entries, "end": end})
        for name in end:
            del live[name]
        step += 1
    return steps


def peak_tokens(steps) -> int:
    """Most tokens live requests hold at any time, each count rounded up to a multiple of 64."""
    held: Dict[str, int] = {}
    peak = 0
    for step in steps:
        for entry in step["entries"]:
            held[entry["id"]] = held.get(entry["id"], 0) + len(entry["tokens"])
        peak = max(peak, sum((n + 63) // 64 * 64 for n in held.values()))
        for name in step["end"]:
            held.pop(name, None)
    return peak


def replay(replayer, steps) -> Dict[str, Dict[int, np.ndarray]]:
    """Run ``steps`` through an engine Replayer; returns logits by request name and position."""
    out: Dict[str, Dict[int, np.ndarray]] = {}
    at: Dict[str, int] = {}
    for step in steps:
        logits = replayer.step(step["entries"], step["end"])
        row = 0
        for entry in step["entries"]:
            start = at.get(entry["id"], 0)
            for w in entry["want"]:
                out.setdefault(entry["id"], {})[start + w] = logits[row]
                row += 1
            at[entry["id"]] = start + len(entry["tokens"])
        for name in step["end"]:
            at.pop(name, None)
    return out
