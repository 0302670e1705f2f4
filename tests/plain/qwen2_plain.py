"""A plain, slow implementation of the Qwen2 dense decoder: whole sequences, no cache, one function
per part, NumPy only.  It shares no code with the engine; it reads a model folder with the
``safetensors`` library and ``json``.

Every function follows a formula of the reference, cited as ``file:line`` under
``crates/vipera-backend-cpu/src/``.  Arithmetic is float64 unless ``dtype`` says otherwise, so the
engine's 32-bit path is compared with something more exact than itself.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, Optional

import numpy as np


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """model.rs:4282-4288: mean of squares, ``inv = 1/sqrt(mean + eps)``, ``(x * inv) * w`` per row."""
    mean = np.mean(x * x, axis=-1, keepdims=True)
    inverse = 1.0 / np.sqrt(mean + eps)
    return x * inverse * weight


def rope_neox(x: np.ndarray, position: int, base: float, rotary_dim: Optional[int] = None) -> np.ndarray:
    """model.rs:4192-4251: for each head, pairs ``(i, i + half)``; ``inv_i = 1 / base^(2i/hd)``;
    ``(s, c) = sincos(pos * inv_i)``; ``x[i] = lo*c - hi*s``; ``x[i+half] = lo*s + hi*c``.

    ``x`` is ``[heads, head_dim]`` of one token.  The inverse frequency is rounded to float32 as the
    reference computes it in ``f32``.
    """
    heads, head_dim = x.shape
    rd = head_dim if rotary_dim is None else rotary_dim
    half = rd // 2
    out = x.copy()
    for i in range(half):
        exponent = np.float32(2.0) * np.float32(i) / np.float32(rd)
        inv = np.float32(1.0) / np.power(np.float32(base), exponent, dtype=np.float32)
        # 32-bit runs round the product as the reference does; 64-bit runs keep it exact
        angle = float(np.float32(position) * inv) if x.dtype == np.float32 else float(position) * float(inv)
        s, c = math.sin(angle), math.cos(angle)
        lo, hi = x[:, i].copy(), x[:, i + half].copy()
        out[:, i] = lo * c - hi * s
        out[:, i + half] = lo * s + hi * c
    return out


def attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: Optional[float] = None,
              window: int = 0) -> np.ndarray:
    """model.rs:1811-1857 for every position of a whole sequence.

    ``q``: ``[T, heads, hd]``; ``k``, ``v``: ``[T, kv_heads, hd]``.  Head ``h`` uses key head
    ``h // (heads // kv_heads)`` (1815, 1826); ``score = dot(q, k) * scale`` with
    ``scale = 1/sqrt(hd)`` (1816, 1829-1838); position ``t`` sees positions ``0..t`` (a count, not a
    mask: 1086-1087), or the last ``window`` of them, itself included (2509); softmax with the
    maximum subtracted (1840-1848); ``out = sum_p (e_p / Z) * v_p`` (1849-1857).
    """
    T, heads, hd = q.shape
    kv_heads = k.shape[1]
    group = heads // kv_heads
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    out = np.zeros_like(q)
    for t in range(T):
        lo = max(0, t + 1 - window) if window > 0 else 0
        for h in range(heads):
            kvh = h // group
            scores = np.array([np.dot(q[t, h], k[p, kvh]) * scale for p in range(lo, t + 1)], dtype=q.dtype)
            best = scores.max()
            e = np.exp(scores - best)
            total = e.sum()
            acc = np.zeros(hd, dtype=q.dtype)
            for idx, p in enumerate(range(lo, t + 1)):
                acc += (e[idx] * (1.0 / total)) * v[p, kvh]
            out[t, h] = acc
    return out


def attention_by_head(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: Optional[float] = None,
                      window: int = 0) -> np.ndarray:
    """The same function as :func:`attention` with one matrix of scores per head instead of one dot product per
    pair of positions, for sequences of thousands of tokens; ``tests/test_plain.py`` holds it to ``attention``."""
    T, heads, hd = q.shape
    group = heads // k.shape[1]
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    position = np.arange(T)
    visible = position[None, :] <= position[:, None]
    if window > 0:
        visible &= position[None, :] > position[:, None] - window
    out = np.zeros_like(q)
    for h in range(heads):
        scores = np.where(visible, (q[:, h] @ k[:, h // group].T) * scale, -np.inf)
        e = np.exp(scores - scores.max(axis=1, keepdims=True))
        out[:, h] = (e / e.sum(axis=1, keepdims=True)) @ v[:, h // group]
    return out


def silu(z: np.ndarray) -> np.ndarray:
    """model.rs:4368-4370: ``z / (1 + exp(-z))``."""
    return z / (1.0 + np.exp(-z))


def linear(x: np.ndarray, weight: np.ndarray, bias: Optional[np.ndarray] = None) -> np.ndarray:
    """model.rs:623-629: ``y = W x`` (weights row-major ``[out, in]``, quant.rs:1-4), bias added after."""
    y = x @ weight.T
    if bias is not None:
        y = y + bias
    return y


def swiglu_mlp(h: np.ndarray, w_gate: np.ndarray, w_up: np.ndarray, w_down: np.ndarray) -> np.ndarray:
    """model.rs:672-680: ``down(up(h) * silu(gate(h)))``; no biases."""
    return linear(linear(h, w_up) * silu(linear(h, w_gate)), w_down)


def attention_block(h: np.ndarray, w: Dict[str, np.ndarray], prefix: str, cfg: dict, window: int,
                    attend=attention) -> np.ndarray:
    """model.rs:1005-1126: project with bias, rotate q and k (after the bias, 649-656), attend, project out."""
    T = h.shape[0]
    heads, kv_heads, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = linear(h, w[prefix + "q_proj.weight"], w.get(prefix + "q_proj.bias")).reshape(T, heads, hd)
    k = linear(h, w[prefix + "k_proj.weight"], w.get(prefix + "k_proj.bias")).reshape(T, kv_heads, hd)
    v = linear(h, w[prefix + "v_proj.weight"], w.get(prefix + "v_proj.bias")).reshape(T, kv_heads, hd)
    for t in range(T):
        q[t] = rope_neox(q[t], t, cfg["rope_theta"])
        k[t] = rope_neox(k[t], t, cfg["rope_theta"])
    a = attend(q, k, v, window=window).reshape(T, heads * hd)
    return linear(a, w[prefix + "o_proj.weight"])


def layer_window(cfg: dict, index: int) -> int:
    """Layers from ``max_window_layers`` on see the last ``sliding_window`` positions when
    ``use_sliding_window`` is set; the others see everything."""
    if not cfg.get("use_sliding_window") or not cfg.get("sliding_window"):
        return 0
    return int(cfg["sliding_window"]) if index >= int(cfg.get("max_window_layers") or 0) else 0


def normalize_config(cfg: dict) -> dict:
    cfg = dict(cfg)
    cfg.setdefault("num_key_value_heads", cfg["num_attention_heads"])        # model.rs:1352
    cfg.setdefault("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])  # model.rs:1367-1377
    cfg.setdefault("rms_norm_eps", 1e-6)                                      # model.rs:1397
    cfg.setdefault("rope_theta", 10000.0)                                     # model.rs:1398
    return cfg


def forward(cfg: dict, w: Dict[str, np.ndarray], tokens, dtype=np.float64, attend=attention) -> np.ndarray:
    """Logits ``[T, vocab]`` of a whole sequence (model.rs:956-1237): embedding (no scaling, 607-616),
    pre-norm blocks, final norm, output projection; the embedding table is the output matrix when the
    file has none (425)."""
    cfg = normalize_config(cfg)
    w = {name: value.astype(dtype) for name, value in w.items()}
    eps = cfg["rms_norm_eps"]
    x = w["model.embed_tokens.weight"][np.asarray(tokens)]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = rms_norm(x, w[p + "input_layernorm.weight"], eps)
        x = x + attention_block(h, w, p + "self_attn.", cfg, layer_window(cfg, i), attend)
        h = rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu_mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    h = rms_norm(x, w["model.norm.weight"], eps)
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    return linear(h, head)


def load_folder(folder: str):
    """``(config dict, weights as float64 arrays)`` of a model folder, read with the safetensors library."""
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as handle:
        cfg = json.load(handle)
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    return cfg, {name: t.double().numpy() for name, t in tensors.items()}


def greedy_generate(cfg: dict, w: Dict[str, np.ndarray], prompt, max_new: int, eos=()):
    """Greedy continuation by recomputing the whole sequence each time; ties go to the lowest id
    (crates/vipera-sampler/src/lib.rs:135-156; ``np.argmax`` returns the first maximum)."""
    tokens = list(prompt)
    out = []
    for _ in range(max_new):
        logits = forward(cfg, w, tokens)[-1]
        token = int(np.argmax(logits))
        out.append(token)
        tokens.append(token)
        if token in eos:
            break
    return out
