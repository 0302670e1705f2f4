"""The plain C++ twins of the kernels against the plain Python implementation, on the CPU: two independent plain
implementations of the reference's formulas have to agree, part by part and for a whole tiny model."""
import math

import numpy as np
import pytest
import torch

from helpers import CONFIGS, make_folder, random_tokens, rel_err
from plain import qwen2_plain as P
from plain import sampler_plain as S
from plain_cpp import DT, call, library


def test_bfloat16_conversion_over_every_pattern():
    lib = library()
    patterns = torch.arange(65536, dtype=torch.int32).to(torch.int16)      # all bit patterns
    as_float = torch.empty(65536, dtype=torch.float32)
    lib.plain_bf16_to_float(patterns.data_ptr(), as_float.data_ptr(), 65536)
    want = patterns.view(torch.bfloat16).float()
    assert torch.equal(as_float.view(torch.int32), want.view(torch.int32))
    # and back: round to nearest even, compared with torch on values between the representable ones
    g = torch.Generator().manual_seed(0)
    values = torch.cat([torch.randn(100000, generator=g) * 10.0 ** torch.randint(-30, 30, (100000,), generator=g).float(),
                        torch.tensor([0.0, -0.0, 1.0, -2.0, float("inf"), -float("inf"), 1.00390625, 1.01171875,
                                      3.3895313892515355e38])])
    back = torch.empty(values.numel(), dtype=torch.int16)
    lib.plain_float_to_bf16(values.contiguous().data_ptr(), back.data_ptr(), values.numel())
    assert torch.equal(back, values.to(torch.bfloat16).view(torch.int16))


def test_rmsnorm_and_swiglu_twins():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 70, generator=g) * 3
    w = 1 + 0.1 * torch.randn(70, generator=g)
    out = torch.empty(5, 70)
    call("plain_rmsnorm", x, w, None, out, DT[torch.float32], 5, 70, 1e-5, None)
    assert rel_err(out.numpy(), P.rms_norm(x.double().numpy(), w.double().numpy(), 1e-5)) < 1e-6
    assert abs(float(torch.tensor([3.0, 4.0]).pow(2).mean().sqrt()) - math.sqrt(12.5)) < 1e-6
    vec = torch.empty(1, 2)                                             # the reference's own vector, model.rs:4465-4471
    call("plain_rmsnorm", torch.tensor([[3.0, 4.0]]), torch.ones(2), None, vec, 0, 1, 2, 0.0, None)
    assert np.allclose(vec.numpy(), np.array([[3.0, 4.0]]) / math.sqrt(12.5), rtol=1e-6)
    rows = torch.tensor([4, 1], dtype=torch.int32)
    picked = torch.empty(2, 70)
    call("plain_rmsnorm", x, w, rows, picked, 0, 2, 70, 1e-5, None)
    assert torch.equal(picked, out[[4, 1]])
    gate_up = torch.randn(3, 2 * 48, generator=g) * 4
    got = torch.empty(3, 48)
    call("plain_swiglu", gate_up, got, 0, 3, 48, 0, None)
    want = gate_up[:, 48:].double().numpy() * P.silu(gate_up[:, :48].double().numpy())
    assert rel_err(got.numpy(), want) < 1e-6
    inter = torch.empty(3, 48)                                           # groups of 16 gate columns, then their up columns
    fused = torch.stack([gate_up[:, :48].reshape(3, 3, 16), gate_up[:, 48:].reshape(3, 3, 16)], dim=2).reshape(3, 96)
    call("plain_swiglu", fused.contiguous(), inter, 0, 3, 48, 1, None)
    assert torch.equal(inter, got)


@pytest.mark.parametrize("hd,rotary_dim", [(16, 16), (48, 48), (64, 32)])
def test_rotation_and_cache_write_twin(hd, rotary_dim):
    heads, kv_heads, bs, base = 3, 2, 8, 50000.0
    positions = [0, 1, 9, 300]
    g = torch.Generator().manual_seed(hd)
    qkv = torch.randn(4, (heads + 2 * kv_heads) * hd, generator=g)
    half = rotary_dim // 2
    index = np.arange(half, dtype=np.float32)
    inv = torch.from_numpy((np.float32(1.0) / np.power(np.float32(base), np.float32(2.0) * index / np.float32(rotary_dim),
                                                       dtype=np.float32)).astype(np.float32))
    table = torch.full((1, 40), -1, dtype=torch.int32)
    for page, p in enumerate(positions):
        table[0, p // bs] = page + 1 if table[0, p // bs] < 0 else table[0, p // bs]
    k_cache, v_cache = torch.zeros(6, kv_heads, bs, hd), torch.zeros(6, kv_heads, hd, bs)
    rotated = qkv.clone()
    pos_t, entry = torch.tensor(positions, dtype=torch.int32), torch.zeros(4, dtype=torch.int32)
    call("plain_rope_kvwrite", rotated, 0, pos_t, inv, None, rotary_dim, k_cache, v_cache, entry, table, 40, bs, 4,
         heads, kv_heads, hd, None)
    for t, pos in enumerate(positions):
        x = qkv[t].numpy().reshape(heads + 2 * kv_heads, hd)
        want = x.copy()
        want[:heads + kv_heads, :rotary_dim] = P.rope_neox(x[:heads + kv_heads, :rotary_dim].copy(), pos, base)
        assert np.max(np.abs(rotated[t].numpy().reshape(-1, hd) - want)) < 2e-6 * max(1.0, float(np.abs(want).max()))
        page, slot = int(table[0, pos // bs]), pos % bs
        assert torch.equal(k_cache[page, :, slot, :], rotated[t, heads * hd:(heads + kv_heads) * hd].view(kv_heads, hd))
        assert torch.equal(v_cache[page, :, :, slot], qkv[t, (heads + kv_heads) * hd:].view(kv_heads, hd))
    # the table of sines and cosines gives the same rotation
    angles = torch.empty(4, half, 2)
    call("plain_rope_angles", pos_t, inv, half, 4, angles, None)
    again = qkv.clone()
    call("plain_rope_kvwrite", again, 0, pos_t, inv, angles, rotary_dim, None, None, entry, None, 0, 0, 4, heads, kv_heads,
         hd, None)
    assert torch.equal(again, rotated)
    # the reference's own vectors (model.rs:4653-4661): base 1 rotates every pair by `pos` radians; position 0 is the identity
    row = torch.tensor([[1.0, 0.0, 2.0, 5.0, 0.0, 0.0]])                # one q head, one k head, one v head of width 2
    call("plain_rope_kvwrite", row, 0, torch.tensor([1], dtype=torch.int32), torch.ones(1), None, 2, None, None,
         torch.zeros(1, dtype=torch.int32), None, 0, 0, 1, 1, 1, 2, None)
    assert np.allclose(row[0, :2].numpy(), [math.cos(1.0), math.sin(1.0)], atol=1e-7)
    still = torch.tensor([[2.0, 5.0, 2.0, 5.0, 0.0, 0.0]])
    call("plain_rope_kvwrite", still, 0, torch.tensor([0], dtype=torch.int32), torch.ones(1), None, 2, None, None,
         torch.zeros(1, dtype=torch.int32), None, 0, 0, 1, 1, 1, 2, None)
    assert still[0].tolist() == [2.0, 5.0, 2.0, 5.0, 0.0, 0.0]


def test_products_twins():
    g = torch.Generator().manual_seed(2)
    a, w, bias = torch.randn(7, 40, generator=g), torch.randn(13, 40, generator=g), torch.randn(13, generator=g)
    out = torch.empty(7, 13)
    call("plain_gemm_generic", a, 0, w, 0, bias, out, 0, 7, 13, 40, 40, 13, 0, None)
    want = P.linear(a.double().numpy(), w.double().numpy(), bias.double().numpy())
    assert rel_err(out.numpy(), want) < 1e-6
    base = torch.randn(7, 13, generator=g)
    acc = base.clone()
    call("plain_gemm_generic", a, 0, w, 0, None, acc, 0, 7, 13, 40, 40, 13, 1, None)
    assert rel_err(acc.numpy(), base.double().numpy() + a.double().numpy() @ w.double().numpy().T) < 1e-6
    ab, wb = a.to(torch.bfloat16), w.to(torch.bfloat16)
    low = torch.empty(7, 13, dtype=torch.bfloat16)
    call("plain_gemm_bf16", ab, wb, bias, low, 1, 7, 13, 40, 40, 13, 0, 64, 0, None, 0, None)
    assert rel_err(low.float().numpy(), P.linear(ab.double().numpy(), wb.double().numpy(), bias.double().numpy())) < 5e-3
    gate, up = torch.randn(32, 40, generator=g).to(torch.bfloat16), torch.randn(32, 40, generator=g).to(torch.bfloat16)
    fused = torch.stack([gate.view(2, 16, 40), up.view(2, 16, 40)], dim=1).reshape(64, 40).contiguous()
    gated = torch.empty(7, 32, dtype=torch.bfloat16)
    call("plain_gemm_bf16_gated", ab, fused, gated, 7, 64, 40, 40, 32, 1, None)
    gd, ud = ab.double().numpy() @ gate.double().numpy().T, ab.double().numpy() @ up.double().numpy().T
    assert rel_err(gated.float().numpy(), ud * P.silu(gd)) < 5e-3


@pytest.mark.parametrize("window", [0, 5])
def test_attention_twins_over_a_shuffled_table(window):
    heads, kv_heads, hd, bs, T = 4, 2, 16, 4, 19
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(T, n, hd, generator=g) for n in (heads, kv_heads, kv_heads))
    want = P.attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), window=window).reshape(T, heads * hd)
    pages = list(torch.randperm(8, generator=g)[: (T + bs - 1) // bs].tolist())
    table = torch.tensor([pages + [-1] * 3], dtype=torch.int32)
    k_cache, v_cache = torch.zeros(8, kv_heads, bs, hd), torch.zeros(8, kv_heads, hd, bs)
    for p in range(T):
        k_cache[pages[p // bs], :, p % bs, :] = k[p]
        v_cache[pages[p // bs], :, :, p % bs] = v[p]
    qkv = torch.cat([q.reshape(T, -1), torch.zeros(T, 2 * kv_heads * hd)], dim=1).contiguous()
    out = torch.empty(T, heads * hd)
    positions, entry = torch.arange(T, dtype=torch.int32), torch.zeros(T, dtype=torch.int32)
    call("plain_attn_generic", qkv, qkv.shape[1], k_cache, v_cache, out, 0, positions, entry, table, table.shape[1], bs, T,
         heads, kv_heads, hd, 1 / math.sqrt(hd), window, None, None)
    assert rel_err(out.numpy(), want) < 1e-6
    # the bfloat16 entry points: a prompt cut into a portion of 13 tokens and six single tokens
    qb, kb, vb = qkv.to(torch.bfloat16), k_cache.to(torch.bfloat16), v_cache.to(torch.bfloat16)
    low = torch.zeros(T, heads * hd, dtype=torch.bfloat16)
    call("plain_attn_bf16_prefill", qb, qb.shape[1], kb, vb, low, torch.tensor([0, 0], dtype=torch.int32), 1,
         torch.tensor([0, 13], dtype=torch.int32), torch.tensor([0], dtype=torch.int32), table, table.shape[1], bs, heads,
         kv_heads, hd, 1 / math.sqrt(hd), window, 0, None, 0, 0, 0, None)
    for t in range(13, T):   # each later token as an entry of its own that reads the same pages
        call("plain_attn_bf16_decode", qb, qb.shape[1], kb, vb, low, None, torch.tensor([0], dtype=torch.int32), 1,
             torch.tensor([t, t + 1], dtype=torch.int32), torch.tensor([t], dtype=torch.int32), table, table.shape[1], bs,
             heads, kv_heads, hd, 1 / math.sqrt(hd), window, 128, 1, 0, 0, None)
    exact = P.attention(qb[:, :heads * hd].double().numpy().reshape(T, heads, hd),
                        kb.double().numpy()[pages].transpose(0, 2, 1, 3).reshape(-1, kv_heads, hd)[:T],
                        vb.double().numpy()[pages].transpose(0, 3, 1, 2).reshape(-1, kv_heads, hd)[:T], window=window)
    assert rel_err(low.float().numpy(), exact.reshape(T, heads * hd)) < 5e-3


def test_sampling_twins():
    g = torch.Generator().manual_seed(4)
    logits = torch.randn(6, 50, generator=g) * 3
    logits[2, 7] = float("inf")
    logits[3, :] = float("nan")
    logits[4, 10] = logits[4, 20] = logits[4].max() + 1           # a tie: the lowest id wins
    temperature = torch.tensor([0.0, 0.8, 0.0, 0.0, 0.0, 1.3])
    top_k = torch.tensor([0, 5, 0, 0, 0, 0], dtype=torch.int32)
    top_p = torch.tensor([1.0, 0.9, 1.0, 1.0, 1.0, 0.7])
    min_p = torch.tensor([0.0, 0.05, 0.0, 0.0, 0.0, 0.0])
    uniform = torch.tensor([0.3, 0.41, 0.5, 0.5, 0.5, 0.77], dtype=torch.float64)
    out = torch.empty(6, dtype=torch.int32)
    call("plain_sample", logits, 6, 50, temperature, top_k, top_p, min_p, uniform, out, None, None, 0,
         None, None, None, None, None, 0, None)
    assert out[0] == S.greedy(logits[0].numpy()) and out[2] == S.greedy(logits[2].numpy())
    assert out[3] == -1 and out[4] == 10
    for row in (1, 5):   # the kept set is the reference's; the draw walks it in id order
        kept = S.kept_set(logits[row].numpy(), float(temperature[row]), int(top_k[row]), float(top_p[row]), float(min_p[row]))
        by_id = sorted(kept)
        assert int(out[row]) == S.draw(by_id, float(uniform[row]))
    pen = logits[:2].clone()
    rows, tokens, counts = (torch.tensor(x, dtype=torch.int32) for x in ([0, 0, 1], [3, 9, 3], [2, 1, 4]))
    call("plain_penalize", pen, 50, rows, tokens, counts, torch.tensor([1.3, 1.0]), torch.tensor([0.2, 0.0]),
         torch.tensor([0.1, 0.5]), 3, None)
    assert np.allclose(pen[0].numpy(), S.penalize(logits[0].numpy(), [3, 3, 9], 1.3, 0.2, 0.1), rtol=1e-6, atol=1e-6)
    assert np.allclose(pen[1].numpy(), S.penalize(logits[1].numpy(), [3, 3, 3, 3], 1.0, 0.0, 0.5), rtol=1e-6, atol=1e-6)
    call("plain_logit_bias", pen, 50, torch.tensor([1], dtype=torch.int32), torch.tensor([4], dtype=torch.int32),
         torch.tensor([2.5]), 1, None)
    assert abs(float(pen[1, 4]) - float(S.penalize(logits[1].numpy(), [3] * 4, 1.0, 0.0, 0.5, [(4, 2.5)])[4])) < 1e-6


def _forward_through_twins(cfg, w, tokens, bs=8):
    """A whole sequence through the C++ twins in 32-bit, as one step of one request over a paged cache."""
    cfg = P.normalize_config(cfg)
    T, H = len(tokens), cfg["hidden_size"]
    heads, kv_heads, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    f = lambda name: torch.from_numpy(w[name]).float().contiguous()  # noqa: E731
    x = torch.empty(T, H)
    call("plain_embed_gather", f("model.embed_tokens.weight"), 0, torch.tensor(tokens, dtype=torch.int32), None, None, x, T,
         H, cfg["vocab_size"], None)
    index = np.arange(hd // 2, dtype=np.float32)
    inv = torch.from_numpy((np.float32(1.0) / np.power(np.float32(cfg["rope_theta"]), np.float32(2.0) * index / np.float32(hd),
                                                       dtype=np.float32)).astype(np.float32))
    pages = (T + bs - 1) // bs
    table = torch.arange(pages - 1, -1, -1, dtype=torch.int32).view(1, pages).contiguous()   # pages in reverse order
    positions, entry = torch.arange(T, dtype=torch.int32), torch.zeros(T, dtype=torch.int32)
    width = (heads + 2 * kv_heads) * hd
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = torch.empty(T, H)
        call("plain_rmsnorm", x, f(p + "input_layernorm.weight"), None, h, 0, T, H, float(cfg["rms_norm_eps"]), None)
        w_qkv = torch.cat([f(p + f"self_attn.{n}_proj.weight") for n in "qkv"]).contiguous()
        b_qkv = torch.cat([f(p + f"self_attn.{n}_proj.bias") for n in "qkv"]).contiguous()
        qkv = torch.empty(T, width)
        call("plain_gemm_generic", h, 0, w_qkv, 0, b_qkv, qkv, 0, T, width, H, H, width, 0, None)
        k_cache, v_cache = torch.zeros(pages, kv_heads, bs, hd), torch.zeros(pages, kv_heads, hd, bs)
        call("plain_rope_kvwrite", qkv, 0, positions, inv, None, hd, k_cache, v_cache, entry, table, pages, bs, T, heads,
             kv_heads, hd, None)
        attn = torch.empty(T, heads * hd)
        call("plain_attn_generic", qkv, width, k_cache, v_cache, attn, 0, positions, entry, table, pages, bs, T, heads,
             kv_heads, hd, 1.0 / math.sqrt(hd), P.layer_window(cfg, i), None, None)
        call("plain_gemm_generic", attn, 0, f(p + "self_attn.o_proj.weight"), 0, None, x, 0, T, H, heads * hd, heads * hd, H, 1,
             None)
        call("plain_rmsnorm", x, f(p + "post_attention_layernorm.weight"), None, h, 0, T, H, float(cfg["rms_norm_eps"]), None)
        inter = cfg["intermediate_size"]
        w_gu = torch.cat([f(p + "mlp.gate_proj.weight"), f(p + "mlp.up_proj.weight")]).contiguous()
        gate_up, act = torch.empty(T, 2 * inter), torch.empty(T, inter)
        call("plain_gemm_generic", h, 0, w_gu, 0, None, gate_up, 0, T, 2 * inter, H, H, 2 * inter, 0, None)
        call("plain_swiglu", gate_up, act, 0, T, inter, 0, None)
        call("plain_gemm_generic", act, 0, f(p + "mlp.down_proj.weight"), 0, None, x, 0, T, H, inter, inter, H, 1, None)
    h = torch.empty(T, H)
    call("plain_rmsnorm", x, f("model.norm.weight"), None, h, 0, T, H, float(cfg["rms_norm_eps"]), None)
    head = f("lm_head.weight") if "lm_head.weight" in w else f("model.embed_tokens.weight")
    logits = torch.empty(T, cfg["vocab_size"])
    call("plain_gemm_generic", h, 0, head, 0, None, logits, 0, T, cfg["vocab_size"], H, H, cfg["vocab_size"], 0, None)
    return logits.numpy()


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_a_whole_model_through_the_twins_equals_the_python_plain_implementation(name, tmp_path):
    config, seed = CONFIGS[name]
    cfg, w = P.load_folder(make_folder(tmp_path / name, config, seed))
    tokens = random_tokens(cfg["vocab_size"], 37, seed + 10)
    want = P.forward(cfg, w, tokens)
    got = _forward_through_twins(cfg, w, tokens)
    assert rel_err(got, want) < 2e-5
    assert np.array_equal(np.argmax(got, axis=-1), np.argmax(want, axis=-1))
