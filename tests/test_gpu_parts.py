"""The small kernels alone, each part of a layer alone, a run order that repeats a layer and shares a
cache, and a toy mixer with state of its own that is registered, built and stepped from this file
without any change to the package."""
import contextlib
import math
from dataclasses import dataclass
from typing import List

import numpy as np
import pytest
import torch

from helpers import CONFIG_A, CONFIG_B, assert_tokens_follow_plain, make_folder, random_tokens, rel_err
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _runtime(dtype):
    from vipera_rs_amd.runtime import Runtime
    return Runtime(DEV, dtype)


# --- kernels alone ------------------------------------------------------------------------------------
@pytest.mark.parametrize("table_dtype", [torch.float32, torch.bfloat16])
def test_embed_gather(table_dtype):
    from vipera_rs_amd.ops import kernels
    table = torch.randn(331, 100).to(table_dtype).to(DEV)
    tokens = torch.tensor([330, 0, 17, 17, 200], dtype=torch.int32, device=DEV)
    out = torch.empty(5, 100, device=DEV)
    kernels.embed_gather(table, tokens, out)
    assert torch.equal(out, table.float()[tokens.long()])


@pytest.mark.parametrize("width", [100, 3584, 8200, 97])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_kernel(width, out_dtype):
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(width)
    x = (torch.randn(6, width, generator=g) * 3).to(DEV)
    w = (1 + 0.1 * torch.randn(width, generator=g)).to(DEV)
    want = torch.tensor(P.rms_norm(x.cpu().double().numpy(), w.cpu().double().numpy(), 1e-5))
    out = torch.empty(6, width, dtype=out_dtype, device=DEV)
    kernels.rmsnorm(x, w, 1e-5, out)
    tol = 2e-6 if out_dtype == torch.float32 else 5e-3
    assert rel_err(out.float().cpu().numpy(), want.numpy()) < tol
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)       # rows picked by index
    picked = torch.empty(2, width, dtype=out_dtype, device=DEV)
    kernels.rmsnorm(x, w, 1e-5, picked, rows)
    assert torch.equal(picked, out[[4, 1]])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hd,rotary_dim", [(16, 16), (48, 48), (128, 128), (64, 32), (32, 0), (24, 12), (40, 20)])  # the last two: one element per lane
def test_rope_and_cache_write(dtype, hd, rotary_dim):
    from vipera_rs_amd.ops import kernels
    from vipera_rs_amd.parts.rotary import neox_inverse_frequencies
    heads, kv_heads, bs, base = 3, 2, 8, 50000.0
    positions = [0, 1, 7, 8, 300, 41]
    entry_of = [0, 0, 0, 0, 1, 1]
    table = torch.tensor([[5, 2, -1, -1, -1, -1], [9, 9, 9, 9, 9, 0] + [-1] * 0], dtype=torch.int32)
    table = torch.full((2, 40), -1, dtype=torch.int32)
    table[0, 0], table[0, 1] = 5, 2
    table[1, 300 // bs], table[1, 41 // bs] = 7, 3
    g = torch.Generator().manual_seed(hd)
    qkv = torch.randn(6, (heads + 2 * kv_heads) * hd, generator=g).to(dtype)
    k_cache = torch.zeros(10, kv_heads, bs, hd, dtype=dtype)
    v_cache = torch.zeros(10, kv_heads, hd, bs, dtype=dtype)
    inv = torch.from_numpy(neox_inverse_frequencies(rotary_dim, base)) if rotary_dim else None
    dev = lambda t: t.to(DEV) if t is not None else None  # noqa: E731
    qkv_d, k_d, v_d = dev(qkv.clone()), dev(k_cache), dev(v_cache)
    kernels.rope_kvwrite(qkv_d, dev(torch.tensor(positions, dtype=torch.int32)), dev(inv), rotary_dim, k_d, v_d,
                         dev(torch.tensor(entry_of, dtype=torch.int32)), dev(table), heads, kv_heads, hd)
    got = qkv_d.float().cpu().numpy()
    if rotary_dim:  # with the step's table of sines and cosines: the same bits in q, k and the cache
        pos_d = dev(torch.tensor(positions, dtype=torch.int32))
        angles = kernels.rope_angles(pos_d, dev(inv), len(positions))
        assert angles.shape == (len(positions), rotary_dim // 2, 2)
        qkv_t, k_t, v_t = dev(qkv.clone()), dev(k_cache), dev(v_cache)
        kernels.rope_kvwrite(qkv_t, pos_d, dev(inv), rotary_dim, k_t, v_t, dev(torch.tensor(entry_of, dtype=torch.int32)),
                             dev(table), heads, kv_heads, hd, angles)
        assert torch.equal(qkv_t, qkv_d) and torch.equal(k_t, k_d) and torch.equal(v_t, v_d)
    tol = 2e-6 if dtype == torch.float32 else 8e-3
    for t, pos in enumerate(positions):
        # 32-bit rows make the plain rotation round the angle to 32-bit as the reference does (model.rs:4199-4201);
        # with a 64-bit angle the two differ by the angle's rounding, about position * 6e-8
        row = qkv[t].float().numpy()
        for head in range(heads + kv_heads):
            x = row[head * hd:(head + 1) * hd].reshape(1, hd)
            want = x.copy()
            if rotary_dim:
                want[:, :rotary_dim] = P.rope_neox(x[:, :rotary_dim].copy(), pos, base)
            assert np.max(np.abs(got[t, head * hd:(head + 1) * hd] - want[0])) < tol * max(1.0, np.max(np.abs(want)))
        # v is untouched, and the cache holds the rotated k and the v at the token's page and slot
        v_in = qkv[t, (heads + kv_heads) * hd:].float().numpy()
        assert np.array_equal(got[t, (heads + kv_heads) * hd:], v_in)
        page, slot = int(table[entry_of[t], pos // bs]), pos % bs
        k_now = qkv_d[t, heads * hd:(heads + kv_heads) * hd].view(kv_heads, hd)
        assert torch.equal(k_d[page, :, slot, :], k_now)
        assert torch.equal(v_d[page, :, :, slot].float().cpu(), torch.tensor(v_in).view(kv_heads, hd))
    written = {(int(table[e, p // bs]), p % bs) for e, p in zip(entry_of, positions)}
    for page in range(10):
        for slot in range(bs):
            if (page, slot) not in written:
                assert float(k_d[page, :, slot, :].abs().max()) == 0.0 and float(v_d[page, :, :, slot].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hd,rotary_dim,bs", [(128, 128, 16), (64, 32, 8), (48, 48, 24), (32, 16, 16)])
def test_rope_of_a_large_step_writes_what_the_small_step_kernel_writes(dtype, hd, rotary_dim, bs):
    """With the step's table of sines the kernel takes eight tokens a workgroup and, where they are eight
    consecutive positions of one request from a multiple of eight on, writes the value pages eight slots at a time.
    Portions that start anywhere, a request without a page, a last group of fewer tokens: q, k and both caches
    hold bit for bit what the kernel of the small steps leaves (which the test above holds to the plain rotation)."""
    from vipera_rs_amd.ops import kernels
    from vipera_rs_amd.parts.rotary import neox_inverse_frequencies
    heads, kv_heads = 5, 2
    portions = [(8, 32), (5, 13), (0, 3), (64, 16), (16, 8), (3, 5)]      # (first position, tokens) per entry
    positions = [first + i for first, count in portions for i in range(count)]
    entry_of = [e for e, (_, count) in enumerate(portions) for _ in range(count)]
    width = 96 // bs + 1
    table = torch.full((len(portions), width), -1, dtype=torch.int32)
    order = torch.randperm(len(portions) * width, generator=torch.Generator().manual_seed(bs)).view(len(portions), width)
    for e, (first, count) in enumerate(portions):
        for block in range(first // bs, (first + count - 1) // bs + 1):
            table[e, block] = int(order[e, block])
    table[4, 16 // bs] = -1                                              # this request's tokens are not kept
    pages = len(portions) * width
    g = torch.Generator().manual_seed(hd + bs)
    qkv = torch.randn(len(positions), (heads + 2 * kv_heads) * hd, generator=g).to(dtype)
    inv = torch.from_numpy(neox_inverse_frequencies(rotary_dim, 10000.0)).to(DEV)
    pos_d = torch.tensor(positions, dtype=torch.int32, device=DEV)
    entry_d = torch.tensor(entry_of, dtype=torch.int32, device=DEV)
    results = []
    for angles in (None, kernels.rope_angles(pos_d, inv, len(positions))):
        q_d = qkv.clone().to(DEV)
        k_d = torch.zeros(pages, kv_heads, bs, hd, dtype=dtype, device=DEV)
        v_d = torch.zeros(pages, kv_heads, hd, bs, dtype=dtype, device=DEV)
        kernels.rope_kvwrite(q_d, pos_d, inv, rotary_dim, k_d, v_d, entry_d, table.to(DEV), heads, kv_heads, hd, angles)
        results.append((q_d, k_d, v_d))
    for small, large in zip(*results):
        assert torch.equal(small, large)
    assert float(results[1][2].abs().max()) > 0.0
    # without a cache (a layer that reads another layer's) only q and k are rotated
    q_only = qkv.clone().to(DEV)
    kernels.rope_kvwrite(q_only, pos_d, inv, rotary_dim, None, None, entry_d, None, heads, kv_heads, hd,
                         kernels.rope_angles(pos_d, inv, len(positions)))
    assert torch.equal(q_only, results[0][0])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_kernel(dtype):
    from vipera_rs_amd.ops import kernels
    gate_up = (torch.randn(7, 2 * 200) * 4).to(dtype).to(DEV)
    out = torch.empty(7, 200, dtype=dtype, device=DEV)
    kernels.swiglu(gate_up, out)
    g, u = gate_up[:, :200].double().cpu().numpy(), gate_up[:, 200:].double().cpu().numpy()
    assert rel_err(out.float().cpu().numpy(), u * P.silu(g)) < (2e-6 if dtype == torch.float32 else 5e-3)


def test_device_random_weights_follow_the_host_stream():
    from vipera_rs_amd.ops import kernels
    from vipera_rs_amd.weights import standard_normal, tensor_key
    key = tensor_key(5, "model.layers.3.mlp.down_proj.weight")
    out = torch.empty(10_001, device=DEV)
    kernels.fill_normal(out, key, 0.02, 1.0)
    want = 1.0 + 0.02 * standard_normal(key, 10_001)
    np.testing.assert_allclose(out.cpu().numpy(), want.astype(np.float32), rtol=2e-6, atol=1e-7)


# --- parts alone -------------------------------------------------------------------------------------------
def _random_part_tensors(cls, spec, prefix, seed, runtime):
    from vipera_rs_amd.weights import kept_dtype, random_tensor
    host, device = {}, {}
    for t in cls.declare(spec, prefix):
        if t.optional:    # a tensor a folder need not hold
            continue
        value = random_tensor(t, seed, torch.float32)
        kept = kept_dtype(t, torch.float32 if runtime.dtype == torch.float32 else torch.bfloat16, runtime.dtype)
        device[t.name] = value.to(kept).to(runtime.device)
        host[t.name] = device[t.name].double().cpu().numpy()
    return host, device


class _OneLayerCache:
    """A cache manager and storage for a single attention part, and batches over them."""

    def __init__(self, runtime, kv_spec, block_size=8, pages=40):
        from vipera_rs_amd.cache import CacheGroupSpec, CacheManager, CacheStorage
        from vipera_rs_amd.models.decoder import CacheNeed
        groups = [CacheGroupSpec(block_size, pages, kv_spec.window)]
        self.cache = CacheManager(groups, 4)
        self.storage = CacheStorage([CacheNeed(0, kv_spec, None)], groups, 4, runtime)
        self.runtime = runtime

    def batch(self, entries):
        from vipera_rs_amd.engine.batch import build_batch
        for e in entries:
            self.cache.reserve(e.request, e.start, e.start + len(e.tokens))
        return build_batch(entries, self.cache, 1000, self.runtime.device)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_mlp_embedding_and_head_parts(dtype):
    from vipera_rs_amd.config import PartSpec
    from vipera_rs_amd.parts import part_class
    rt = _runtime(dtype)
    tol = 1e-5 if dtype == "float32" else 1.5e-2
    x = torch.randn(9, 72).to(DEV)
    # norm
    spec = PartSpec("rmsnorm", {"width": 72, "eps": 1e-5, "name": "ln"})
    cls = part_class("norm", "rmsnorm")
    host, dev = _random_part_tensors(cls, spec, "p.", 1, rt)
    norm = cls(spec, "p.", rt)
    norm.load(dev)
    h = norm.forward(x)
    assert h.dtype == rt.dtype
    assert rel_err(h.float().cpu().numpy(), P.rms_norm(x.double().cpu().numpy(), host["p.ln.weight"], 1e-5)) < tol
    # feed-forward adds into the 32-bit residual
    spec = PartSpec("gated_mlp", {"hidden": 72, "intermediate": 200, "activation": "silu", "name": "mlp"})
    cls = part_class("ffn", "gated_mlp")
    host, dev = _random_part_tensors(cls, spec, "p.", 2, rt)
    mlp = cls(spec, "p.", rt)
    mlp.load(dev)
    residual = torch.randn(9, 72).to(DEV)
    before = residual.double().cpu().numpy()
    mlp.forward(h, None, residual)
    hh = h.double().cpu().numpy()
    want = before + P.swiglu_mlp(hh, host["p.mlp.gate_proj.weight"], host["p.mlp.up_proj.weight"], host["p.mlp.down_proj.weight"])
    assert rel_err(residual.cpu().numpy(), want) < tol
    # embedding and output projection, untied and tied
    espec = PartSpec("embedding", {"vocab": 331, "width": 72, "name": "emb"})
    ecls = part_class("embedding", "embedding")
    ehost, edev = _random_part_tensors(ecls, espec, "", 3, rt)
    emb = ecls(espec, "", rt)
    emb.load(edev)
    tokens = torch.tensor([0, 330, 5], dtype=torch.int32, device=DEV)
    got = emb.forward(tokens, 3)
    assert got.dtype == torch.float32 and np.array_equal(got.cpu().numpy(), ehost["emb.weight"][[0, 330, 5]].astype(np.float32))
    hcls = part_class("head", "lm_head")
    for tied in (None, "emb"):
        hspec = PartSpec("lm_head", {"vocab": 331, "width": 72, "name": "out", "tied_to": tied})
        hhost, hdev = _random_part_tensors(hcls, hspec, "", 4, rt)
        assert (len(hhost) == 0) == (tied is not None)
        head = hcls(hspec, "", rt)
        head.load({**edev, **hdev})
        logits = head.forward(h)
        weight = ehost["emb.weight"] if tied else hhost["out.weight"]
        assert logits.dtype == torch.float32 and rel_err(logits.cpu().numpy(), hh @ weight.T) < tol
        if tied:
            assert head.weight.data_ptr() == emb.table.data_ptr()      # the same buffer, no copy


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv_heads,hd,window,bias", [(4, 2, 16, 0, True), (3, 1, 32, 11, True), (6, 6, 48, 0, False)])
def test_attention_part_in_portions(dtype, heads, kv_heads, hd, window, bias):
    from vipera_rs_amd.config import PartSpec
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.parts import part_class
    rt = _runtime(dtype)
    hidden = 56
    spec = PartSpec("attention", {"hidden": hidden, "heads": heads, "kv_heads": kv_heads, "head_dim": hd, "qkv_bias": bias,
                                  "out_bias": False, "window": window, "scale": None, "name": "attn"})
    cls = part_class("mixer", "attention")
    host, dev = _random_part_tensors(cls, spec, "l.", 5, rt)
    for name in host:                       # larger weights, so that the scores are not all alike
        if name.endswith("proj.weight"):
            dev[name] = (dev[name].float() * 8).to(dev[name].dtype)
            host[name] = dev[name].double().cpu().numpy()
    mixer = cls(spec, "l.", rt)
    mixer.load(dev)
    pos_spec = PartSpec("rotary_neox", {"head_dim": hd, "rotary_dim": hd, "base": 10000.0})
    position = part_class("position", "rotary_neox")(pos_spec, "l.", rt)
    T = 37
    h = torch.randn(T, hidden).to(rt.dtype).to(DEV)
    cfg = {"num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": hd, "rope_theta": 10000.0}
    w = {k.replace("l.attn.", ""): v for k, v in host.items()}
    want = P.attention_block(h.double().cpu().numpy(), w, "", cfg, window)
    env = _OneLayerCache(rt, mixer.cache_spec())
    residual = torch.zeros(T, hidden, device=DEV)
    at = 0
    for size in (5, 1, 16, 2, 13):          # portions of changing size; every one adds its rows
        batch = env.batch([StepEntry(0, at, [1] * size)])
        mixer.forward(h[at:at + size].contiguous(), batch, env.storage.kv[0], None, position, residual[at:at + size])
        env.cache.advance(0, at + size)
        at += size
    assert rel_err(residual.cpu().numpy(), want) < (2e-5 if dtype == "float32" else 2e-2)


# --- a run order that names a layer twice and lets an entry read another entry's cache ---------------------------
def _plain_scheduled(cfg, w, tokens, schedule):
    """Plain forward with an explicit run order: (layer, cache_of) pairs; a reading entry uses the keys
    and values that the owning entry computed (from the owner's input), and its own queries."""
    cfg = P.normalize_config(cfg)
    T = len(tokens)
    heads, kv_heads, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    x = w["model.embed_tokens.weight"][np.asarray(tokens)]
    kept = {}
    for index, (layer, cache_of) in enumerate(schedule):
        p = f"model.layers.{layer}."
        h = P.rms_norm(x, w[p + "input_layernorm.weight"], cfg["rms_norm_eps"])
        a = p + "self_attn."
        q = P.linear(h, w[a + "q_proj.weight"], w[a + "q_proj.bias"]).reshape(T, heads, hd)
        for t in range(T):
            q[t] = P.rope_neox(q[t], t, cfg["rope_theta"])
        if cache_of is None:
            k = P.linear(h, w[a + "k_proj.weight"], w[a + "k_proj.bias"]).reshape(T, kv_heads, hd)
            v = P.linear(h, w[a + "v_proj.weight"], w[a + "v_proj.bias"]).reshape(T, kv_heads, hd)
            for t in range(T):
                k[t] = P.rope_neox(k[t], t, cfg["rope_theta"])
            kept[index] = (k, v)
        else:
            k, v = kept[cache_of]
        x = x + P.linear(P.attention(q, k, v).reshape(T, heads * hd), w[a + "o_proj.weight"])
        h = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + P.swiglu_mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    h = P.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    return P.linear(h, w["model.embed_tokens.weight"])


def test_the_run_order_is_data(tmp_path):
    from vipera_rs_amd.config import Qwen2Config, ScheduleEntry, register_architecture, unregister_architecture
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    from vipera_rs_amd.models.decoder import DecoderModel

    order = [(0, None), (1, None), (0, None), (1, 1)]     # layer 0 twice (two caches); the last entry reads entry 1's cache

    class Looped(Qwen2Config):
        architecture = "LoopedForCausalLM"

        def schedule(self):
            return [ScheduleEntry(layer, cache_of) for layer, cache_of in order]

    register_architecture("LoopedForCausalLM", Looped, lambda config, runtime: DecoderModel(config, runtime))
    try:
        folder = make_folder(tmp_path / "looped", dict(CONFIG_A, architectures=["LoopedForCausalLM"]), 4)
        cfg, w = P.load_folder(folder)
        tokens = random_tokens(256, 29, 9)
        want = _plain_scheduled(cfg, w, tokens, order)
        runner = ModelRunner.from_folder(folder, dtype="float32", block_size=8, num_blocks=16, num_slots=2)
        assert sum(kv is not None for kv in runner.storage.kv) == 4
        assert runner.storage.kv[3] is runner.storage.kv[1] and runner.storage.kv[2] is not runner.storage.kv[0]
        rows, at = [], 0
        for size in (11, 1, 2, 15):
            runner.cache.reserve(0, at, at + size)
            rows.append(runner.step([StepEntry(0, at, tokens[at:at + size], list(range(size)))]).cpu().numpy())
            at += size
        assert rel_err(np.concatenate(rows), want) < 1e-4
    finally:
        unregister_architecture("LoopedForCausalLM")


# --- a toy mixer with state of its own, defined here ----------------------------------------------------------------
STATE_DECAY, STATE_WIDTH = 0.9, 24


@contextlib.contextmanager
def _stateful_toy():
    """Registers ``s_t = decay * s_{t-1} + W_in h_t``, ``y_t = W_out s_t`` (one vector of state per request, no
    pages) as the mixer of layer 0 of a toy architecture whose layer 1 is ordinary attention: different mixers
    in different layers of one model.  Yields the plain implementation of that model."""
    from vipera_rs_amd.config import (LayerSpec, PartSpec, Qwen2Config, register_architecture, unregister_architecture)
    from vipera_rs_amd.models.decoder import DecoderModel
    from vipera_rs_amd.parts import Mixer, StateSpec, register_mixer, unregister
    from vipera_rs_amd.weights import MATRIX, TensorSpec

    class RunningState(Mixer):
        def __init__(self, spec, prefix, runtime):
            super().__init__(spec, prefix, runtime)
            self.hidden = spec.params["hidden"]
            self.w_in = self.w_out = None

        @classmethod
        def declare(cls, spec, prefix):
            base = f"{prefix}{spec.params['name']}."
            return [TensorSpec(base + "in.weight", (STATE_WIDTH, spec.params["hidden"]), MATRIX, std=0.3),
                    TensorSpec(base + "out.weight", (spec.params["hidden"], STATE_WIDTH), MATRIX, std=0.3)]

        def load(self, tensors):
            base = f"{self.prefix}{self.spec.params['name']}."
            self.w_in, self.w_out = tensors[base + "in.weight"].float(), tensors[base + "out.weight"].float()

        @classmethod
        def declare_cache(cls, spec):
            return None, StateSpec((STATE_WIDTH,), torch.float32)

        def forward(self, h, batch, cache, state, position, residual, reads_only=False):
            u = h.float() @ self.w_in.T
            if batch.all_single:
                # one token per entry: only what lies on the device is looked at, so the step can be captured
                slots = batch.slots.long()
                fresh = (batch.entry_first_pos == 0).unsqueeze(1)                      # zero on first use
                s = STATE_DECAY * torch.where(fresh, torch.zeros_like(u), state.index_select(0, slots)) + u
                residual += s @ self.w_out.T
                state.index_copy_(0, slots, s)
                return
            at = 0
            for count, first, slot in zip(batch.host_counts, batch.host_first_pos, batch.host_slots):
                s = torch.zeros(STATE_WIDTH, device=h.device) if first == 0 else state[slot].clone()
                for t in range(at, at + count):
                    s = STATE_DECAY * s + u[t]
                    residual[t] += s @ self.w_out.T
                state[slot] = s
                at += count

    class ToyConfig(Qwen2Config):
        architecture = "ToyStateForCausalLM"

        def layer_specs(self) -> List[LayerSpec]:
            specs = super().layer_specs()
            first = specs[0]
            specs[0] = LayerSpec(first.block, PartSpec("running_state", {"hidden": self.hidden_size, "name": "state"}),
                                 first.ffn, first.mixer_norm, first.ffn_norm, PartSpec("none", {}), first.prefix)
            return specs

    def plain(cfg, w, tokens):
        cfg = P.normalize_config(cfg)
        x = w["model.embed_tokens.weight"][np.asarray(tokens)]
        h = P.rms_norm(x, w["model.layers.0.input_layernorm.weight"], cfg["rms_norm_eps"])
        s, ys = np.zeros(STATE_WIDTH), []
        for t in range(len(tokens)):
            s = STATE_DECAY * s + w["model.layers.0.state.in.weight"] @ h[t]
            ys.append(w["model.layers.0.state.out.weight"] @ s)
        x = x + np.stack(ys)
        h = P.rms_norm(x, w["model.layers.0.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + P.swiglu_mlp(h, *(w[f"model.layers.0.mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
        h = P.rms_norm(x, w["model.layers.1.input_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + P.attention_block(h, w, "model.layers.1.self_attn.", cfg, 0)
        h = P.rms_norm(x, w["model.layers.1.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + P.swiglu_mlp(h, *(w[f"model.layers.1.mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
        head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
        return P.linear(P.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]), head)

    register_mixer("running_state", RunningState)
    register_architecture("ToyStateForCausalLM", ToyConfig, lambda config, runtime: DecoderModel(config, runtime))
    try:
        yield plain
    finally:
        unregister_architecture("ToyStateForCausalLM")
        unregister("mixer", "running_state")


def test_a_stateful_toy_mixer_is_registered_built_and_stepped(tmp_path):
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner

    with _stateful_toy() as plain:
        folder = make_folder(tmp_path / "toy", dict(CONFIG_A, architectures=["ToyStateForCausalLM"]), 6)
        cfg, w = P.load_folder(folder)
        assert "model.layers.0.state.in.weight" in w and "model.layers.0.self_attn.q_proj.weight" not in w
        runner = ModelRunner.from_folder(folder, dtype="float32", block_size=8, num_blocks=24, num_slots=3)
        # a row per slot and the scratch row of a captured step's padding entries
        assert runner.storage.state[0].shape == (3 + 1, STATE_WIDTH) and runner.storage.kv[0] is None
        assert runner.storage.kv[1] is not None and runner.storage.state[1] is None
        requests = {0: random_tokens(256, 23, 1), 1: random_tokens(256, 17, 2), 2: random_tokens(256, 9, 3)}
        want = {r: plain(cfg, w, toks) for r, toks in requests.items()}
        # mixed steps: portions of some requests beside single tokens of others; request 2 starts late in the
        # slot and pages that request 1 gave back, so state left in a slot must not leak into a new request
        at = {r: 0 for r in requests}
        plan = [[(0, 7), (1, 2)], [(0, 1), (1, 9)], [(1, 6)], [(0, 13), (2, 4)], [(0, 2), (2, 1)], [(2, 4)]]
        for step in plan:
            entries = []
            for r, size in step:
                runner.cache.reserve(r, at[r], at[r] + size)
                entries.append(StepEntry(r, at[r], requests[r][at[r]:at[r] + size], list(range(size))))
            logits = runner.step(entries).cpu().numpy()
            row = 0
            for r, size in step:
                assert rel_err(logits[row:row + size], want[r][at[r]:at[r] + size]) < 1e-4, (r, at[r])
                row += size
                at[r] += size
                if at[r] == len(requests[r]):
                    runner.cache.release(r)
        assert at == {r: len(t) for r, t in requests.items()} and runner.cache.check() == ""


@pytest.mark.parametrize("pipelined", [False, True])
def test_a_stateful_toy_mixer_generates_through_captured_steps_with_padding(tmp_path, pipelined):
    """Three live requests decode in a captured step of four entries (``pipelined``: each step launched before the
    tokens of the step before have reached the host, which reads them on the device).  The padding entry writes the scratch
    state row and not slot 0, which a live request holds, and the first use of a graph runs a step once: either
    fault would change a request's state and, from there on, its tokens."""
    from vipera_rs_amd import Engine
    from vipera_rs_amd.cli import plan_model

    with _stateful_toy() as plain:
        config = dict(CONFIG_A, architectures=["ToyStateForCausalLM"], tie_word_embeddings=False)
        folder = make_folder(tmp_path / "toy", config, 8)
        cfg, w = P.load_folder(folder)
        prompts = [random_tokens(256, n, 50 + n) for n in (7, 12, 3)]
        engine = Engine(folder, dtype="float32", block_size=8, num_blocks=24, max_num_seqs=3, use_graphs=True,
                        pipelined=pipelined)
        assert engine.pipelined == pipelined
        got = engine.generate(prompts, max_new_tokens=20)
        graphs = engine.runner.graphs
        assert graphs.replays >= 19 and any(key[0] == 4 for key in graphs.graphs), "no padded captured step ran"
        assert engine.runner.storage.scratch_slot == 3
        checked = 0
        for p, g in zip(prompts, got):
            assert len(g.tokens) == 20
            logits = plain(cfg, w, p + g.tokens[:-1])
            checked += assert_tokens_follow_plain(logits, len(p), g.tokens, 2.5e-5, f"prompt of {len(p)}")
        assert checked > 40
        # the state's bytes are part of the memory plan: one row per request and the scratch row
        planned = plan_model(folder, 64, 3, "float32", 8)
        assert planned["state_bytes"] == (3 + 1) * STATE_WIDTH * 4
        assert engine.stats()["kv_bytes"] == engine.runner.storage.bytes >= planned["state_bytes"]


# --- an arrangement with four norms and an embedding that adds a learned position, defined here -------------------
def test_a_block_with_four_norms_and_an_embedding_that_adds_positions(tmp_path):
    """``x += norm_b(mixer(norm_a(x))); x += norm_d(ffn(norm_c(x)))`` with the two extra norms named in
    ``LayerSpec.extras``, and ``x_0 = table[token] + places[position]``: another arrangement and another embedding
    are registered from this file; the framework's blocks, models and step function are not touched."""
    from vipera_rs_amd.config import (LayerSpec, PartSpec, Qwen2Config, register_architecture, unregister_architecture)
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    from vipera_rs_amd.models.decoder import DecoderModel
    from vipera_rs_amd.parts import Block, Part, part_class, register_block, register_embedding, unregister
    from vipera_rs_amd.weights import MATRIX, TensorSpec

    ROLES = ("mixer_norm", "after_mixer", "ffn_norm", "after_ffn")

    class Sandwich(Block):
        def __init__(self, spec, runtime):
            super().__init__(spec, runtime)
            norms = {"mixer_norm": spec.mixer_norm, "ffn_norm": spec.ffn_norm, **spec.extras}
            self.norms = {role: part_class("norm", norms[role].kind)(norms[role], spec.prefix, runtime) for role in ROLES}
            self.mixer = part_class("mixer", spec.mixer.kind)(spec.mixer, spec.prefix, runtime)
            self.ffn = part_class("ffn", spec.ffn.kind)(spec.ffn, spec.prefix, runtime)
            self.position = part_class("position", spec.position.kind)(spec.position, spec.prefix, runtime)

        @classmethod
        def declare(cls, spec):
            norms = {"mixer_norm": spec.mixer_norm, "ffn_norm": spec.ffn_norm, **spec.extras}
            out = []
            for role in ROLES:
                out += part_class("norm", norms[role].kind).declare(norms[role], spec.prefix)
            out += part_class("mixer", spec.mixer.kind).declare(spec.mixer, spec.prefix)
            out += part_class("ffn", spec.ffn.kind).declare(spec.ffn, spec.prefix)
            return out

        def load(self, tensors):
            for part in (*self.norms.values(), self.mixer, self.ffn, self.position):
                part.load(tensors)

        def forward(self, x, batch, cache, state, reads_only=False):
            # a part adds its output into the 32-bit buffer it is given: an empty one collects the output alone
            branch = torch.zeros_like(x)
            self.mixer.forward(self.norms["mixer_norm"].forward(x), batch, cache, state, self.position, branch, reads_only)
            x += self.norms["after_mixer"].forward(branch).float()
            branch.zero_()
            self.ffn.forward(self.norms["ffn_norm"].forward(x), batch, branch)
            x += self.norms["after_ffn"].forward(branch).float()

    class PlacedEmbedding(Part):
        reads_device_tokens = False

        @classmethod
        def declare(cls, spec, prefix):
            p = spec.params
            return [TensorSpec("model.embed_tokens.weight", (p["vocab"], p["width"]), MATRIX),
                    TensorSpec("model.embed_places.weight", (p["places"], p["width"]), MATRIX, std=0.05)]

        def load(self, tensors):
            self.table = tensors["model.embed_tokens.weight"]
            self.places = tensors["model.embed_places.weight"]

        def embed(self, batch):
            return (self.table[batch.tokens[:batch.num_tokens].long()].float()
                    + self.places[batch.positions[:batch.num_tokens].long()].float())

    class SandwichConfig(Qwen2Config):
        architecture = "ToySandwichForCausalLM"

        def layer_specs(self) -> List[LayerSpec]:
            out = []
            for spec in super().layer_specs():
                norm = spec.mixer_norm.params
                extras = {"after_mixer": PartSpec("rmsnorm", dict(norm, name="post_mixer_norm")),
                          "after_ffn": PartSpec("rmsnorm", dict(norm, name="post_ffn_norm"))}
                out.append(LayerSpec("sandwich", spec.mixer, spec.ffn, spec.mixer_norm, spec.ffn_norm, spec.position,
                                     spec.prefix, extras))
            return out

        def embedding_spec(self):
            return PartSpec("placed", {"vocab": self.vocab_size, "width": self.hidden_size, "places": 96})

    def plain(cfg, w, tokens):
        cfg = P.normalize_config(cfg)
        eps = cfg["rms_norm_eps"]
        x = w["model.embed_tokens.weight"][np.asarray(tokens)] + w["model.embed_places.weight"][:len(tokens)]
        for i in range(cfg["num_hidden_layers"]):
            p = f"model.layers.{i}."
            h = P.rms_norm(x, w[p + "input_layernorm.weight"], eps)
            x = x + P.rms_norm(P.attention_block(h, w, p + "self_attn.", cfg, 0), w[p + "post_mixer_norm.weight"], eps)
            h = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
            y = P.swiglu_mlp(h, *(w[f"{p}mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
            x = x + P.rms_norm(y, w[p + "post_ffn_norm.weight"], eps)
        return P.linear(P.rms_norm(x, w["model.norm.weight"], eps), w["lm_head.weight"])

    register_block("sandwich", Sandwich)
    register_embedding("placed", PlacedEmbedding)
    register_architecture("ToySandwichForCausalLM", SandwichConfig, lambda config, runtime: DecoderModel(config, runtime))
    try:
        config = dict(CONFIG_B, architectures=["ToySandwichForCausalLM"])
        for dtype, stored, tol in (("float32", torch.float32, 1e-4), ("bfloat16", torch.bfloat16, 3e-2)):
            folder = make_folder(tmp_path / f"sandwich_{dtype}", config, 12, stored)
            cfg, w = P.load_folder(folder)
            assert "model.layers.2.post_ffn_norm.weight" in w and "model.embed_places.weight" in w
            tokens = random_tokens(300, 60, 77)
            want = plain(cfg, w, tokens)
            runner = ModelRunner.from_folder(folder, dtype=dtype, block_size=8, num_blocks=12, num_slots=2)
            rows, at = [], 0
            for size in (23, 2, 1, 17, 1, 1, 15):
                runner.cache.reserve(0, at, at + size)
                rows.append(runner.step([StepEntry(0, at, tokens[at:at + size], list(range(size)))]).cpu().numpy())
                at += size
            assert at == len(tokens) and rel_err(np.concatenate(rows), want) < tol, dtype
    finally:
        unregister_architecture("ToySandwichForCausalLM")
        unregister("block", "sandwich")
        unregister("embedding", "placed")


# --- a feed-forward with routing and another position encoding, defined here --------------------------------------
def test_a_routed_feed_forward_and_another_position_encoding(tmp_path):
    """Layer 0 gets a top-1-of-three-experts feed-forward (router in 32-bit) and a position encoding that
    is no rotation (a sinusoid of the position added to q and k); layer 1 stays as it is.  Both parts
    live in this file and are only registered with the framework."""
    from vipera_rs_amd.config import (LayerSpec, PartSpec, Qwen2Config, register_architecture, unregister_architecture)
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    from vipera_rs_amd.models.decoder import DecoderModel
    from vipera_rs_amd.parts import (FeedForward, PositionEncoding, register_ffn, register_position, unregister)
    from vipera_rs_amd.weights import MATRIX, TensorSpec

    EXPERTS, INNER = 3, 40

    class TopOne(FeedForward):
        @classmethod
        def declare(cls, spec, prefix):
            hidden = spec.params["hidden"]
            base = f"{prefix}moe."
            out = [TensorSpec(base + "router.weight", (EXPERTS, hidden), MATRIX, std=0.5)]
            for e in range(EXPERTS):
                out.append(TensorSpec(f"{base}experts.{e}.up.weight", (INNER, hidden), MATRIX, std=0.2))
                out.append(TensorSpec(f"{base}experts.{e}.down.weight", (hidden, INNER), MATRIX, std=0.2))
            return out

        def load(self, tensors):
            base = f"{self.prefix}moe."
            self.router = tensors[base + "router.weight"].float()
            self.up = [tensors[f"{base}experts.{e}.up.weight"].float() for e in range(EXPERTS)]
            self.down = [tensors[f"{base}experts.{e}.down.weight"].float() for e in range(EXPERTS)]

        def forward(self, h, batch, residual):
            x = h.float()
            probs = torch.softmax(x @ self.router.T, dim=-1)          # 32-bit router
            weight, choice = probs.max(dim=-1)
            for e in range(EXPERTS):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    y = torch.relu(x[rows] @ self.up[e].T) @ self.down[e].T
                    residual[rows] += weight[rows, None] * y

    class Tilt(PositionEncoding):
        @classmethod
        def declare(cls, spec, prefix):
            return []

        def load(self, tensors):
            pass

        def apply(self, qkv, batch, heads, kv_heads, head_dim):
            width = (heads + kv_heads) * head_dim                       # q and k, not v
            dims = torch.arange(head_dim, device=qkv.device, dtype=torch.float32).repeat(heads + kv_heads)
            signal = 0.5 * torch.sin(batch.positions.float()[:, None] * 0.1 * (dims[None, :] + 1.0))
            qkv[:, :width] = (qkv[:, :width].float() + signal).to(qkv.dtype)

    class MixedConfig(Qwen2Config):
        architecture = "ToyRoutedForCausalLM"

        def layer_specs(self) -> List[LayerSpec]:
            specs = super().layer_specs()
            first = specs[0]
            specs[0] = LayerSpec(first.block, first.mixer, PartSpec("top_one", {"hidden": self.hidden_size}),
                                 first.mixer_norm, first.ffn_norm, PartSpec("tilt", {}), first.prefix)
            return specs

    def plain(cfg, w, tokens):
        cfg = P.normalize_config(cfg)
        T = len(tokens)
        heads, kv_heads, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
        x = w["model.embed_tokens.weight"][np.asarray(tokens)]
        h = P.rms_norm(x, w["model.layers.0.input_layernorm.weight"], cfg["rms_norm_eps"])
        a = "model.layers.0.self_attn."
        q = P.linear(h, w[a + "q_proj.weight"], w.get(a + "q_proj.bias")).reshape(T, heads, hd)
        k = P.linear(h, w[a + "k_proj.weight"], w.get(a + "k_proj.bias")).reshape(T, kv_heads, hd)
        v = P.linear(h, w[a + "v_proj.weight"], w.get(a + "v_proj.bias")).reshape(T, kv_heads, hd)
        signal = 0.5 * np.sin(np.arange(T)[:, None] * 0.1 * (np.arange(hd)[None, :] + 1.0))
        q, k = q + signal[:, None, :], k + signal[:, None, :]
        x = x + P.linear(P.attention(q, k, v, window=0).reshape(T, heads * hd), w[a + "o_proj.weight"])
        h = P.rms_norm(x, w["model.layers.0.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        logits = h @ w["model.layers.0.moe.router.weight"].T
        probs = np.exp(logits - logits.max(-1, keepdims=True))
        probs /= probs.sum(-1, keepdims=True)
        for t in range(T):
            e = int(probs[t].argmax())
            y = np.maximum(w[f"model.layers.0.moe.experts.{e}.up.weight"] @ h[t], 0.0)
            x[t] = x[t] + probs[t, e] * (w[f"model.layers.0.moe.experts.{e}.down.weight"] @ y)
        h = P.rms_norm(x, w["model.layers.1.input_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + P.attention_block(h, w, "model.layers.1.self_attn.", cfg, 0)
        h = P.rms_norm(x, w["model.layers.1.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + P.swiglu_mlp(h, *(w[f"model.layers.1.mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
        return P.linear(P.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]), w["model.embed_tokens.weight"])

    register_ffn("top_one", TopOne)
    register_position("tilt", Tilt)
    register_architecture("ToyRoutedForCausalLM", MixedConfig, lambda config, runtime: DecoderModel(config, runtime))
    try:
        folder = make_folder(tmp_path / "routed", dict(CONFIG_A, architectures=["ToyRoutedForCausalLM"]), 8)
        cfg, w = P.load_folder(folder)
        assert "model.layers.0.moe.router.weight" in w and "model.layers.0.mlp.gate_proj.weight" not in w
        tokens = random_tokens(256, 31, 4)
        want = plain(cfg, w, tokens)
        runner = ModelRunner.from_folder(folder, dtype="float32", block_size=8, num_blocks=16, num_slots=2)
        rows, at = [], 0
        for size in (9, 1, 1, 13, 2, 5):
            runner.cache.reserve(0, at, at + size)
            rows.append(runner.step([StepEntry(0, at, tokens[at:at + size], list(range(size)))]).cpu().numpy())
            at += size
        assert rel_err(np.concatenate(rows), want) < 1e-4
    finally:
        unregister_architecture("ToyRoutedForCausalLM")
        unregister("ffn", "top_one")
        unregister("position", "tilt")


def test_a_position_part_with_per_head_norms_of_q_and_k(tmp_path):
    """What the reference hooks in before the rotation for architectures that have it (per-head RMS norms of q and k,
    crates/vipera-backend-cpu/src/model.rs:312-313, 630-645) needs no change to the attention part: a position
    encoding declares tensors of its own and changes q and k in place before they reach the cache.  Layer 0 gets such
    a part from this file (norm per head with a weight of the head's width, then the NeoX rotation); layer 1 stays
    as it is, fused rotation and all."""
    from vipera_rs_amd.config import (LayerSpec, PartSpec, Qwen2Config, register_architecture, unregister_architecture)
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    from vipera_rs_amd.models.decoder import DecoderModel
    from vipera_rs_amd.parts import PositionEncoding, register_position, unregister
    from vipera_rs_amd.parts.rotary import neox_inverse_frequencies
    from vipera_rs_amd.weights import VECTOR, TensorSpec

    class NormedRotary(PositionEncoding):
        @classmethod
        def declare(cls, spec, prefix):
            hd = int(spec.params["head_dim"])
            return [TensorSpec(f"{prefix}self_attn.{n}_norm.weight", (hd,), VECTOR, "one_plus_normal", std=0.3) for n in "qk"]

        def load(self, tensors):
            self.gain = {n: tensors[f"{self.prefix}self_attn.{n}_norm.weight"].float() for n in "qk"}
            hd = int(self.spec.params["head_dim"])
            self.inv = torch.from_numpy(neox_inverse_frequencies(hd, float(self.spec.params["base"]))).to(self.runtime.device)
            self.eps = float(self.spec.params["eps"])

        def apply(self, qkv, batch, heads, kv_heads, head_dim):
            angle = batch.positions.float()[:, None] * self.inv[None, :]          # 32-bit, as the rotation kernels have it
            sin, cos = torch.sin(angle)[:, None, :], torch.cos(angle)[:, None, :]
            at = 0
            for name, count in (("q", heads), ("k", kv_heads)):
                x = qkv[:, at:at + count * head_dim].float().view(-1, count, head_dim)
                x = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + self.eps) * self.gain[name]
                lo, hi = x[..., :head_dim // 2], x[..., head_dim // 2:]
                x = torch.cat([lo * cos - hi * sin, lo * sin + hi * cos], dim=-1)
                qkv[:, at:at + count * head_dim] = x.reshape(-1, count * head_dim).to(qkv.dtype)
                at += count * head_dim

    class NormedConfig(Qwen2Config):
        architecture = "ToyNormedForCausalLM"

        def layer_specs(self) -> List[LayerSpec]:
            specs = super().layer_specs()
            first = specs[0]
            position = PartSpec("normed_rotary", {"head_dim": self.head_dim, "base": self.rope_theta, "eps": 1e-6})
            specs[0] = LayerSpec(first.block, first.mixer, first.ffn, first.mixer_norm, first.ffn_norm, position, first.prefix)
            return specs

    def plain(cfg, w, tokens):
        cfg = P.normalize_config(cfg)
        T = len(tokens)
        heads, kv_heads, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
        x = w["model.embed_tokens.weight"][np.asarray(tokens)]
        h = P.rms_norm(x, w["model.layers.0.input_layernorm.weight"], cfg["rms_norm_eps"])
        a = "model.layers.0.self_attn."
        q = P.linear(h, w[a + "q_proj.weight"], w.get(a + "q_proj.bias")).reshape(T, heads, hd)
        k = P.linear(h, w[a + "k_proj.weight"], w.get(a + "k_proj.bias")).reshape(T, kv_heads, hd)
        v = P.linear(h, w[a + "v_proj.weight"], w.get(a + "v_proj.bias")).reshape(T, kv_heads, hd)
        q = P.rms_norm(q, w[a + "q_norm.weight"], 1e-6)            # over a head's width, one weight for all heads
        k = P.rms_norm(k, w[a + "k_norm.weight"], 1e-6)
        q = np.stack([P.rope_neox(q[t], t, cfg["rope_theta"]) for t in range(T)])
        k = np.stack([P.rope_neox(k[t], t, cfg["rope_theta"]) for t in range(T)])
        x = x + P.linear(P.attention(q, k, v, window=0).reshape(T, heads * hd), w[a + "o_proj.weight"])
        h = P.rms_norm(x, w["model.layers.0.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + P.swiglu_mlp(h, *(w[f"model.layers.0.mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
        h = P.rms_norm(x, w["model.layers.1.input_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + P.attention_block(h, w, "model.layers.1.self_attn.", cfg, 0)
        h = P.rms_norm(x, w["model.layers.1.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + P.swiglu_mlp(h, *(w[f"model.layers.1.mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
        return P.linear(P.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]), w["model.embed_tokens.weight"])

    register_position("normed_rotary", NormedRotary)
    register_architecture("ToyNormedForCausalLM", NormedConfig, lambda config, runtime: DecoderModel(config, runtime))
    try:
        folder = make_folder(tmp_path / "normed", dict(CONFIG_A, architectures=["ToyNormedForCausalLM"]), 9)
        cfg, w = P.load_folder(folder)
        assert w["model.layers.0.self_attn.q_norm.weight"].shape == (P.normalize_config(cfg)["head_dim"],)
        assert "model.layers.1.self_attn.q_norm.weight" not in w
        tokens = random_tokens(256, 30, 5)
        want = plain(cfg, w, tokens)
        for dtype, tol in (("float32", 1e-4), ("bfloat16", 3e-2)):
            runner = ModelRunner.from_folder(folder, dtype=dtype, block_size=8, num_blocks=16, num_slots=2)
            rows, at = [], 0
            for size in (11, 1, 1, 9, 2, 6):
                runner.cache.reserve(0, at, at + size)
                rows.append(runner.step([StepEntry(0, at, tokens[at:at + size], list(range(size)))]).float().cpu().numpy())
                at += size
            assert rel_err(np.concatenate(rows), want) < tol, dtype
    finally:
        unregister_architecture("ToyNormedForCausalLM")
        unregister("position", "normed_rotary")


def test_a_toy_feed_forward_takes_a_norm_handed_to_it(tmp_path):
    """A feed-forward defined here accepts a handed-off norm (`parts.NormHandoff`): for steps of up to 16 tokens
    the attention before it leaves `x * gain` and its workgroups' sums of squares instead of the norm running
    as a kernel, and the toy divides by the root mean square itself.  Longer steps reach it with `h` as ever.
    Both ways give the plain implementation's logits."""
    from vipera_rs_amd.config import (LayerSpec, PartSpec, Qwen2Config, register_architecture, unregister_architecture)
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    from vipera_rs_amd.models.decoder import DecoderModel
    from vipera_rs_amd.parts import FeedForward, register_ffn, unregister
    from vipera_rs_amd.weights import MATRIX, TensorSpec
    INNER = 48
    seen = {"handed": 0, "plain": 0}

    class Handed(FeedForward):
        @classmethod
        def declare(cls, spec, prefix):
            hidden = spec.params["hidden"]
            return [TensorSpec(f"{prefix}toy.up.weight", (INNER, hidden), MATRIX, std=0.2),
                    TensorSpec(f"{prefix}toy.down.weight", (hidden, INNER), MATRIX, std=0.2)]

        def load(self, tensors):
            self.up = tensors[f"{self.prefix}toy.up.weight"].float()
            self.down = tensors[f"{self.prefix}toy.down.weight"].float()

        def accepts_handoff(self, tokens):
            return tokens <= 16

        def forward(self, h, batch, residual, handoff=None):
            if handoff is not None:
                seen["handed"] += 1
                tokens, width = handoff.scaled.shape
                squares = handoff.sumsq[: handoff.groups * 16].view(handoff.groups, 16).sum(0)[:tokens]
                h = handoff.scaled.float() * torch.rsqrt(squares / width + handoff.eps)[:, None]
            else:
                seen["plain"] += 1
            residual += torch.relu(h.float() @ self.up.T) @ self.down.T

    class ToyConfig(Qwen2Config):
        architecture = "ToyHandedForCausalLM"

        def layer_specs(self) -> List[LayerSpec]:
            specs = super().layer_specs()
            first = specs[0]
            specs[0] = LayerSpec(first.block, first.mixer, PartSpec("handed", {"hidden": self.hidden_size}),
                                 first.mixer_norm, first.ffn_norm, first.position, first.prefix)
            return specs

    def plain(cfg, w, tokens):
        cfg = P.normalize_config(cfg)
        x = w["model.embed_tokens.weight"][np.asarray(tokens)]
        h = P.rms_norm(x, w["model.layers.0.input_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + P.attention_block(h, w, "model.layers.0.self_attn.", cfg, 0)
        h = P.rms_norm(x, w["model.layers.0.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + np.maximum(h @ w["model.layers.0.toy.up.weight"].T, 0.0) @ w["model.layers.0.toy.down.weight"].T
        h = P.rms_norm(x, w["model.layers.1.input_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + P.attention_block(h, w, "model.layers.1.self_attn.", cfg, 0)
        h = P.rms_norm(x, w["model.layers.1.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + P.swiglu_mlp(h, *(w[f"model.layers.1.mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
        return P.linear(P.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]), w["model.embed_tokens.weight"])

    register_ffn("handed", Handed)
    register_architecture("ToyHandedForCausalLM", ToyConfig, lambda config, runtime: DecoderModel(config, runtime))
    try:
        folder = make_folder(tmp_path / "handed", dict(CONFIG_A, architectures=["ToyHandedForCausalLM"]), 9, torch.bfloat16)
        cfg, w = P.load_folder(folder)
        tokens = random_tokens(256, 45, 6)
        want = plain(cfg, w, tokens)
        runner = ModelRunner.from_folder(folder, dtype="bfloat16", block_size=8, num_blocks=16, num_slots=2)
        rows, at = [], 0
        for size in (20, 1, 1, 16, 2, 5):
            runner.cache.reserve(0, at, at + size)
            rows.append(runner.step([StepEntry(0, at, tokens[at:at + size], list(range(size)))]).cpu().numpy())
            at += size
        assert rel_err(np.concatenate(rows), want) < 3e-2
        assert seen == {"handed": 5, "plain": 1}
    finally:
        unregister_architecture("ToyHandedForCausalLM")
        unregister("ffn", "handed")


# --- the first tokens of a sequence --------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(tmp_path, dtype):
    from vipera_rs_amd.engine.batch import StepEntry
    from vipera_rs_amd.engine.runner import ModelRunner
    folder = make_folder(tmp_path / "m", CONFIG_B, 1, torch.float32 if dtype == "float32" else torch.bfloat16)
    cfg, w = P.load_folder(folder)
    runner = ModelRunner.from_folder(folder, dtype=dtype, block_size=8, num_blocks=8, num_slots=4)
    tol = 1e-4 if dtype == "float32" else 3e-2
    for rid, tokens in enumerate(([7], [7, 7], [299, 0, 150])):
        want = P.forward(cfg, w, tokens)
        runner.cache.reserve(rid, 0, len(tokens))
        whole = runner.step([StepEntry(rid, 0, tokens, list(range(len(tokens))))]).cpu().numpy()
        assert rel_err(whole, want) < tol
        runner.cache.release(rid)
        rows = []
        for pos, token in enumerate(tokens):     # and one by one from position 0
            runner.cache.reserve(10 + rid, pos, pos + 1)
            rows.append(runner.step([StepEntry(10 + rid, pos, [token], [0])]).cpu().numpy()[0])
        runner.cache.release(10 + rid)
        assert rel_err(np.stack(rows), want) < tol
