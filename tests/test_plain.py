"""What pins the plain implementation beside the reference's text: vectors that the reference's own
tests hold, special cases that reduce to a library routine, and invariants; each chosen so that a
plausible mistake (a wrong sign or pairing, a norm in the wrong place, an off-by-one mask) fails it."""
import math

import numpy as np
import pytest
import torch

from helpers import CONFIG_A, CONFIG_B, CONFIG_D, make_folder
from plain import qwen2_plain as P
from plain import sampler_plain as S


# --- vectors from the reference's tests ------------------------------------------------------------
def test_rms_norm_vector():
    # crates/vipera-backend-cpu/src/model.rs:4465-4471: [3, 4] with unit weight and eps 0 -> x / sqrt(12.5)
    out = P.rms_norm(np.array([3.0, 4.0]), np.ones(2), 0.0)
    np.testing.assert_allclose(out, np.array([3.0, 4.0]) / math.sqrt(12.5), rtol=1e-12)


def test_rope_vectors():
    # model.rs:4653-4661: rope([1, 0], pos 1, base 1) = [cos 1, sin 1]; position 0 is the identity
    out = P.rope_neox(np.array([[1.0, 0.0]]), 1, 1.0)
    np.testing.assert_allclose(out[0], [math.cos(1.0), math.sin(1.0)], rtol=1e-7)
    np.testing.assert_allclose(P.rope_neox(np.array([[2.0, 5.0]]), 0, 10000.0)[0], [2.0, 5.0])


def test_attention_vectors():
    # model.rs:5451-5470: one position returns its value; two positions weigh the first 1 / (1 + e^(-1/sqrt 2))
    q = np.array([[[1.0, 0.0]], [[1.0, 0.0]]])
    k = np.array([[[1.0, 0.0]], [[0.0, 0.0]]])
    v = np.array([[[1.0, 0.0]], [[0.0, 1.0]]])
    out = P.attention(q, k, v)
    np.testing.assert_allclose(out[0, 0], [1.0, 0.0])
    w0 = 1.0 / (1.0 + math.exp(-1.0 / math.sqrt(2.0)))
    np.testing.assert_allclose(out[1, 0], [w0, 1.0 - w0], rtol=1e-12)


def test_grouped_heads_share_a_key_head():
    # model.rs:6095-6108: two query heads over one key head both return that head's value
    q = np.random.default_rng(0).normal(size=(1, 2, 2))
    out = P.attention(q, np.array([[[0.5, 0.5]]]), np.array([[[2.0, 3.0]]]))
    np.testing.assert_allclose(out.reshape(-1), [2.0, 3.0, 2.0, 3.0])
    # four heads over two key heads: heads 0,1 -> key head 0; heads 2,3 -> key head 1 (integer division)
    v = np.array([[[1.0, 1.0], [7.0, 7.0]]])
    out = P.attention(np.zeros((1, 4, 2)), np.zeros((1, 2, 2)), v)
    np.testing.assert_allclose(out[0, :, 0], [1.0, 1.0, 7.0, 7.0])


def test_silu_against_the_logistic_function():
    # model.rs:4527-4538: within 2e-6 of z * sigmoid(z) on [-30, 30)
    from scipy.special import expit
    z = np.linspace(-30, 30, 2001)
    np.testing.assert_allclose(P.silu(z), z * expit(z), rtol=2e-6, atol=1e-12)
    assert P.silu(np.array([0.0]))[0] == 0.0 and abs(P.silu(np.array([40.0]))[0] - 40.0) < 1e-9


# --- special cases that reduce to a library routine ---------------------------------------------------
def test_rms_norm_is_division_by_the_root_mean_square():
    x = np.random.default_rng(1).normal(size=(5, 33))
    out = P.rms_norm(x, np.ones(33), 0.0)
    np.testing.assert_allclose(out, x / np.linalg.norm(x, axis=-1, keepdims=True) * math.sqrt(33), rtol=1e-12)
    np.testing.assert_allclose(np.sqrt(np.mean(out * out, axis=-1)), 1.0, rtol=1e-12)
    # eps is added to the mean inside the root, and the weight multiplies afterwards
    w = np.arange(1, 34, dtype=np.float64)
    np.testing.assert_allclose(P.rms_norm(x, w, 0.5), x / np.sqrt(np.mean(x * x, -1, keepdims=True) + 0.5) * w, rtol=1e-12)


def test_attention_without_rotation_is_masked_softmax():
    rng = np.random.default_rng(2)
    T, H, D = 9, 3, 8
    q, k, v = (rng.normal(size=(T, H, D)) for _ in range(3))
    got = P.attention(q, k, v)
    qt, kt, vt = (torch.tensor(a).permute(1, 0, 2) for a in (q, k, v))
    want = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, is_causal=True).permute(1, 0, 2).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)


def test_one_position_attention_returns_the_value():
    rng = np.random.default_rng(3)
    q, k, v = rng.normal(size=(1, 4, 6)), rng.normal(size=(1, 2, 6)), rng.normal(size=(1, 2, 6))
    np.testing.assert_allclose(P.attention(q, k, v)[0], np.repeat(v[0], 2, axis=0))


def test_linear_is_a_matrix_product_with_the_bias_added_after():
    rng = np.random.default_rng(4)
    x, w, b = rng.normal(size=(3, 5)), rng.normal(size=(7, 5)), rng.normal(size=7)
    np.testing.assert_allclose(P.linear(x, w, b), np.einsum("tk,nk->tn", x, w) + b, rtol=1e-12)


# --- invariants ------------------------------------------------------------------------------------------
def test_rotation_keeps_lengths_and_pairs_i_with_i_plus_half():
    rng = np.random.default_rng(5)
    x = rng.normal(size=(2, 8))
    out = P.rope_neox(x, 11, 10000.0)
    half = 4
    for i in range(half):   # the pair (i, i + half) keeps its length; (2i, 2i + 1) would not
        np.testing.assert_allclose(out[:, i] ** 2 + out[:, i + half] ** 2, x[:, i] ** 2 + x[:, i + half] ** 2, rtol=1e-12)
    assert not np.allclose(out[:, 0] ** 2 + out[:, 1] ** 2, x[:, 0] ** 2 + x[:, 1] ** 2)
    # the first pair turns by exactly `position` radians (inverse frequency 1), counter-clockwise
    unit = np.zeros((1, 8)); unit[0, 0] = 1.0
    turned = P.rope_neox(unit, 1, 10000.0)
    np.testing.assert_allclose([turned[0, 0], turned[0, half]], [math.cos(1.0), math.sin(1.0)], rtol=1e-7)


def test_scores_depend_on_distances_only():
    rng = np.random.default_rng(6)
    q, k = rng.normal(size=(1, 16)), rng.normal(size=(1, 16))
    base = 1000000.0
    dots = [float(P.rope_neox(q, p + shift, base)[0] @ P.rope_neox(k, p, base)[0]) for p, shift in ((3, 4), (40, 4), (400, 4))]
    np.testing.assert_allclose(dots, dots[0], rtol=1e-5)
    assert abs(dots[0] - float(P.rope_neox(q, 8, base)[0] @ P.rope_neox(k, 3, base)[0])) > 1e-3   # another distance differs


def test_softmax_is_shift_invariant_and_causal():
    rng = np.random.default_rng(7)
    T, H, D = 7, 2, 4
    q, k, v = (rng.normal(size=(T, H, D)) for _ in range(3))
    out = P.attention(q, k, v)
    k2, v2 = k.copy(), v.copy()
    k2[5:], v2[5:] = 99.0, -99.0              # later positions never change earlier outputs
    np.testing.assert_allclose(P.attention(q, k2, v2)[:5], out[:5])
    # a window of w sees exactly the last w positions: with w = 1 every token returns its own value
    np.testing.assert_allclose(P.attention(q, k, v, window=1), v)
    full = P.attention(q[:3], k[:3], v[:3])
    np.testing.assert_allclose(P.attention(q, k, v, window=3)[2], full[2])   # position 2 sees 0..2 either way
    assert not np.allclose(P.attention(q, k, v, window=3)[5], out[5])


def test_attention_by_head_is_the_same_function():
    rng = np.random.default_rng(8)
    q, k, v = rng.normal(size=(23, 6, 8)), rng.normal(size=(23, 2, 8)), rng.normal(size=(23, 2, 8))
    for window in (0, 1, 5, 23, 40):
        np.testing.assert_allclose(P.attention_by_head(q, k, v, window=window), P.attention(q, k, v, window=window),
                                   rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(P.attention_by_head(q, k, v, scale=0.3), P.attention(q, k, v, scale=0.3), rtol=1e-12)


# --- the whole model ------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    return P.load_folder(make_folder(tmp_path_factory.mktemp("plain_b"), CONFIG_B, 1))


def test_no_layers_leaves_norm_and_head_of_the_embedding(tmp_path):
    cfg = dict(CONFIG_A, num_hidden_layers=0)
    c, w = P.load_folder(make_folder(tmp_path / "m", cfg, 0))
    tokens = [3, 200, 3]
    logits = P.forward(c, w, tokens)
    e = w["model.embed_tokens.weight"][tokens]
    want = P.rms_norm(e, w["model.norm.weight"], c["rms_norm_eps"]) @ w["model.embed_tokens.weight"].T   # tied head
    np.testing.assert_allclose(logits, want, rtol=1e-12)
    np.testing.assert_allclose(logits[0], logits[2])


def test_zero_output_projections_make_logits_independent_of_context(model_b):
    c, w = model_b
    w = dict(w)
    for i in range(c["num_hidden_layers"]):
        w[f"model.layers.{i}.self_attn.o_proj.weight"] = np.zeros_like(w[f"model.layers.{i}.self_attn.o_proj.weight"])
    a = P.forward(c, w, [5, 9, 250, 7])
    b = P.forward(c, w, [100, 7])
    np.testing.assert_allclose(a[3], b[1], rtol=1e-10)


def test_a_prefix_never_depends_on_what_follows(model_b):
    c, w = model_b
    tokens = [4, 8, 15, 16, 23, 42, 108, 299, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20]
    whole = P.forward(c, w, tokens)
    np.testing.assert_allclose(P.forward(c, w, tokens[:10]), whole[:10], rtol=1e-9, atol=1e-12)
    # with windowed layers (21 positions, the fourth configuration's option) the logits beyond the window differ
    # from full attention, and not before
    windowed = P.forward(dict(c, **{k: CONFIG_D[k] for k in ("use_sliding_window", "sliding_window",
                                                             "max_window_layers")}), w, tokens)
    np.testing.assert_allclose(windowed[:21], whole[:21], rtol=1e-9, atol=1e-12)
    assert np.max(np.abs(windowed[27] - whole[27])) > 1e-6


def test_float32_arithmetic_stays_close_to_float64(model_b):
    c, w = model_b
    tokens = list(range(40, 70))
    a, b = P.forward(c, w, tokens), P.forward(c, w, tokens, dtype=np.float32)
    assert np.max(np.abs(a - b)) / np.max(np.abs(a)) < 1e-5


# --- sampling -----------------------------------------------------------------------------------------------------
def test_generator_vectors():
    # xorshift64* seeded through SplitMix64 (crates/vipera-sampler/src/rng.rs:13-57)
    assert S.splitmix64(0) == 0xE220A8397B1DCDAF
    r1, r2 = S.Rng(7), S.Rng(7)
    seq = [r1.next_u64() for _ in range(5)]
    assert seq == [r2.next_u64() for _ in range(5)] and len(set(seq)) == 5
    assert S.Rng(8).next_u64() != seq[0]
    u = [S.Rng(3).next_f64() for _ in range(1)] + [S.Rng(4).next_f64()]
    assert all(0.0 <= x < 1.0 for x in u)
    import vipera_rs_amd  # noqa: F401
    from vipera_rs_amd.sampling import Rng
    ours, theirs = Rng(12345), S.Rng(12345)       # the engine's generator is the same generator
    assert [ours.next_f64() for _ in range(20)] == [theirs.next_f64() for _ in range(20)]
    # the xorshift64* step itself, worked by hand from state 1: x ^= x >> 12 leaves 1, x ^= x << 25 gives
    # 2^25 + 1 = 33554433, x ^= x >> 27 leaves it, and 33554433 * 0x2545F4914F6CDD1D mod 2^64 is the output
    for rng in (S.Rng(0), Rng(0)):
        rng.state = 1
        assert rng.next_u64() == 5180492295206395165 == (33554433 * 0x2545F4914F6CDD1D) % (1 << 64)
        assert rng.state == 33554433
    # a wrong shift or direction changes it: the three shifts are not interchangeable
    assert ((1 ^ (1 << 12)) * 0x2545F4914F6CDD1D) % (1 << 64) != 5180492295206395165


def test_greedy_and_cuts():
    # crates/vipera-conformance/src/lib.rs:461-484: ties to the lowest id, non-finite skipped
    assert S.greedy(np.array([1.0, 3.0, 3.0, 2.0])) == 1
    assert S.greedy(np.array([float("nan"), float("inf"), 0.5, float("-inf")])) == 2
    with pytest.raises(ValueError):
        S.greedy(np.array([float("nan")]))
    logits = np.log(np.array([0.5, 0.25, 0.15, 0.1], dtype=np.float32))
    assert [i for i, _ in S.kept_set(logits, 1.0, 0, 1.0, 0.0)] == [0, 1, 2, 3]
    assert [i for i, _ in S.kept_set(logits, 1.0, 2, 1.0, 0.0)] == [0, 1]                 # top-k
    assert [i for i, _ in S.kept_set(logits, 1.0, 0, 0.7, 0.0)] == [0, 1]                 # top-p: 0.5 + 0.25 >= 0.7
    assert [i for i, _ in S.kept_set(logits, 1.0, 0, 1.0, 0.4)] == [0, 1]                 # min-p: 0.4 * 0.5 = 0.2
    assert [i for i, _ in S.kept_set(logits, 1.0, 1, 1.0, 0.0)] == [0]                    # top-k of 1 is the argmax
    # a temperature near zero approaches greedy
    assert [i for i, _ in S.kept_set(logits, 0.01, 0, 0.999, 0.0)] == [0]


def test_reference_frequencies():
    # crates/vipera-sampler/src/lib.rs:945-955: 0.75 / 0.25 within 0.05 over 4,000 draws
    logits = np.array([math.log(3.0), 0.0], dtype=np.float32)
    kept = S.kept_set(logits, 1.0, 0, 1.0, 0.0)
    rng = S.Rng(0)
    share = np.mean([S.draw(kept, rng.next_f64()) == 0 for _ in range(4000)])
    assert abs(share - 0.75) < 0.05
