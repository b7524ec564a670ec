"""Pins for the plain implementation beside the reference's text: library routines where a special
case reduces to one, invariants, and vectors chosen so that a plausible mistake (a wrong sign or
pairing, a norm in the wrong place, a wrong head mapping) fails."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from plain import qwen3_plain as P


def rand(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape)


# ------------------------------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("width", [1, 17, 32, 33, 128, 1024])
def test_rms_norm_is_the_library_routine(width):
    x, w = rand((3, width), 1), rand(width, 2)
    want = F.rms_norm(torch.from_numpy(x), (width,), torch.from_numpy(w), eps=1e-5).numpy()
    np.testing.assert_allclose(P.rms_norm(x, w, 1e-5), want, rtol=1e-12, atol=1e-12)


def test_rms_norm_invariants():
    x = rand((4, 64), 3)
    ones = np.ones(64)
    y = P.rms_norm(x, ones, 1e-12)
    np.testing.assert_allclose((y * y).mean(-1), 1.0, rtol=1e-9)              # unit mean square
    np.testing.assert_allclose(P.rms_norm(7.5 * x, ones, 1e-12), y, rtol=1e-9)  # scale of the input drops out
    assert np.all(P.rms_norm(x, np.zeros(64), 1e-6) == 0)                       # the weight multiplies directly (no 1 + w)
    # eps sits inside the root, added to the mean square
    v = np.array([[3.0, 4.0]])
    np.testing.assert_allclose(P.rms_norm(v, np.ones(2), 0.5), v / math.sqrt(12.5 + 0.5))
    # the reference's own vector (tests/core_tests.cpp:316-326), against the formula by hand
    v = np.array([1, -2, 3, -4, 5, 6, -7, 8, 9], dtype=np.float64)
    np.testing.assert_allclose(P.rms_norm(v, np.full(9, 2.0), 1e-6), 2 * v / math.sqrt(285 / 9 + 1e-6))


# ------------------------------------------------------------------------------------------ rotation
def test_rope_table_is_the_reference_formula():
    """Independent evaluation of frequency = base^(-2 i / D), angle = p * frequency in 32-bit
    (tests/cuda_ops_tests.cu:54-65)."""
    D, base = 128, 1000000.0
    cos, sin = P.rope_cos_sin([0, 1, 17, 2047], D, base)
    for row, p in enumerate([0, 1, 17, 2047]):
        for i in [0, 1, 5, 63]:
            freq = np.float32(math.pow(base, -2.0 * i / D))
            angle = float(np.float32(p) * freq)
            assert cos[row, i] == pytest.approx(math.cos(angle), abs=1e-12)
            assert sin[row, i] == pytest.approx(math.sin(angle), abs=1e-12)
    assert np.all(cos[0] == 1) and np.all(sin[0] == 0)


def test_rope_pairs_signs_and_lengths():
    D = 8
    cos, sin = P.rope_cos_sin([1], D, 10000.0)
    # a unit vector on index 0 turns by +1 radian (frequency 1) into index 0 and index D/2: the pair is (j, j + D/2)
    x = np.zeros((1, 1, D))
    x[0, 0, 0] = 1.0
    y = P.rope_rotate(x, cos, sin)[0, 0]
    want = np.zeros(D)
    want[0], want[4] = math.cos(1.0), math.sin(1.0)
    np.testing.assert_allclose(y, want, atol=1e-7)
    # and a unit vector on index D/2 turns into (-sin, cos)
    x[:] = 0
    x[0, 0, 4] = 1.0
    y = P.rope_rotate(x, cos, sin)[0, 0]
    want[0], want[4] = -math.sin(1.0), math.cos(1.0)
    np.testing.assert_allclose(y, want, atol=1e-7)
    # position 0 changes nothing; each (j, j + D/2) pair keeps its length, interleaved pairs (2j, 2j + 1) do not
    x = rand((3, 2, D), 4)
    cos, sin = P.rope_cos_sin([0, 5, 9], D, 10000.0)
    y = P.rope_rotate(x, cos, sin)
    np.testing.assert_array_equal(y[0], x[0])
    np.testing.assert_allclose(y[..., :4] ** 2 + y[..., 4:] ** 2, x[..., :4] ** 2 + x[..., 4:] ** 2, rtol=1e-9)
    assert not np.allclose(y[1:, :, 0::2] ** 2 + y[1:, :, 1::2] ** 2, x[1:, :, 0::2] ** 2 + x[1:, :, 1::2] ** 2)


def test_rope_scores_depend_on_distance_only():
    D = 32
    q, k = rand((1, 1, D), 5), rand((1, 1, D), 6)

    def score(m, n):
        cq, sq = P.rope_cos_sin([m], D, 10000.0)
        ck, sk = P.rope_cos_sin([n], D, 10000.0)
        return float(np.sum(P.rope_rotate(q, cq, sq) * P.rope_rotate(k, ck, sk)))
    assert score(7, 3) == pytest.approx(score(104, 100), abs=1e-4)
    assert score(7, 3) == pytest.approx(score(4, 0), abs=1e-5)
    assert abs(score(7, 3) - score(3, 7)) > 1e-3                         # the sign of the distance counts


# ------------------------------------------------------------------------------------------ attention
def sdpa(q, k, v, causal, scale):
    """Library attention on [T, H, D] arrays with the kv heads repeated (consecutive query heads share)."""
    g = q.shape[1] // k.shape[1]
    tq = torch.from_numpy(q).transpose(0, 1)
    tk = torch.from_numpy(k).repeat_interleave(g, dim=1).transpose(0, 1)
    tv = torch.from_numpy(v).repeat_interleave(g, dim=1).transpose(0, 1)
    return F.scaled_dot_product_attention(tq, tk, tv, is_causal=causal, scale=scale).transpose(0, 1).numpy()


@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (17, 4, 1, 33), (33, 4, 2, 16), (40, 6, 3, 48), (9, 1, 1, 8)])
def test_attention_is_the_library_routine(shape):
    T, hq, hkv, d = shape
    q, k, v = rand((T, hq, d), 7), rand((T, hkv, d), 8), rand((T, hkv, d), 9)
    got = P.causal_attention(q, k, v, np.arange(T), 0.3)
    np.testing.assert_allclose(got, sdpa(q, k, v, True, 0.3), rtol=1e-9, atol=1e-12)
    # without a mask: give every query the last position's view by asking only for the last row
    np.testing.assert_allclose(got[-1], sdpa(q[-1:], k, v, False, 0.3)[0], rtol=1e-9, atol=1e-12)


def test_attention_head_mapping_and_causality():
    T, hq, hkv, d = 6, 4, 2, 8
    q, k, v = rand((T, hq, d), 10), rand((T, hkv, d), 11), rand((T, hkv, d), 12)
    base = P.causal_attention(q, k, v, np.arange(T), 0.5)
    # heads 0, 1 read kv head 0 and heads 2, 3 read kv head 1: changing kv head 1 leaves heads 0, 1 alone
    k2, v2 = k.copy(), v.copy()
    k2[:, 1] += 1.0
    v2[:, 1] -= 2.0
    moved = P.causal_attention(q, k2, v2, np.arange(T), 0.5)
    np.testing.assert_array_equal(moved[:, :2], base[:, :2])
    assert not np.allclose(moved[:, 2:], base[:, 2:])
    # multi-head attention is the special case with the kv heads written out
    np.testing.assert_allclose(P.causal_attention(q, np.repeat(k, 2, axis=1), np.repeat(v, 2, axis=1), np.arange(T), 0.5),
                               base, rtol=1e-12)
    # a later token changes nothing before it; the first token sees itself only
    k2, v2 = k.copy(), v.copy()
    k2[4:], v2[4:] = 9.0, -9.0
    np.testing.assert_array_equal(P.causal_attention(q, k2, v2, np.arange(T), 0.5)[:4], base[:4])
    np.testing.assert_allclose(base[0], np.repeat(v[0], 2, axis=0), rtol=1e-12)
    # rows of the softmax sum to one: with equal values everywhere the output is that value
    np.testing.assert_allclose(P.causal_attention(q, k, np.full_like(v, 2.5), np.arange(T), 0.5), 2.5, rtol=1e-12)


def test_attention_window():
    T, d = 12, 8
    q, k, v = rand((T, 2, d), 13), rand((T, 1, d), 14), rand((T, 1, d), 15)
    got = P.causal_attention(q, k, v, np.arange(T), 0.4, window=5)
    for t in range(T):
        lo = max(0, t - 4)                           # keys t-4 .. t: five of them
        want = sdpa(q[t:t + 1], k[lo:t + 1], v[lo:t + 1], False, 0.4)[0]
        np.testing.assert_allclose(got[t], want, rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(P.causal_attention(q, k, v, np.arange(T), 0.4, window=T),
                               P.causal_attention(q, k, v, np.arange(T), 0.4), rtol=1e-12)


# ------------------------------------------------------------------------------------------ the block
CFG = dict(num_attention_heads=4, num_key_value_heads=2, head_dim=8, rms_norm_eps=1e-6, rope_theta=10000.0,
           hidden_size=12, intermediate_size=20, num_hidden_layers=1, vocab_size=30)


def weights(seed=0):
    r = np.random.default_rng(seed)
    return {"q_proj": r.standard_normal((32, 12)) * 0.4, "k_proj": r.standard_normal((16, 12)) * 0.4,
            "v_proj": r.standard_normal((16, 12)) * 0.4, "o_proj": r.standard_normal((12, 32)) * 0.4,
            "q_norm": 1 + 0.2 * r.standard_normal(8), "k_norm": 1 + 0.2 * r.standard_normal(8),
            "gate_proj": r.standard_normal((20, 12)) * 0.4, "up_proj": r.standard_normal((20, 12)) * 0.4,
            "down_proj": r.standard_normal((12, 20)) * 0.4,
            "input_layernorm": 1 + 0.2 * r.standard_normal(12), "post_attention_layernorm": 1 + 0.2 * r.standard_normal(12)}


def test_the_head_norm_comes_before_the_rotation_and_spares_v():
    w = weights()
    w["q_norm"] = np.array([1, 1, 1, 1, 0, 0, 0, 0], dtype=np.float64)       # wipes the second half of every head
    x = rand((3, 12), 16)
    q, k, v = P.project_qkv(x, w, CFG, np.array([0, 1, 2]))
    assert np.all(q[0, :, 4:] == 0)                                            # position 0: nothing turns
    assert np.all(np.abs(q[1:, :, 4:]) > 0)                                    # norm first, so the rotation refills it
    np.testing.assert_allclose(v.reshape(3, 16), x @ w["v_proj"].T, rtol=1e-12)
    # each normed head has the weight's mean square (times 1): the norm is per head over D, not over the row
    w = weights()
    w["q_norm"][:] = 1.0
    q, _, _ = P.project_qkv(x, w, CFG, np.array([0, 1, 2]))
    np.testing.assert_allclose((q * q).mean(-1), 1.0, rtol=1e-5)


def test_swiglu_is_silu_times_up():
    w = weights()
    x = rand((5, 12), 17)
    g, u = torch.from_numpy(x @ w["gate_proj"].T), torch.from_numpy(x @ w["up_proj"].T)
    want = (F.silu(g) * u).numpy() @ w["down_proj"].T
    np.testing.assert_allclose(P.swiglu_mlp(x, w), want, rtol=1e-10)


def test_layer_is_prenorm_with_two_residuals():
    w = weights()
    h = rand((4, 12), 18)
    pos = np.arange(4)
    mid = h + P.attention_block(P.rms_norm(h, w["input_layernorm"], 1e-6), w, CFG, pos)
    want = mid + P.swiglu_mlp(P.rms_norm(mid, w["post_attention_layernorm"], 1e-6), w)
    np.testing.assert_allclose(P.decoder_layer(h, w, CFG, pos), want, rtol=1e-12)
    # with the output projections at zero the layer is the identity
    w0 = dict(w, o_proj=np.zeros((12, 32)), down_proj=np.zeros((12, 20)))
    np.testing.assert_array_equal(P.decoder_layer(h, w0, CFG, pos), h)


def test_a_shift_of_all_positions_changes_nothing():
    w = weights()
    h = rand((7, 12), 19)
    a = P.decoder_layer(h, w, CFG, np.arange(7))
    b = P.decoder_layer(h, w, CFG, np.arange(7) + 37)
    np.testing.assert_allclose(a, b, atol=2e-5)
    c = P.decoder_layer(h, w, CFG, np.arange(7) * 2)                           # distances do count
    assert np.abs(a - c).max() > 1e-3


# ------------------------------------------------------------------------------------------ the model
def test_whole_model(model_folders, tmp_path):
    import json
    import os
    import shutil
    from safetensors.torch import load_file, save_file
    m = P.PlainQwen3(model_folders["A"])
    tokens = [5, 9, 200, 31, 7, 7, 100]
    full = m.logits(tokens)
    assert full.shape == (7, 256)
    np.testing.assert_allclose(m.logits(tokens, [6, 2]), full[[6, 2]], rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(m.logits(tokens[:4]), full[:4], rtol=1e-9, atol=1e-12)     # causal
    # tied output = untied with a copy of the embedding
    folder = str(tmp_path / "untied")
    shutil.copytree(model_folders["A"], folder)
    t = load_file(os.path.join(folder, "model.safetensors"))
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    save_file(t, os.path.join(folder, "model.safetensors"))
    cfg = json.load(open(os.path.join(folder, "config.json")))
    cfg["tie_word_embeddings"] = False
    json.dump(cfg, open(os.path.join(folder, "config.json"), "w"))
    np.testing.assert_allclose(P.PlainQwen3(folder).logits(tokens), full, rtol=1e-10, atol=1e-12)
    # greedy feeds its own tokens back
    out = m.greedy(tokens[:3], 3)
    assert out[0] == int(np.argmax(m.logits(tokens[:3])[-1]))
    assert out[1] == int(np.argmax(m.logits(tokens[:3] + out[:1])[-1]))


def test_sampling_rules():
    row = np.array([0.1, 2.0, 2.0, -1.0])
    assert P.greedy_token(row) == 1                                            # ties -> lowest id
    cdf = P.temperature_cdf(row, 0.7)
    want = torch.softmax(torch.tensor(row) / 0.7, 0).cumsum(0).numpy()
    np.testing.assert_allclose(cdf, want, rtol=1e-12)
    assert P.temperature_token(row, 0.7, 0.0) == 0
    assert P.temperature_token(row, 0.7, float(cdf[0]) + 1e-9) == 1
    assert P.temperature_token(row, 0.7, 0.999999) == 3
    assert P.temperature_token(row, 1e-3, 0.3) == 1                            # T -> 0 is greedy
