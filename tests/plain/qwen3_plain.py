"""Plain, slow Qwen3 dense decoder: whole sequences, no cache, float64 numpy.

Written from the formulas of the reference runtime (paths relative to the reference
checkout).  One function per part; nothing here is imported by the engine and nothing of
the engine is imported here.  Weights come from a safetensors file through the safetensors
package (the engine has a reader of its own).
"""
from __future__ import annotations

import json
import os

import numpy as np


# ----------------------------------------------------------------------------- parts

def rms_norm(x, weight, eps):
    """y_i = (x_i * s) * w_i with s = 1/sqrt(sum(x^2)/n + eps); the weight multiplies
    directly (no 1+w).  src/minillm/kernels.cpp:209-216."""
    x = np.asarray(x, dtype=np.float64)
    scale = 1.0 / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) / x.shape[-1] + eps)
    return (x * scale) * np.asarray(weight, dtype=np.float64)


def rope_cos_sin(positions, head_dim, base):
    """freq_j = base^(-2j/D), angle = float(pos) * freq_j in 32-bit, j in [0, D/2).
    src/minillm/runtime.cpp:231-241."""
    half = head_dim // 2
    j = np.arange(half, dtype=np.float64)
    freq = np.power(np.float64(base), -2.0 * j / head_dim).astype(np.float32)
    angle = (np.asarray(positions, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float32)
    angle = angle.astype(np.float64)
    return np.cos(angle), np.sin(angle)


def rope_rotate(x, cos, sin):
    """Split-half rotation: pairs are (j, j + D/2); x_j' = x_j c - x_{j+half} s,
    x_{j+half}' = x_j s + x_{j+half} c.  x: [T, H, D]; cos, sin: [T, D/2].
    src/minillm/runtime.cpp:256-266."""
    half = x.shape[-1] // 2
    left, right = x[..., :half], x[..., half:]
    c, s = cos[:, None, :], sin[:, None, :]
    return np.concatenate([left * c - right * s, left * s + right * c], axis=-1)


def causal_attention(q, k, v, positions, scale, window=None):
    """q: [T, Hq, D], k, v: [T, Hkv, D] of ONE sequence whose token t sits at positions[t]
    (ascending, gap-free).  Query head h reads kv head h // (Hq/Hkv): consecutive query
    heads share a kv head.  A query at position p sees the keys at positions <= p (and
    > p - window when a window is given); score = q.k * scale, softmax over the keys,
    out = sum_j a_j v_j.  src/minillm/runtime.cpp:279-313."""
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    group = Hq // Hkv
    pos = np.asarray(positions)
    out = np.zeros((T, Hq, D), dtype=np.float64)
    for h in range(Hq):
        kvh = h // group
        scores = (q[:, h, :] @ k[:, kvh, :].T) * scale          # [T, T]
        visible = pos[None, :] <= pos[:, None]
        if window is not None:
            visible &= pos[None, :] > pos[:, None] - window
        scores = np.where(visible, scores, -np.inf)
        scores = scores - scores.max(axis=-1, keepdims=True)
        e = np.exp(scores)
        a = e / e.sum(axis=-1, keepdims=True)
        out[:, h, :] = a @ v[:, kvh, :]
    return out


def project_qkv(x, w, cfg, positions):
    """q = n Wq^T, k = n Wk^T, v = n Wv^T (no bias); per head RMSNorm over D with q_norm /
    k_norm and the layer's eps, BEFORE the rotation; v is neither normed nor rotated.
    Returns q [T, Hq, D], k and v [T, Hkv, D].  src/minillm/runtime.cpp:250-277."""
    T = x.shape[0]
    Hq, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = (x @ w["q_proj"].T).reshape(T, Hq, D)
    k = (x @ w["k_proj"].T).reshape(T, Hkv, D)
    v = (x @ w["v_proj"].T).reshape(T, Hkv, D)
    q = rms_norm(q, w["q_norm"], cfg["rms_norm_eps"])
    k = rms_norm(k, w["k_norm"], cfg["rms_norm_eps"])
    cos, sin = rope_cos_sin(positions, D, cfg["rope_theta"])
    return rope_rotate(q, cos, sin), rope_rotate(k, cos, sin), v


def attention_block(x, w, cfg, positions, window=None):
    """The mixer of a layer on its already normed input x [T, E]: projections, attention with
    scale 1/sqrt(D), output projection.  src/minillm/runtime.cpp:250-319."""
    T = x.shape[0]
    q, k, v = project_qkv(x, w, cfg, positions)
    o = causal_attention(q, k, v, positions, 1.0 / np.sqrt(cfg["head_dim"]), window)
    return o.reshape(T, -1) @ w["o_proj"].T


def swiglu_mlp(x, w):
    """a = (g / (1 + exp(-g))) * u with g = x Wgate^T, u = x Wup^T; out = a Wdown^T.
    src/minillm/runtime.cpp:323-336."""
    g = x @ w["gate_proj"].T
    u = x @ w["up_proj"].T
    return ((g / (1.0 + np.exp(-g))) * u) @ w["down_proj"].T


def decoder_layer(h, w, cfg, positions, window=None):
    """Pre-norm residual layer: h += attn(norm(h)); h += mlp(norm(h)).
    src/minillm/runtime.cpp:245-337."""
    eps = cfg["rms_norm_eps"]
    h = h + attention_block(rms_norm(h, w["input_layernorm"], eps), w, cfg, positions, window)
    h = h + swiglu_mlp(rms_norm(h, w["post_attention_layernorm"], eps), w)
    return h


def embed(tokens, table):
    """h_t = table[token_t].  src/minillm/runtime.cpp:224-228."""
    return table[np.asarray(tokens, dtype=np.int64)]


def output_logits(h, final_norm, lm_head, eps):
    """logits = RMSNorm(h, model.norm) Wout^T; Wout is lm_head or, tied, the embedding.
    src/minillm/runtime.cpp:338-351."""
    return rms_norm(h, final_norm, eps) @ lm_head.T


# ----------------------------------------------------------------------------- model

_LAYER_NAMES = {
    "input_layernorm": "input_layernorm.weight",
    "post_attention_layernorm": "post_attention_layernorm.weight",
    "q_proj": "self_attn.q_proj.weight",
    "k_proj": "self_attn.k_proj.weight",
    "v_proj": "self_attn.v_proj.weight",
    "o_proj": "self_attn.o_proj.weight",
    "q_norm": "self_attn.q_norm.weight",
    "k_norm": "self_attn.k_norm.weight",
    "gate_proj": "mlp.gate_proj.weight",
    "up_proj": "mlp.up_proj.weight",
    "down_proj": "mlp.down_proj.weight",
}


class PlainQwen3:
    """Tensor names as the reference binds them, under their safetensors names
    (src/minillm/qwen3_model.cpp:57-80)."""

    def __init__(self, folder, round_to=None):
        import torch
        from safetensors.torch import load_file

        with open(os.path.join(folder, "config.json")) as f:
            self.cfg = json.load(f)
        raw = load_file(os.path.join(folder, "model.safetensors"))

        def get(name):
            t = raw[name]
            if round_to == "bfloat16":
                t = t.to(torch.bfloat16)
            return t.to(torch.float64).numpy()

        self.embed = get("model.embed_tokens.weight")
        self.final_norm = get("model.norm.weight")
        self.lm_head = get("lm_head.weight") if "lm_head.weight" in raw else self.embed
        self.layers = []
        for i in range(self.cfg["num_hidden_layers"]):
            self.layers.append({k: get(f"model.layers.{i}.{v}") for k, v in _LAYER_NAMES.items()})

    def hidden(self, tokens, first_position=0):
        positions = np.arange(first_position, first_position + len(tokens))
        h = embed(tokens, self.embed)
        for w in self.layers:
            h = decoder_layer(h, w, self.cfg, positions)
        return h

    def logits(self, tokens, want=None):
        """Logits [len(want), V] of one whole sequence (every position when want is None)."""
        h = self.hidden(tokens)
        if want is not None:
            h = h[np.asarray(want, dtype=np.int64)]
        return output_logits(h, self.final_norm, self.lm_head, self.cfg["rms_norm_eps"])

    def greedy(self, prompt, n):
        """First maximum wins (apps/mini_main.cpp:104-105)."""
        tokens = list(prompt)
        out = []
        for _ in range(n):
            row = self.logits(tokens, [len(tokens) - 1])[0]
            t = int(np.argmax(row))
            out.append(t)
            tokens.append(t)
        return out


# ----------------------------------------------------------------------------- sampling

def greedy_token(row):
    """Largest value, ties -> lowest id (src/minillm/cuda/ops.cu:166-201)."""
    return int(np.argmax(np.asarray(row, dtype=np.float64)))


def temperature_cdf(row, temperature):
    """Cumulative distribution of softmax(row / T) in float64."""
    z = np.asarray(row, dtype=np.float64) / temperature
    e = np.exp(z - z.max())
    return np.cumsum(e / e.sum())


def temperature_token(row, temperature, u):
    """Inverse-CDF draw: the first token whose cumulative probability exceeds u."""
    cdf = temperature_cdf(row, temperature)
    return int(min(np.searchsorted(cdf, u, side="right"), len(cdf) - 1))
