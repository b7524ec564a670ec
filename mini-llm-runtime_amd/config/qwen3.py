"""Qwen3 dense decoder: config.json keys, checks and tensor names.

The checks follow the reference's `load_dimensions` (src/minillm/qwen3_model.cpp:9-40):
sizes in 1..1e6, q heads a multiple of kv heads, an even head size taken from its own key
(never hidden/heads unless the key is absent), finite positive eps and rope base, no rope
scaling.  The reference has no biases and attends to all earlier keys, so a configuration
that asks for attention biases or a sliding window is refused.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Tuple

from .registry import ConfigError, register_architecture
from .specs import (AttentionSpec, LayerRun, LayerSpec, MlpSpec, ModelSpec, NormSpec,
                    PositionSpec)

_LIMIT = 1_000_000


def _integer(data, key, default=None):
    value = data.get(key, default)
    if isinstance(value, bool) or not isinstance(value, int):
        raise ConfigError(f"config.json: `{key}` must be an integer, got {value!r}")
    if value < 1 or value > _LIMIT:
        raise ConfigError(f"config.json: `{key}` = {value} is outside 1..{_LIMIT}")
    return value


def _positive_float(data, key):
    value = data.get(key)
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config.json: `{key}` must be a number, got {value!r}")
    value = float(value)
    if not math.isfinite(value) or value <= 0:
        raise ConfigError(f"config.json: `{key}` = {value} must be finite and positive")
    return value


@register_architecture("Qwen3ForCausalLM")
@dataclass(frozen=True)
class Qwen3Config:
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    eos_token_ids: Tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, data):
        for key in ("hidden_size", "num_hidden_layers", "num_attention_heads",
                    "intermediate_size", "vocab_size", "max_position_embeddings",
                    "rms_norm_eps", "rope_theta"):
            if key not in data:
                raise ConfigError(f"config.json: missing `{key}`")
        heads = _integer(data, "num_attention_heads")
        kv_heads = _integer(data, "num_key_value_heads", heads)
        hidden = _integer(data, "hidden_size")
        if "head_dim" in data and data["head_dim"] is not None:
            head_dim = _integer(data, "head_dim")
        elif hidden % heads == 0:
            head_dim = hidden // heads
        else:
            raise ConfigError("config.json: no `head_dim` and hidden_size is no multiple of the heads")
        if heads % kv_heads != 0:
            raise ConfigError(f"config.json: num_attention_heads {heads} is no multiple of "
                              f"num_key_value_heads {kv_heads}")
        if head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim {head_dim} must be even for the rotation")
        scaling = data.get("rope_scaling")
        if scaling is not None and not (isinstance(scaling, dict) and
                                        scaling.get("rope_type", scaling.get("type")) in
                                        (None, "none", "default")):
            raise ConfigError("config.json: rope_scaling is not supported")
        for key in ("attention_bias", "use_sliding_window"):
            if data.get(key) is not None and not isinstance(data[key], bool):
                raise ConfigError(f"config.json: `{key}` must be true or false")
        if data.get("attention_bias"):
            raise ConfigError("config.json: attention_bias is not supported (Qwen3 dense has no biases)")
        if data.get("use_sliding_window"):
            raise ConfigError("config.json: use_sliding_window is not supported (full causal attention)")
        # (a list that names the kind of attention of every layer: anything but full attention everywhere would
        # be computed wrongly here, so it is refused rather than passed over)
        kinds = data.get("layer_types")
        if kinds is not None:
            layers = _integer(data, "num_hidden_layers")
            if not isinstance(kinds, list) or len(kinds) != layers or any(not isinstance(k, str) for k in kinds):
                raise ConfigError("config.json: `layer_types` must name the attention of each of the "
                                  f"{layers} layers")
            if any(k != "full_attention" for k in kinds):
                raise ConfigError("config.json: layer_types other than full_attention are not supported")
        if data.get("model_type") is not None and data["model_type"] != "qwen3":
            raise ConfigError(f"config.json: model_type {data['model_type']!r} does not go with {cls.architecture}")
        act = data.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act {act!r} is not supported (silu)")
        tie = data.get("tie_word_embeddings", False)
        if not isinstance(tie, bool):
            raise ConfigError("config.json: `tie_word_embeddings` must be true or false")
        eos = data.get("eos_token_id")
        if eos is None:
            eos_ids = ()
        elif isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, list) and all(isinstance(e, int) and not isinstance(e, bool) for e in eos):
            eos_ids = tuple(eos)
        else:
            raise ConfigError("config.json: `eos_token_id` must be an integer or a list of integers")
        vocab = _integer(data, "vocab_size")
        for e in eos_ids:
            if e < 0 or e >= vocab:
                raise ConfigError(f"config.json: eos_token_id {e} is outside the vocabulary")
        return cls(
            hidden_size=hidden,
            num_hidden_layers=_integer(data, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=_integer(data, "intermediate_size"),
            vocab_size=vocab,
            max_position_embeddings=_integer(data, "max_position_embeddings"),
            rms_norm_eps=_positive_float(data, "rms_norm_eps"),
            rope_theta=_positive_float(data, "rope_theta"),
            tie_word_embeddings=tie,
            eos_token_ids=eos_ids,
        )

    def to_dict(self):
        out = {
            "architectures": [self.architecture],
            "model_type": "qwen3",
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
            "use_sliding_window": False,
        }
        if self.eos_token_ids:
            out["eos_token_id"] = (self.eos_token_ids[0] if len(self.eos_token_ids) == 1
                                   else list(self.eos_token_ids))
        return out

    # ---- the model as parts -------------------------------------------------------------
    def model_spec(self):
        norm = NormSpec("rmsnorm", self.hidden_size, self.rms_norm_eps)
        head_norm = NormSpec("rmsnorm", self.head_dim, self.rms_norm_eps)
        mixer = AttentionSpec(
            kind="gqa_attention", hidden=self.hidden_size, q_heads=self.num_attention_heads,
            kv_heads=self.num_key_value_heads, head_dim=self.head_dim,
            scale=1.0 / math.sqrt(self.head_dim), qk_norm=head_norm,
            position=PositionSpec("rope_split_half", self.head_dim, self.rope_theta), window=None)
        ffn = MlpSpec("swiglu", self.hidden_size, self.intermediate_size, "silu")
        layer = LayerSpec("prenorm", norm, mixer, norm, ffn)
        n = self.num_hidden_layers
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden=self.hidden_size,
            layers=tuple(layer for _ in range(n)),
            schedule=tuple(LayerRun(i, i) for i in range(n)),
            final_norm=norm, tie_embeddings=self.tie_word_embeddings,
            max_positions=self.max_position_embeddings, eos_token_ids=self.eos_token_ids)

    # ---- tensor names (src/minillm/qwen3_model.cpp:59-78, under their safetensors names) --
    @staticmethod
    def global_tensor_name(local):
        return {"embed.weight": "model.embed_tokens.weight", "final_norm.weight": "model.norm.weight",
                "head.weight": "lm_head.weight"}[local]

    @staticmethod
    def layer_tensor_name(layer, part, local):
        table = {
            ("norm1", "weight"): "input_layernorm.weight",
            ("norm2", "weight"): "post_attention_layernorm.weight",
            ("mixer", "q_proj"): "self_attn.q_proj.weight",
            ("mixer", "k_proj"): "self_attn.k_proj.weight",
            ("mixer", "v_proj"): "self_attn.v_proj.weight",
            ("mixer", "o_proj"): "self_attn.o_proj.weight",
            ("mixer", "q_norm.weight"): "self_attn.q_norm.weight",
            ("mixer", "k_norm.weight"): "self_attn.k_norm.weight",
            ("ffn", "gate_proj"): "mlp.gate_proj.weight",
            ("ffn", "up_proj"): "mlp.up_proj.weight",
            ("ffn", "down_proj"): "mlp.down_proj.weight",
        }
        return f"model.layers.{layer}.{table[(part, local)]}"
